"""The LDS layouts of the prefill-chunk map, checked on the host: the operand reads must put the 16
lanes that a 128-bit LDS read serves together on 16 different bank groups, and the stores must not
collide either.  The address arithmetic below restates psi-dec_amd/csrc/split_kv_chunk_kernel.h
(k_row0 / k_swz, vt_row0, k_store0 / k_store1 and the transposing store of store_tile); the lane
groups are the ones measured on MI355X: lanes 0-3, 12-15 and 20-27 go together, then 4-11, 16-19 and
28-31, and the same in the upper half of the wave."""
D = 256
ROW = D * 2  # bytes per K row

READ_ROUNDS = [
    [0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27],
    [4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31],
]
READ_ROUNDS += [[lane + 32 for lane in group] for group in READ_ROUNDS[:2]]


def bank_group(byte_offset):
    """16-byte group among the 64 four-byte banks."""
    return (byte_offset % 256) // 16


def k_read_offset(lane, ks, block):
    mt, mc = lane & 15, lane >> 4
    row = 8 * (mt >> 2) + (mt & 3) + 4 * block
    return row * ROW + (((4 * ks + mc) ^ mt) * 16)


def vt_read_offset(lane, db):
    mt, mc = lane & 15, lane >> 4
    return mt * 64 + (mt >> 3) * 64 + (((mc + 2 * (mt >> 2)) & 3) * 16) + db * (16 * 64 + 2 * 64)


def vt_slot_offset(row, key):
    """Byte offset of element (dim row, key) of the transposed V tile, as the stores place it."""
    octet, within = key // 8, key % 8
    slot = (octet + 2 * ((row % 8) // 4)) & 3
    return row * 64 + (row // 8) * 64 + slot * 16 + within * 2


def test_rounds_partition_the_wave():
    assert sorted(lane for group in READ_ROUNDS for lane in group) == list(range(64))


def test_k_operand_reads_are_conflict_free():
    for ks in range(D // 32):
        for block in range(2):
            for group in READ_ROUNDS:
                assert len({bank_group(k_read_offset(lane, ks, block)) for lane in group}) == 16


def test_vt_operand_reads_are_conflict_free():
    for db in range(D // 16):
        for group in READ_ROUNDS:
            assert len({bank_group(vt_read_offset(lane, db)) for lane in group}) == 16


def test_vt_reads_find_what_the_stores_wrote():
    """Lane (mt, mc) of dim block db reads keys 8 * mc .. + 7 of dim 16 * db + mt."""
    for db in range(D // 16):
        for lane in range(64):
            mt, mc = lane & 15, lane >> 4
            assert vt_read_offset(lane, db) == vt_slot_offset(16 * db + mt, 8 * mc)


def test_xor_slots_would_collide():
    """The layout this one replaced - slot XOR (row / 4) % 4 - is conflict-free over plain quarters
    of the wave and two-way conflicted over the real rounds."""
    def old(lane):
        mt, mc = lane & 15, lane >> 4
        return mt * 64 + (mt >> 3) * 64 + ((mc ^ ((mt >> 2) & 3)) * 16)
    for quarter in range(4):
        assert len({bank_group(old(lane)) for lane in range(16 * quarter, 16 * quarter + 16)}) == 16
    assert all(len({bank_group(old(lane)) for lane in group}) == 8 for group in READ_ROUNDS)


def test_transposing_stores_cover_distinct_banks():
    """One 32-bit store instruction of a wave: 16 key pairs x 4 dim chunks, row 8 * chunk + e."""
    for wave in range(8):
        for e in range(8):
            banks = set()
            for lane in range(64):
                tid = 64 * wave + lane
                v_pair, v_chunk = tid % 16, tid // 16
                offset = vt_slot_offset(8 * v_chunk + e, 2 * v_pair)
                assert offset % 4 == 0
                banks.add((offset % 256) // 4)
            assert len(banks) == 64


def test_k_stores_keep_rows_whole():
    """A 128-bit K store places chunk c of key row r at chunk c ^ (r % 4 + 4 * (r / 8)): a permutation
    of the row that the operand read undoes."""
    for row in range(32):
        swizzle = (row & 3) + 4 * (row >> 3)
        assert sorted(chunk ^ swizzle for chunk in range(32)) == list(range(32))
    for lane in range(64):
        mt, mc = lane & 15, lane >> 4
        for ks in range(D // 32):
            for block in range(2):
                row = 8 * (mt >> 2) + (mt & 3) + 4 * block
                stored_chunk = ((k_read_offset(lane, ks, block) - row * ROW) // 16) ^ ((row & 3) + 4 * (row >> 3))
                assert stored_chunk == 4 * ks + mc  # dims 32 * ks + 8 * mc .. + 7
