"""The LDS layout of the prefill-chunk map, checked on the host.  A tile holds 32 keys at head_dim 256 and 64 at
head_dim 128 (16 KiB either way).  A K tile is [keys][head_dim] elements with the 16-byte chunk index XORed with
key % 16; a V tile is [keys][head_dim] f16 with the 32-byte chunk index XORed with key % 8.  The operand reads must put the lanes that an LDS read serves together on different bank groups and must
find what the fetching waves put there: K arrives by loads that write 1 KiB in lane order (the layout is made by each
lane's choice of global address), V by 128-bit stores.  The address arithmetic below restates
psi-dec_amd/csrc/split_kv_chunk_kernel.h (k_row0, v_row0, v_swizzle, k_lane, v_lane); the lane groups of a 128-bit
access are the ones measured on MI355X: lanes 0-3, 12-15 and 20-27 go together, then 4-11, 16-19 and 28-31, and the
same in the upper half of the wave."""
import pytest

READ_ROUNDS = [
    [0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27],
    [4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31],
]
READ_ROUNDS += [[lane + 32 for lane in group] for group in READ_ROUNDS[:2]]
WAVES = 8


def keys_of(d):
    return 64 if d == 128 else 32


def wave_rows(d):
    return keys_of(d) // WAVES


def bank_group(byte_offset):
    """16-byte group among the 64 four-byte banks."""
    return (byte_offset % 256) // 16


def k_read_offset(d, lane, ks, block):
    """128-bit read of the A operand of K * Q^T: key 16 * block + mt, elements 32 * ks + 8 * mc .. + 7."""
    mt, mc = lane & 15, lane >> 4
    return mt * d * 2 + (((4 * ks + mc) ^ mt) * 16) + block * 16 * d * 2


def v_read_offset(d, lane, db, block):
    """64-bit transposing read: the lane hands in key 16 * block + 4 * mc + mt / 4, dims 16 * db + 4 * (mt % 4) .. + 3."""
    mt, mc = lane & 15, lane >> 4
    key = 4 * mc + (mt >> 2)
    return key * d * 2 + (mt & 3) * 8 + ((db * 32) ^ ((key & 7) * 32)) + block * 16 * d * 2


def fetch_geometry(d):
    row_chunks = d // 8                 # 16-byte chunks per row
    rows_per_load = 64 // row_chunks    # rows that one load of a wave covers
    return row_chunks, rows_per_load, wave_rows(d) // rows_per_load


def k_landing(d, wave, lane, i):
    """Load i of a wave: (LDS offset in the tile where the lane's 16 bytes land, key, 16-byte chunk they come from)."""
    row_chunks, rows_per_load, _ = fetch_geometry(d)
    row_in_load, slot = lane // row_chunks, lane % row_chunks
    key = wave_rows(d) * wave + rows_per_load * i + row_in_load
    lands = (wave_rows(d) * wave + rows_per_load * i) * d * 2 + lane * 16
    return lands, key, slot ^ (key & 15)


def v_store(d, wave, lane, i):
    """Store i of a wave: (LDS offset in the tile, key, 16-byte chunk of the row that the lane holds)."""
    row_chunks, rows_per_load, _ = fetch_geometry(d)
    row_in_load, slot = lane // row_chunks, lane % row_chunks
    key = wave_rows(d) * wave + rows_per_load * i + row_in_load
    where = key * d * 2 + ((((slot >> 1) ^ (key & 7)) << 1) | (slot & 1)) * 16
    return where, key, slot


def test_rounds_partition_the_wave():
    assert sorted(lane for group in READ_ROUNDS for lane in group) == list(range(64))


@pytest.mark.parametrize("d", [128, 256])
def test_k_operand_reads_are_conflict_free_and_find_what_landed(d):
    loads = fetch_geometry(d)[2]
    where = {}
    for wave in range(WAVES):
        for i in range(loads):
            for lane in range(64):
                lands, key, chunk = k_landing(d, wave, lane, i)
                assert lands // (d * 2) == key, "a lane's bytes land in the row of their key"
                where[(key, chunk)] = lands
    assert len(where) == keys_of(d) * d // 8 and len(set(where.values())) == len(where)
    for block in range(keys_of(d) // 16):
        for ks in range(d // 32):
            for group in READ_ROUNDS:
                assert len({bank_group(k_read_offset(d, lane, ks, block)) for lane in group}) == 16
            for lane in range(64):
                mt, mc = lane & 15, lane >> 4
                # key 16 * block + mt, elements 32 * ks + 8 * mc .. + 7 = chunk 4 * ks + mc
                assert k_read_offset(d, lane, ks, block) == where[(16 * block + mt, 4 * ks + mc)]


@pytest.mark.parametrize("d", [128, 256])
def test_transposing_reads_spread_their_keys_over_the_banks_and_find_what_was_stored(d):
    """The 16 lanes of a quarter wave read 4 keys x 32 bytes, two quarters 8 keys: every key's 32 bytes in a bank
    group pair of its own."""
    loads = fetch_geometry(d)[2]
    where = {}
    for wave in range(WAVES):
        for i in range(loads):
            for lane in range(64):
                at, key, chunk = v_store(d, wave, lane, i)
                assert at // (d * 2) == key
                where[(key, chunk)] = at
    assert len(where) == keys_of(d) * d // 8 and len(set(where.values())) == len(where)
    for block in range(keys_of(d) // 16):
        for db in range(d // 16):
            for half in range(2):
                pairs = set()
                for lane in range(32 * half, 32 * half + 32):
                    off = v_read_offset(d, lane, db, block)
                    assert off % 8 == 0
                    mt, mc = lane & 15, lane >> 4
                    key = 16 * block + 4 * mc + (mt >> 2)
                    first_dim = 16 * db + 4 * (mt & 3)  # 4 dims = 8 bytes inside chunk first_dim / 8
                    assert off == where[(key, first_dim // 8)] + (first_dim % 8) * 2
                    pairs.add((off % 256) // 32)
                assert len(pairs) == 8  # eight keys, eight different 32-byte bank ranges


@pytest.mark.parametrize("d", [128, 256])
def test_v_stores_are_conflict_free(d):
    """A 128-bit store is served in the same rounds of 16 lanes."""
    loads = fetch_geometry(d)[2]
    for wave in range(WAVES):
        for i in range(loads):
            for group in READ_ROUNDS:
                assert len({bank_group(v_store(d, wave, lane, i)[0]) for lane in group}) == 16
