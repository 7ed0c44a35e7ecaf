"""The LDS layout of the prefill-chunk map, checked on the host: the K tile in rows of head_dim * 2 bytes with the
16-byte chunk index XORed with key % 16, the V tile in rows of head_dim * 2 + 32 bytes.  The operand reads must put
the 16 lanes that a 128-bit LDS read serves together on 16 different bank groups, must find what the loading
waves stored, and the stores must fill whole rows.  The address arithmetic below restates psi-dec_amd/csrc/split_kv_chunk_kernel.h (
k_row0, vt_base, k_store, v_store); the lane groups are the ones measured on MI355X: lanes 0-3, 12-15 and 20-27 go together, then 4-11,
16-19 and 28-31, and the same in the upper half of the wave."""
import pytest

READ_ROUNDS = [
    [0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27],
    [4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31],
]
READ_ROUNDS += [[lane + 32 for lane in group] for group in READ_ROUNDS[:2]]
KEYS = 32


def pitch(d):
    return d * 2 + 32


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
    return (4 * mc + (mt >> 2)) * pitch(d) + (mt & 3) * 8 + db * 32 + block * 16 * pitch(d)


def loader_key_chunk(d, thread, i):
    chunks = d // 8
    return thread // chunks + (256 // chunks) * i, thread % chunks


def k_store_offset(d, thread, i):
    """128-bit store of loading thread `thread` (0 .. 255), load i, into the K tile."""
    key, chunk = loader_key_chunk(d, thread, i)
    return key * d * 2 + ((chunk ^ (key & 15)) * 16)


def v_store_offset(d, thread, i):
    key, chunk = loader_key_chunk(d, thread, i)
    return key * pitch(d) + chunk * 16


def test_rounds_partition_the_wave():
    assert sorted(lane for group in READ_ROUNDS for lane in group) == list(range(64))


@pytest.mark.parametrize("d", [128, 256])
def test_k_operand_reads_are_conflict_free_and_find_what_was_stored(d):
    loads = KEYS * (d // 8) // 256
    where = {}
    for thread in range(256):
        for i in range(loads):
            where[loader_key_chunk(d, thread, i)] = k_store_offset(d, thread, i)
    assert len(where) == KEYS * d // 8 and len(set(where.values())) == len(where)
    for block in range(2):
        for ks in range(d // 32):
            for group in READ_ROUNDS:
                assert len({bank_group(k_read_offset(d, lane, ks, block)) for lane in group}) == 16
            for lane in range(64):
                mt, mc = lane & 15, lane >> 4
                # key 16 * block + mt, elements 32 * ks + 8 * mc .. + 7 = chunk 4 * ks + mc
                assert k_read_offset(d, lane, ks, block) == where[(16 * block + mt, 4 * ks + mc)]


@pytest.mark.parametrize("d", [128, 256])
def test_transposing_reads_spread_their_keys_over_the_banks(d):
    """The 16 lanes of a quarter wave read 4 keys x 32 bytes, two quarters 8 keys: every key's 32 bytes in a bank
    group pair of its own."""
    for block in range(2):
        for db in range(d // 16):
            for half in range(2):
                pairs = set()
                for lane in range(32 * half, 32 * half + 32):
                    off = v_read_offset(d, lane, db, block)
                    assert off % 8 == 0
                    mt, mc = lane & 15, lane >> 4
                    assert off == (16 * block + 4 * mc + (mt >> 2)) * pitch(d) + (16 * db + 4 * (mt & 3)) * 2
                    pairs.add((off % 256) // 32)
                assert len(pairs) == 8  # eight keys, eight different 32-byte bank ranges


@pytest.mark.parametrize("d", [128, 256])
def test_stores_fill_the_tiles_in_whole_rows(d):
    loads = KEYS * (d // 8) // 256
    covered = set()
    for thread in range(256):
        for i in range(loads):
            key, byte = divmod(v_store_offset(d, thread, i), pitch(d))
            assert key < KEYS and byte < d * 2 and byte % 16 == 0
            covered.add((key, byte))
            assert k_store_offset(d, thread, i) // (d * 2) == key  # the K store stays in its row
    assert len(covered) == KEYS * d // 8


def test_stores_of_head_dim_256_are_conflict_free():
    """A 128-bit store is served in the same rounds of 16 lanes; with 512-byte rows every round stays inside one row,
    where the XOR only permutes the chunks."""
    for wave in range(4):
        for i in range(4):
            for group in READ_ROUNDS:
                assert len({bank_group(k_store_offset(256, 64 * wave + lane, i)) for lane in group}) == 16
                assert len({bank_group(v_store_offset(256, 64 * wave + lane, i)) for lane in group}) == 16
