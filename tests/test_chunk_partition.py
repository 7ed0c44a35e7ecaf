"""The partition planner for prefill chunks (psi_hip_split_kv_chunk_partition_tokens; no counterpart in the
reference, which has no fixed partitions): the library through its C ABI against a restatement of its model in a
dozen lines, on the shapes whose launches were timed on MI355X and on random batches, and the properties a caller
relies on.  The timings quoted are of the row-group map alone, 24 Q / 4 KV heads of 256, one MI355X."""
import heapq
import random

import pytest


def config(psi, hq, hkv, d, page_tokens, dtype=None):
    dtype = psi.Dtype.Bfloat16 if dtype is None else dtype
    return psi.GQASplitKVConfig(io_dtype=dtype, page_bytes=2 * hkv * d * page_tokens * dtype.item_size(),
                                num_q_heads=hq, num_kv_heads=hkv, head_dim=d)


def model(reqs, hq, hkv, d, ts, partition, units=256):
    """Items = (token group, partition) x KV heads x head subsets, cost = KV tiles + 9; units take the heaviest item
    left as they become free; plus what the items' partial rows cost."""
    group = hq // hkv
    subsets = 3 if group == 6 else (2 if group > 5 else 1)
    heads = (group + subsets - 1) // subsets
    group_tiles = min(256 // (heads * ts), 32)
    # chunks that short that their tokens times all the heads of a KV head fit one workgroup: no head subsets
    all_heads_tiles = 256 // (group * ts)
    widest = max(min(max((chunk + ts - 1) // ts for _, chunk in reqs), group_tiles), 1)
    if widest <= all_heads_tiles:
        subsets, group_tiles = 1, max(min(all_heads_tiles, group_tiles), 1)
    group_tokens = group_tiles * ts
    tile_keys = 64 if d == 128 else 32
    costs = []
    for prefix, chunk in reqs:
        for a in range(0, chunk, group_tokens):
            kv_end = prefix + min(a + group_tokens, chunk)
            for lo in range(0, kv_end, partition):
                costs.append((min(lo + partition, kv_end) - lo + tile_keys - 1) // tile_keys + 9.0)
    costs.sort(reverse=True)
    copies = hkv * subsets
    items = len(costs) * copies
    if items > 8 * units:
        end = max(sum(costs) * copies / units + 0.5 * costs[-1], costs[0])
    else:
        free = [0.0] * units
        end = 0.0
        for c in costs:
            for _ in range(copies):
                t = heapq.heappop(free) + c
                end = max(end, t)
                heapq.heappush(free, t)
    return end + 0.06 * d / 256.0 * items


def candidates(longest):
    unsplit = min((longest + 255) // 256 * 256, 1 << 20)
    out, p = [], 256
    while p < unsplit and p <= 32768:
        out.append(p)
        p += 256 if p < 2048 else (1024 if p < 8192 else 2048)
    return out + [unsplit]


def planned(reqs, hq, hkv, d, ts, units=256):
    longest = max(prefix + chunk for prefix, chunk in reqs)
    best, answer = None, 0
    for p in candidates(longest):
        if p * 64 < longest and p != candidates(longest)[-1]:
            continue
        cost = model(reqs, hq, hkv, d, ts, p, units)
        if best is None or cost <= best:
            best, answer = cost, p
    return answer


def ask(psi, cfg, ts, reqs, units=0):
    cu = [0]
    for _, chunk in reqs:
        cu.append(cu[-1] + chunk)
    return psi.chunk_partition_tokens(cfg, ts, [prefix for prefix, _ in reqs], cu, units)


@pytest.mark.parametrize("prefix,chunk,expected", [
    (4096, 2048, 4096),    # the measured workload: 238 us; 2048 -> 260, 3072 -> 291, 5120 -> 274
    (4096, 512, 1024),     # 73 us against 220 us with 4096-token partitions (96 items for 256 units)
    (4096, 1024, 2048),    # 124 us against 221 us (4096) and 144 us (1024)
    (0, 2048, 1024),       # 72 us against 119 us (4096) and 90 us (512)
    (8192, 2048, 7168),    # 400 us against 459 us (4096)
    (16384, 2048, 14336),  # 729 us with 13312 against 798 us (4096)
])
def test_the_timed_shapes(psi, prefix, chunk, expected):
    cfg = config(psi, 24, 4, 256, 16)
    assert ask(psi, cfg, 8, [(prefix, chunk)]) == expected == planned([(prefix, chunk)], 24, 4, 256, 8)


def test_library_and_restatement_agree_on_random_batches(psi):
    rng = random.Random(11)
    for _ in range(60):
        hkv = rng.choice([1, 2, 4, 8])
        group = rng.choice([1, 2, 4, 5, 6, 7, 8])
        d = rng.choice([128, 256])
        cfg = config(psi, hkv * group, hkv, d, rng.choice([8, 16, 32]))
        reqs = [(rng.choice([0, 1, 17, 500, 4096, 9000, 20000, 300000]), rng.choice([1, 8, 100, 512, 2048, 5000]))
                for _ in range(rng.randint(1, 4))]
        units = rng.choice([0, 64, 256, 304])
        got = ask(psi, cfg, 8, reqs, units)
        assert got == planned(reqs, hkv * group, hkv, d, 8, units or 256), (reqs, hkv, group, d, units)
        assert got % 256 == 0 and 256 <= got <= (max(p + c for p, c in reqs) + 255) // 256 * 256


def test_geometries_without_a_row_group_kernel_and_empty_batches(psi):
    assert ask(psi, config(psi, 8, 2, 64, 16), 8, [(4096, 2048)]) == 0              # head_dim 64
    assert ask(psi, config(psi, 8, 2, 256, 16, psi.Dtype.Float32), 8, [(4096, 2048)]) == 0  # f32 storage
    assert psi.chunk_partition_tokens(config(psi, 24, 4, 256, 16), 8, [], [0]) == 0


def test_fewer_units_want_fewer_longer_items(psi):
    cfg = config(psi, 24, 4, 256, 16)
    assert ask(psi, cfg, 8, [(4096, 512)], 32) >= ask(psi, cfg, 8, [(4096, 512)], 256)


def test_a_decreasing_prefix_sum_is_refused(psi):
    with pytest.raises(Exception, match="cu_tokens must not decrease"):
        psi.chunk_partition_tokens(config(psi, 24, 4, 256, 16), 8, [4096, 100], [0, 2048, 1000])


def test_contexts_beyond_64_of_the_longest_candidate_stay_unsplit_at_worst(psi):
    """The planner never answers 0 for a geometry it serves: the unsplit candidate always stands."""
    got = ask(psi, config(psi, 24, 4, 256, 16), 8, [(3_000_000, 64)])
    assert got % 256 == 0 and got >= 32768
