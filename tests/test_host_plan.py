"""Host-side planning (capacity buckets, variant selection, KV-split plans, page-table index math):
the library through its C ABI and the Python oracle, both against the vectors the reference's own
tests hold, then against each other on random batches.

  buckets            crates/inference-executor-core/src/replay.rs:94-180
  selector matrix    crates/inference-backend-metal/src/components/gqa_split_kv.rs:177-231
  measured selector  crates/inference-executor-metal/src/attn/gqa/mod.rs:370-454
  split plans        crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:535-680
  page table         crates/inference-executor-metal/src/attn/gqa/request_page_table.rs:112-117,141-174
  layer split        crates/inference-executor-metal/src/model/qwen/v3_x/state/gqa.rs:250-277
"""
import ctypes
import random

import numpy as np
import pytest

MAX = 0xFFFFFFFF


def bf16_config(psi, head_dim, group, tokens_per_page, num_kv_heads=2, dtype=None):
    dtype = psi.Dtype.Bfloat16 if dtype is None else dtype
    return psi.GQASplitKVConfig(
        io_dtype=dtype, page_bytes=2 * num_kv_heads * head_dim * tokens_per_page * dtype.item_size(),
        num_q_heads=num_kv_heads * group, num_kv_heads=num_kv_heads, head_dim=head_dim)


def as_tuple(v):
    if v.is_tiled():
        return ("TiledQ", v.q_token_tile_size, v.kv_token_tile_size, v.q_head_tile_size)
    return ("SingleQ", v.kv_token_tile_size, v.num_threads_per_threadblock, v.q_head_tile_size)


def from_tuple(psi, t):
    if t[0] == "TiledQ":
        return psi.GQASplitKVVariant.TiledQ(t[1], t[2], t[3])
    return psi.GQASplitKVVariant.SingleQ(t[1], t[2], t[3])


# ------------------------------------------------------------------ buckets


@pytest.fixture(params=["oracle", "library"])
def bucket_policy(request, host_oracle, psi):
    if request.param == "oracle":
        def make(cap, boundaries=()):
            p = host_oracle.ReplayBucketPolicy(cap, boundaries)
            return p.buckets, p.capacity
    else:
        def make(cap, boundaries=()):
            p = psi.ReplayBucketPolicy(cap, boundaries)
            return p.buckets(), p.capacity
    return make


def test_default_buckets(bucket_policy):
    base = [1, 2, 4, 6, 8, 12, 16, 20, 24, 32, 40, 48, 56, 64]
    assert bucket_policy(64)[0] == base
    assert bucket_policy(128)[0] == base + [80, 96, 112, 128]
    assert bucket_policy(70)[0][-1] == 70
    assert bucket_policy(6)[0] == [1, 2, 4, 6]


@pytest.mark.parametrize("cap", [65, 79, 80, 81, 127, 128, 129, MAX])
def test_buckets_ordered_at_extension_boundaries(bucket_policy, cap):
    buckets, capacity = bucket_policy(cap)
    assert buckets[-1] == cap and capacity(cap) == cap
    assert all(a < b for a, b in zip(buckets, buckets[1:]))


def test_bucket_capacity(bucket_policy):
    _, capacity = bucket_policy(64)
    assert [capacity(a) for a in (1, 3, 5, 9, 25, 64)] == [1, 4, 6, 12, 32, 64]


def test_topology_boundaries(bucket_policy):
    buckets, capacity = bucket_policy(64, [5, 6, 10, 12, 18])
    assert 0 not in buckets
    assert [capacity(a) for a in (5, 9, 10, 11, 17, 18)] == [5, 9, 11, 11, 17, 20]
    assert bucket_policy(6, [1])[0] == [1, 2, 4, 6]
    buckets, capacity = bucket_policy(8, [6])
    assert buckets == [1, 2, 4, 5, 6, 8]
    assert [capacity(a) for a in (5, 6, 7)] == [5, 6, 8]


def test_padding_stays_within_a_quarter(bucket_policy):
    _, capacity = bucket_policy(256)
    for active in range(1, 257):
        total = capacity(active)
        assert (total - active) * 4 <= total, (active, total)


def test_capacity_rejects_overflow_and_zero(psi, host_oracle):
    with pytest.raises(psi.PsiHipError, match="replay active work exceeds capacity"):
        psi.ReplayBucketPolicy(6).capacity(7)
    with pytest.raises(psi.PsiHipError, match="replay bucket requires active work"):
        psi.ReplayBucketPolicy(6).capacity(0)
    assert psi.ReplayBucketPolicy(6).capacity_allow_zero(0) == 0
    with pytest.raises(AssertionError):
        host_oracle.ReplayBucketPolicy(6).capacity(7)


def test_buckets_agree_for_every_capacity_up_to_600(psi, host_oracle):
    for cap in range(1, 600):
        assert psi.ReplayBucketPolicy(cap).buckets() == host_oracle.ReplayBucketPolicy(cap).buckets, cap


# ------------------------------------------------------------------ selector


def test_selector_matrix_library(psi):
    t256 = psi.GQASplitKV.new(bf16_config(psi, 256, 6, 16))
    t256p8 = psi.GQASplitKV.new(bf16_config(psi, 256, 6, 8))
    t128 = psi.GQASplitKV.new(bf16_config(psi, 128, 8, 8))
    unsupported = psi.GQASplitKV.new(bf16_config(psi, 256, 8, 4))
    single_partial = psi.GQASplitKV.new_dspark_history(bf16_config(psi, 128, 8, 8))
    assert t256.max_q_tokens_per_partial_output() == 8
    assert t256p8.max_q_tokens_per_partial_output() == 8
    assert as_tuple(t256.select(4, 4)) == ("SingleQ", 256, 256, 6)
    assert as_tuple(t256.select(8, 4)) == ("TiledQ", 8, 16, 3)
    assert as_tuple(t256.select(16, 4)) == ("TiledQ", 8, 16, 6)
    assert as_tuple(t256p8.select(16, 4)) == ("TiledQ", 8, 16, 6)
    assert as_tuple(t128.select(8, 4)) == ("TiledQ", 8, 16, 8)
    for s in (unsupported, single_partial):
        assert s.max_q_tokens_per_partial_output() == 1
        assert as_tuple(s.select(16, 4))[0] == "SingleQ"


def test_selector_matrix_oracle(host_oracle):
    S = host_oracle.SplitKVSelector
    t256, t256p8, t128 = S(True, 256, 16, 6), S(True, 256, 8, 6), S(True, 128, 8, 8)
    assert t256.max_q_tokens_per_partial_output() == 8
    assert t256.select(4, 4) == ("SingleQ", 256, 256, 6)
    assert t256.select(8, 4) == ("TiledQ", 8, 16, 3)
    assert t256.select(16, 4) == ("TiledQ", 8, 16, 6)
    assert t256p8.select(16, 4) == ("TiledQ", 8, 16, 6)
    assert t128.select(8, 4) == ("TiledQ", 8, 16, 8)
    for s in (S(True, 256, 4, 8), S(True, 128, 8, 8, dspark_history=True)):
        assert s.max_q_tokens_per_partial_output() == 1
        assert s.select(16, 4)[0] == "SingleQ"


def test_selector_f32_and_wide_groups_stay_single_q(psi, host_oracle):
    f32 = psi.GQASplitKV.new(bf16_config(psi, 256, 6, 16, dtype=psi.Dtype.Float32))
    assert as_tuple(f32.select(64, 8))[0] == "SingleQ"
    wide = psi.GQASplitKV.new(bf16_config(psi, 128, 16, 8))
    assert as_tuple(wide.select(64, 8))[0] == "SingleQ"
    assert host_oracle.SplitKVSelector(False, 256, 16, 6).select(64, 8)[0] == "SingleQ"
    assert host_oracle.SplitKVSelector(True, 128, 8, 16).select(64, 8)[0] == "SingleQ"


def test_selector_agrees_over_a_grid(psi, host_oracle):
    for (d, g, p) in [(256, 6, 16), (256, 6, 8), (128, 8, 8), (256, 8, 4), (128, 4, 16), (64, 2, 32), (256, 1, 16)]:
        lib = psi.GQASplitKV.new(bf16_config(psi, d, g, p))
        ora = host_oracle.SplitKVSelector(True, d, p, g)
        for tiles in (1, 2, 3, 7, 32):
            for tokens in sorted({tiles, tiles + 1, 2 * tiles - 1, 2 * tiles, 3 * tiles, 4 * tiles - 1, 4 * tiles,
                                  8 * tiles}):
                if tokens < tiles:
                    continue
                assert as_tuple(lib.select(tokens, tiles)) == ora.select(tokens, tiles), (d, g, p, tokens, tiles)


def _select_256_8(psi, host_oracle, token_indices, request_tokens, bucketed):
    cu = [0]
    for n in request_tokens:
        cu.append(cu[-1] + n)
    lib = psi.select_split_kv_variant(psi.GQASplitKV.new(bf16_config(psi, 256, 6, 8)), 128,
                                      psi.GQAReplayBucketPolicy(128) if bucketed else None, token_indices, cu)
    ora = host_oracle.select_split_kv_variant(host_oracle.SplitKVSelector(True, 256, 8, 6), True, 128,
                                              128 if bucketed else 0, token_indices, cu)
    assert as_tuple(lib) == ora
    return ora[0]


@pytest.mark.parametrize("bucketed", [False, True])
def test_d256_page8_selector_measured_crossovers(psi, host_oracle, bucketed):
    for tokens, context in [(1, 65536), (2, 65536), (4, 128), (8, 128), (25, 32)]:
        assert _select_256_8(psi, host_oracle, [context], [tokens], bucketed) == "SingleQ", (tokens, context)
    for tokens, context in [(4, 512), (8, 512), (16, 128), (25, 128), (64, 0)]:
        assert _select_256_8(psi, host_oracle, [context], [tokens], bucketed) == "TiledQ", (tokens, context)


def test_d256_page8_selector_prices_request_local_tail_tiles(psi, host_oracle):
    assert _select_256_8(psi, host_oracle, [65536] * 8, [1] * 8, False) == "SingleQ"
    assert _select_256_8(psi, host_oracle, [1024, 65536], [64, 1], False) == "SingleQ"
    assert _select_256_8(psi, host_oracle, [65536, 1024], [1, 8], False) == "SingleQ"
    assert _select_256_8(psi, host_oracle, [65536, 65536], [8, 1], False) == "TiledQ"


def test_d256_page8_work_model_matches_the_materialised_plan(psi, host_oracle):
    sel = host_oracle.SplitKVSelector(True, 256, 8, 6)
    tiled = sel.select(65, 9)
    work = host_oracle.tiled_q_selection_work(tiled, 6, 128, None, [1024, 65536], [0, 64, 65])
    assert (work["num_kv_splits"], work["active_partial_states"], work["padded_replay_work"]) == (72, 128, 1024)
    md = psi.GQAMetadataBuffers(None, 128)
    shape = md.update([0, 1], [1024, 65536], [0, 64, 65], from_tuple(psi, tiled))
    assert shape.num_sdpa_map_task_templates == 72
    assert shape.num_total_sdpa_map_task_templates * 8 == 1024
    tiles = md.h_q_token_tiles[:2 * shape.num_q_token_tiles].reshape(-1, 2)
    cu = md.h_cu_kv_splits[:shape.num_q_token_tiles + 1]
    assert int(((tiles[:, 1] - tiles[:, 0]) * (cu[1:] - cu[:-1])).sum()) == 128

    work = host_oracle.tiled_q_selection_work(tiled, 6, 128, None, [65536] * 8, list(range(9)))
    assert (work["num_kv_splits"], work["active_partial_states"], work["padded_replay_work"]) == (128, 128, 1024)

    policy = host_oracle.ReplayBucketPolicy(128)
    tiled = sel.select(25, 4)
    work = host_oracle.tiled_q_selection_work(tiled, 6, 128, policy, [65536], [0, 25])
    assert (work["num_kv_splits"], work["active_partial_states"], work["padded_replay_work"]) == (23, 128, 24 * 8)
    shape = md.update_bucketed([0], [65536], [0, 25], from_tuple(psi, tiled), psi.GQAReplayBucketPolicy(128))
    assert shape.num_sdpa_map_task_templates == 23 and shape.num_total_sdpa_map_task_templates == 24


# ------------------------------------------------------------------ split plans

SINGLE = ("SingleQ", 8, 32, 1)
TILED = ("TiledQ", 8, 4, 1)
KAT = dict(req_slots=[2, 5], token_indices=[7, 20], cu_tokens=[0, 2, 5])


def shape_tuple(s):
    return (s.num_tokens, s.num_total_tokens, s.num_q_token_tiles, s.num_total_q_token_tiles,
            s.num_sdpa_map_task_templates, s.num_total_sdpa_map_task_templates, s.reduce_sdpa_partial_outputs)


def test_metadata_kat_library(psi):
    md = psi.GQAMetadataBuffers(None, 8)
    s = md.update(KAT["req_slots"], KAT["token_indices"], KAT["cu_tokens"], from_tuple(psi, SINGLE))
    assert md.h_req_slots[:5].tolist() == [2, 2, 5, 5, 5]
    assert md.h_flat_token_indices[:5].tolist() == [7, 8, 20, 21, 22]
    assert md.h_kv_splits[:24].tolist() == [0, 0, 8, 1, 0, 9, 2, 0, 8, 2, 8, 21, 3, 0, 8, 3, 8, 22, 4, 0, 8, 4, 8, 23]
    assert md.h_cu_kv_splits[:6].tolist() == [0, 1, 2, 4, 6, 8]
    assert shape_tuple(s) == (5, 5, 5, 5, 8, 8, True)

    s = md.update(KAT["req_slots"], KAT["token_indices"], KAT["cu_tokens"], from_tuple(psi, TILED))
    assert md.h_q_token_tiles[:4].tolist() == [0, 2, 2, 5]
    assert md.h_kv_splits[:12].tolist() == [0, 0, 9, 1, 0, 12, 1, 12, 23, MAX, MAX, MAX]
    assert md.h_cu_kv_splits[:3].tolist() == [0, 1, 3]
    assert shape_tuple(s) == (5, 5, 2, 2, 3, 4, True)

    policy = psi.GQAReplayBucketPolicy(8)
    s = md.update_bucketed(KAT["req_slots"], KAT["token_indices"], KAT["cu_tokens"], from_tuple(psi, TILED), policy)
    assert shape_tuple(s) == (5, 6, 2, 2, 3, 4, True)
    s = md.update_bucketed_with_token_capacity(KAT["req_slots"], KAT["token_indices"], KAT["cu_tokens"],
                                               from_tuple(psi, TILED), policy, 5)
    assert shape_tuple(s) == (5, 5, 2, 2, 3, 4, True)
    assert shape_tuple(md.replay_shape()) == shape_tuple(s)
    assert as_tuple(md.split_kv_variant()) == TILED


def test_metadata_kat_oracle(host_oracle):
    m = host_oracle.metadata_update(8, variant=SINGLE, **KAT)
    assert m["req_slots"] == [2, 2, 5, 5, 5] and m["flat_token_indices"] == [7, 8, 20, 21, 22]
    assert m["kv_splits"] == [0, 0, 8, 1, 0, 9, 2, 0, 8, 2, 8, 21, 3, 0, 8, 3, 8, 22, 4, 0, 8, 4, 8, 23]
    assert m["cu_kv_splits"] == [0, 1, 2, 4, 6, 8] and m["shape"] == (5, 5, 5, 5, 8, 8, True)
    m = host_oracle.metadata_update(8, variant=TILED, **KAT)
    assert m["q_token_tiles"] == [0, 2, 2, 5]
    assert m["kv_splits"] == [0, 0, 9, 1, 0, 12, 1, 12, 23, MAX, MAX, MAX]
    assert m["cu_kv_splits"] == [0, 1, 3] and m["shape"] == (5, 5, 2, 2, 3, 4, True)
    assert host_oracle.metadata_update(8, variant=TILED, mode="bucketed", **KAT)["shape"] == (5, 6, 2, 2, 3, 4, True)
    assert host_oracle.metadata_update(8, variant=TILED, mode="caller", caller_tokens=5, **KAT)["shape"] == \
        (5, 5, 2, 2, 3, 4, True)
    m = host_oracle.metadata_update(12, [2, 5, 7], [0, 0, 0], [0, 4, 8, 9], TILED, mode="bucketed")
    assert m["shape"] == (9, 12, 3, 4, 3, 4, True)


def test_bucketed_update_leaves_poisoned_tails_alone(psi):
    md = psi.GQAMetadataBuffers(None, 12)
    md.h_q_token_tiles[:] = 0xA5A5A5A5
    md.h_kv_splits[:] = 0xB6B6B6B6
    md.h_cu_kv_splits[:] = 0xC7C7C7C7
    s = md.update_bucketed([2, 5, 7], [0, 0, 0], [0, 4, 8, 9], from_tuple(psi, TILED), psi.GQAReplayBucketPolicy(12))
    assert shape_tuple(s) == (9, 12, 3, 4, 3, 4, True)
    assert md.h_q_token_tiles[6:8].tolist() == [0xA5A5A5A5] * 2
    assert md.h_kv_splits[9:12].tolist() == [MAX] * 3
    assert md.h_kv_splits[12] == 0xB6B6B6B6
    assert md.h_cu_kv_splits[4] == 0xC7C7C7C7


def test_metadata_contract_violations(psi):
    md = psi.GQAMetadataBuffers(None, 12)
    policy = psi.GQAReplayBucketPolicy(12)
    single = from_tuple(psi, SINGLE)
    with pytest.raises(psi.PsiHipError, match="must not exceed the caller-owned token capacity"):
        md.update_bucketed_with_token_capacity([0], [0], [0, 9], single, policy, 8)
    with pytest.raises(psi.PsiHipError, match="must not exceed the metadata capacity"):
        md.update_bucketed_with_token_capacity([0], [0], [0, 9], single, policy, 13)
    with pytest.raises(psi.PsiHipError, match="nondecreasing"):
        md.update([0, 1], [0, 0], [0, 3, 2], single)
    with pytest.raises(psi.PsiHipError):
        md.update([0], [0], [0, 13], single)  # more tokens than capacity
    with pytest.raises(psi.PsiHipError):
        md.update([0], [0], [0, 0], single)  # empty batch
    with pytest.raises(psi.PsiHipError):
        md.update([0], [MAX], [0, 2], single)  # position overflows u32


def test_fixed_partition_plan(psi, host_oracle):
    md = psi.GQAMetadataBuffers(None, 4, max_kv_splits=64)
    single = psi.GQASplitKVVariant.SingleQ(256, 256, 6)
    s = md.update_fixed_partition([0, 1, 2], [1023, 511, 1300], [0, 1, 2, 3], single, 512)
    splits, cu = host_oracle.fixed_partition_splits([1023, 511, 1300], 512)
    assert splits == [0, 0, 512, 0, 512, 1024, 1, 0, 512, 2, 0, 512, 2, 512, 1024, 2, 1024, 1301]
    assert md.h_kv_splits[:len(splits)].tolist() == splits
    assert md.h_cu_kv_splits[:4].tolist() == cu == [0, 2, 3, 6]
    assert s.num_sdpa_map_task_templates == 6 and s.num_total_sdpa_map_task_templates == 6
    with pytest.raises(psi.PsiHipError):
        psi.GQAMetadataBuffers(None, 4, max_kv_splits=5).update_fixed_partition(
            [0, 1, 2], [1023, 511, 1300], [0, 1, 2, 3], single, 512)


def random_batch(rng, max_tokens):
    n_req = rng.randint(1, min(6, max_tokens))
    budget = max_tokens
    counts = []
    for r in range(n_req):
        left = n_req - r - 1
        c = rng.randint(0 if r else 1, max(1, min(20, budget - left)))
        c = min(c, budget - left) if budget - left > 0 else 0
        counts.append(max(c, 0))
        budget -= counts[-1]
    if sum(counts) == 0:
        counts[0] = 1
    cu = [0]
    for c in counts:
        cu.append(cu[-1] + c)
    starts = [rng.choice([0, 1, 7, 63, 64, 500, 4095, rng.randrange(0, 70000)]) for _ in range(n_req)]
    slots = [rng.randrange(0, 16) for _ in range(n_req)]
    return slots, starts, cu


@pytest.mark.parametrize("seed", range(40))
def test_plans_agree_on_random_batches(psi, host_oracle, seed):
    rng = random.Random(seed)
    max_tokens = rng.choice([8, 12, 33, 64, 128])
    slots, starts, cu = random_batch(rng, max_tokens)
    variant = rng.choice([("SingleQ", rng.choice([8, 64, 256]), 256, 6), ("TiledQ", 8, rng.choice([4, 16]), 3)])
    mode = rng.choice(["exact", "bucketed", "caller"])
    boundaries = rng.choice([(), (5,), (6, 10, 18)])
    caller = min(max_tokens, cu[-1] + rng.randint(0, 3))
    exp = host_oracle.metadata_update(max_tokens, slots, starts, cu, variant, mode=mode, caller_tokens=caller,
                                      boundaries=boundaries)
    md = psi.GQAMetadataBuffers(None, max_tokens)
    v = from_tuple(psi, variant)
    if mode == "exact":
        s = md.update(slots, starts, cu, v)
    elif mode == "bucketed":
        s = md.update_bucketed(slots, starts, cu, v, psi.GQAReplayBucketPolicy(max_tokens, boundaries))
    else:
        s = md.update_bucketed_with_token_capacity(slots, starts, cu, v,
                                                   psi.GQAReplayBucketPolicy(max_tokens, boundaries), caller)
    assert shape_tuple(s) == exp["shape"]
    t = cu[-1]
    assert md.h_req_slots[:t].tolist() == exp["req_slots"]
    assert md.h_flat_token_indices[:t].tolist() == exp["flat_token_indices"]
    assert md.h_q_token_tiles[:len(exp["q_token_tiles"])].tolist() == exp["q_token_tiles"]
    assert md.h_kv_splits[:len(exp["kv_splits"])].tolist() == exp["kv_splits"]
    assert md.h_cu_kv_splits[:len(exp["cu_kv_splits"])].tolist() == exp["cu_kv_splits"]


@pytest.mark.parametrize("seed", range(10))
def test_plan_invariants(psi, seed):
    """What any valid plan satisfies, whatever the greedy order: every row's splits tile [0, ctx)
    on KV-tile boundaries, in order, and the budget is respected."""
    rng = random.Random(100 + seed)
    max_tokens = rng.choice([16, 64, 128])
    slots, starts, cu = random_batch(rng, max_tokens)
    tile = rng.choice([8, 256])
    md = psi.GQAMetadataBuffers(None, max_tokens)
    s = md.update(slots, starts, cu, psi.GQASplitKVVariant.SingleQ(tile, 256, 6))
    assert s.num_sdpa_map_task_templates <= max_tokens
    ks = md.h_kv_splits[:3 * s.num_sdpa_map_task_templates].reshape(-1, 3)
    cu_s = md.h_cu_kv_splits[:s.num_tokens + 1]
    for row in range(s.num_tokens):
        part = ks[cu_s[row]:cu_s[row + 1]]
        ctx = int(md.h_flat_token_indices[row]) + 1
        assert len(part) >= 1 and (part[:, 0] == row).all()
        assert part[0, 1] == 0 and part[-1, 2] == ctx
        assert (part[1:, 1] == part[:-1, 2]).all() and (part[:, 1] < part[:, 2]).all()
        assert (part[:, 1] % tile == 0).all()
    assert (md.h_kv_splits[3 * s.num_sdpa_map_task_templates:3 * s.num_total_sdpa_map_task_templates] == MAX).all()


# ------------------------------------------------------------------ page table index math (no device)


def _start_index(psi, layout, slot, layer, block):
    lib = psi.load()
    out = ctypes.c_uint64()
    st = psi.GQAPageTableLayout(*layout).struct()
    rc = lib.psi_hip_page_table_start_index(ctypes.byref(st), slot, layer, block, ctypes.byref(out))
    return rc, out.value


def test_page_table_start_index(psi, host_oracle):
    layout = (4, 3, 6, 2)
    for slot, layer, block in [(0, 0, 0), (1, 2, 5), (3, 0, 4), (3, 2, 5)]:
        rc, idx = _start_index(psi, layout, slot, layer, block)
        assert rc == 0
        assert idx == ((slot * 3 + layer) * 6 + block) * 2 == host_oracle.page_table_start_index(layout, slot, layer, block)
    for bad in [(4, 0, 0), (0, 3, 0), (0, 0, 6)]:
        assert _start_index(psi, layout, *bad)[0] != 0
        with pytest.raises(AssertionError):
            host_oracle.page_table_start_index(layout, *bad)


def test_page_ids_by_layer(psi, host_oracle):
    lib = psi.load()
    block = (ctypes.c_uint32 * 4)(10, 11, 20, 21)
    out = (ctypes.c_uint32 * 4)()
    assert lib.psi_hip_page_ids_by_layer(block, 4, 2, 2, out) == 0
    assert [list(out[0:2]), list(out[2:4])] == [[10, 11], [20, 21]] == host_oracle.page_ids_by_layer([10, 11, 20, 21], 2, 2)
    assert lib.psi_hip_page_ids_by_layer(block, 3, 2, 2, out) != 0


def test_tokens_per_page(psi, oracle):
    for dtype, es, odt in ((psi.Dtype.Float32, 4, oracle.F32), (psi.Dtype.Bfloat16, 2, oracle.BF16),
                          (psi.Dtype.Float16, 2, oracle.F16)):
        for hkv, d, p in [(1, 2, 2), (2, 256, 16), (4, 256, 16), (4, 128, 8), (8, 64, 32)]:
            cfg = psi.GQAKVPageWriteConfig(dtype=dtype, page_bytes=2 * hkv * d * p * es, num_kv_heads=hkv, head_dim=d)
            assert cfg.num_tokens_per_page() == p == oracle.tokens_per_page(hkv, d, 2 * hkv * d * p * es, odt)
    bad = psi.GQAKVPageWriteConfig(dtype=psi.Dtype.Bfloat16, page_bytes=1000, num_kv_heads=2, head_dim=256)
    with pytest.raises(psi.PsiHipError):
        bad.num_tokens_per_page()


def test_balance_plan_covers_the_same_ranges(psi):
    md = psi.GQAMetadataBuffers(None, 8, max_kv_splits=256)
    single = psi.GQASplitKVVariant.SingleQ(256, 256, 6)
    ctx = [5000, 300, 8192, 1024, 17]
    md.update_fixed_partition(list(range(5)), [c - 1 for c in ctx], list(range(6)), single, 512)
    s = md.balance(24)
    ks = md.h_kv_splits[:3 * s.num_sdpa_map_task_templates].reshape(-1, 3)
    cu = md.h_cu_kv_splits[:6]
    for row, c in enumerate(ctx):
        part = ks[cu[row]:cu[row + 1]]
        assert part[0, 1] == 0 and part[-1, 2] == c and (part[1:, 1] == part[:-1, 2]).all()
        assert (part[:, 0] == row).all()
    w = md.h_worker_cu
    assert w[0] == 0 and w[-1] == s.num_sdpa_map_task_templates and (np.diff(w.astype(np.int64)) >= 0).all()
    # equal shares of the cost (16-token tiles plus 10 per row started; the last worker takes what is left), and
    # inside a worker one row per token: at most workers + tokens rows
    tiles = (-(-ks[:, 2].astype(np.int64) // 16)) - ks[:, 1].astype(np.int64) // 16
    per_worker = [int(tiles[w[i]:w[i + 1]].sum()) for i in range(24)]
    assert sum(per_worker) == sum(-(-c // 16) for c in ctx)
    cost = [t + 10 * int(w[i + 1] - w[i]) for i, t in enumerate(per_worker)]
    assert max(cost[:-1]) - min(cost[:-1]) <= 10 and 0 < cost[-1] <= max(cost[:-1])
    assert s.num_sdpa_map_task_templates <= 24 + len(ctx)
    for i in range(24):
        tokens = ks[w[i]:w[i + 1], 0].tolist()
        assert len(set(tokens)) == len(tokens), "adjacent pieces of a token inside a worker must be one row"


def test_balance_plan_does_not_depend_on_the_partition_length(psi):
    """The balanced cut depends on a batch's 16-token tiles alone: the same contexts planned with partitions of 16,
    512, 2048 tokens or unsplit (every one a multiple of the tile) give the same rows, offsets and worker table."""
    single = psi.GQASplitKVVariant.SingleQ(16, 256, 6)
    rng = np.random.default_rng(11)
    for trial in range(6):
        n = int(rng.integers(1, 24))
        ctx = rng.integers(1, 9000, n).tolist()
        plans = []
        for partition in (16, 512, 2048, 1 << 20):
            md = psi.GQAMetadataBuffers(None, n, max_kv_splits=sum(-(-c // partition) for c in ctx) + 1, max_workers=32)
            md.update_fixed_partition(list(range(n)), [c - 1 for c in ctx], list(range(n + 1)), single, partition)
            s = md.balance(32)
            rows = s.num_sdpa_map_task_templates
            plans.append((rows, md.h_kv_splits[:3 * rows].copy(), md.h_cu_kv_splits[:n + 1].copy(),
                          np.array(md.h_worker_cu).copy()))
        for other in plans[1:]:
            assert other[0] == plans[0][0]
            for a, b in zip(other[1:], plans[0][1:]):
                assert np.array_equal(a, b)


def test_balance_plan_with_more_workers_than_tiles(psi):
    """Tiny batches: workers without work get empty row ranges, nothing is lost."""
    md = psi.GQAMetadataBuffers(None, 4, max_kv_splits=16)
    single = psi.GQASplitKVVariant.SingleQ(256, 256, 6)
    ctx = [40, 1, 17]
    md.update_fixed_partition(list(range(3)), [c - 1 for c in ctx], list(range(4)), single, 512)
    s = md.balance(64)
    ks = md.h_kv_splits[:3 * s.num_sdpa_map_task_templates].reshape(-1, 3)
    cu = md.h_cu_kv_splits[:4]
    for row, c in enumerate(ctx):
        part = ks[cu[row]:cu[row + 1]]
        assert part[0, 1] == 0 and part[-1, 2] == c and (part[1:, 1] == part[:-1, 2]).all()
    w = md.h_worker_cu.astype(np.int64)
    assert w[0] == 0 and w[-1] == s.num_sdpa_map_task_templates and (np.diff(w) >= 0).all()
    assert (np.diff(w) == 0).sum() == 64 - 6 and (np.diff(w) <= 1).all()  # 6 tiles in all, one per busy worker


def test_longest_first_order(psi):
    lib = psi.load()
    rows = np.array([0, 0, 512, 0, 512, 700, 1, 0, 40, 2, 0, 512, 2, 512, 1024, 2, 1024, 1030,
                     MAX, MAX, MAX, MAX, MAX, MAX], np.uint32)
    index = np.zeros(8, np.uint32)
    p = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))  # noqa: E731
    assert lib.psi_hip_split_kv_order_longest_first(p(rows), 8, p(index)) == 0
    got = rows.reshape(-1, 3).tolist()
    assert got[:6] == [[0, 0, 512], [2, 0, 512], [2, 512, 1024], [0, 512, 700], [1, 0, 40], [2, 1024, 1030]]
    assert got[6:] == [[MAX, MAX, MAX]] * 2
    assert index.tolist() == [0, 3, 4, 1, 2, 5, 6, 7]


# ------------------------------------------------------------------ row groups of prefill chunks


def tiled_config(psi, hq, hkv, d=256, p=16, dtype=None):
    dtype = psi.Dtype.Bfloat16 if dtype is None else dtype
    layout = psi.GQAPageTableLayout(8, 1, 64, 1)
    return psi.GQASplitKVTiledQConfig(hq, hkv, d, hq // hkv, 8, 16, 1.0 / 16, 2 * hkv * d * p * dtype.item_size(),
                                      dtype, layout)


def check_groups(meta, shape, tile_size, max_tiles):
    """Every planned row sits in exactly one group; a group is a run of consecutive full tiles of one
    request that start at the same key."""
    rows = meta.h_kv_splits.reshape(-1, 3)
    tiles = meta.h_q_token_tiles.reshape(-1, 2)
    table = meta.h_row_groups.reshape(meta.num_row_groups, meta.group_tiles)
    assert meta.group_tiles == max_tiles
    seen = []
    order = []
    for g in table:
        members = [int(r) for r in g if r != MAX]
        assert members and [int(r) for r in g[:len(members)]] == members, "padding only at the end"
        seen += members
        first = rows[members[0]]
        slot = meta.h_req_slots[tiles[first[0]][0]]
        w, longest = 0, 0
        for i, r in enumerate(members):
            tile, begin, end = (int(x) for x in rows[r])
            assert begin == first[1] and tile == first[0] + i
            assert meta.h_req_slots[tiles[tile][0]] == slot
            if i + 1 < len(members):
                assert tiles[tile][1] - tiles[tile][0] == tile_size and tiles[tile][1] == tiles[tile + 1][0]
            w += int(tiles[tile][1] - tiles[tile][0]) * (end - begin)
            longest = max(longest, end - begin)
        order.append((longest, w))
    assert sorted(seen) == list(range(shape.num_sdpa_map_task_templates)), "rows lost or duplicated"
    # a work item walks its group's KV range whatever the number of its tokens: the longest range goes first, and
    # among equal ranges the group with more tokens x keys
    assert order == sorted(order, reverse=True), "longest group first"
    return table


def test_row_groups_of_a_prefill_chunk(psi):
    """A 70-token chunk on a 300-token prefix, 256-token partitions, next to two decode requests:
    24 Q / 4 KV heads deal 2 heads to a workgroup, so a group holds 16 tiles of 8 tokens."""
    meta = psi.GQAMetadataBuffers(None, 128, max_kv_splits=64)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, 6)
    shape = meta.update_fixed_partition([3, 1, 5], [300, 40, 999], [0, 70, 71, 72], variant, 256)
    assert meta.group_rows(tiled_config(psi, 24, 4)) == meta.num_row_groups > 0
    table = check_groups(meta, shape, 8, 16)
    rows = meta.h_kv_splits.reshape(-1, 3)
    # the chunk has 9 tiles; partition 0 is seen by all of them -> one group of 9
    sizes = sorted(int((g != MAX).sum()) for g in table if rows[g[0]][1] == 0 and rows[g[0]][0] < 9)
    assert sizes == [9]
    # the groups survive a re-ordering of the rows (positions change, membership does not)
    meta.order_longest_first()
    meta.group_rows(tiled_config(psi, 24, 4))
    check_groups(meta, shape, 8, 16)


@pytest.mark.parametrize("hq,hkv,expected", [(16, 2, 8), (8, 2, 8), (4, 4, 32), (10, 2, 6), (14, 2, 8)])
def test_row_group_size_follows_the_head_group(psi, hq, hkv, expected):
    meta = psi.GQAMetadataBuffers(None, 256, max_kv_splits=256)
    shape = meta.update_fixed_partition([0], [0], [0, 200], psi.GQASplitKVVariant.TiledQ(8, 16, min(hq // hkv, 8)), 128)
    assert meta.group_rows(tiled_config(psi, hq, hkv)) > 0
    check_groups(meta, shape, 8, expected)


def test_row_groups_unsupported_geometry_and_greedy_plan(psi):
    meta = psi.GQAMetadataBuffers(None, 64)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, 4)
    shape = meta.update([0, 1], [100, 7], [0, 20, 24], variant)
    # head_dim 64, 4-token pages and f32 storage have no grouped kernel; the reference's TiledQ profiles
    # (128, 8), (256, 8), (256, 16) (gqa_split_kv_tiled_q.rs:66-76) do
    assert meta.group_rows(tiled_config(psi, 8, 2, d=64)) == 0 and meta.group_tiles == 0
    assert meta.group_rows(tiled_config(psi, 8, 2, p=4)) == 0
    assert meta.group_rows(tiled_config(psi, 8, 2, d=128, p=8)) > 0
    assert meta.group_rows(tiled_config(psi, 8, 2, p=8)) > 0
    # the reference's greedy plan cuts every tile differently: groups degenerate but stay complete
    assert meta.group_rows(tiled_config(psi, 8, 2)) > 0
    check_groups(meta, shape, 8, 8)


def test_row_group_table_capacity_is_checked(psi):
    lib = psi.load()
    cfg = tiled_config(psi, 24, 4).struct()
    rows = np.array([0, 0, 16, 1, 0, 16], np.uint32)
    tiles = np.array([0, 8, 8, 10], np.uint32)
    slots = np.zeros(10, np.uint32)
    slots[8:] = 1
    table = np.zeros(5, np.uint32)
    n_tiles, n_groups = ctypes.c_uint32(), ctypes.c_uint32()
    p = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))  # noqa: E731
    rc = lib.psi_hip_split_kv_tiled_q_group_rows(ctypes.byref(cfg), 8, p(rows), 2, p(tiles), 2, p(slots), p(table), 5,
                                                 ctypes.byref(n_tiles), ctypes.byref(n_groups))
    assert rc != 0 and b"row-group table too small" in lib.psi_hip_last_error()
    table = np.zeros(32, np.uint32)
    assert lib.psi_hip_split_kv_tiled_q_group_rows(ctypes.byref(cfg), 8, p(rows), 2, p(tiles), 2, p(slots), p(table),
                                                   32, ctypes.byref(n_tiles), ctypes.byref(n_groups)) == 0
    # two requests never share a group; and no group is wider than the 5 tiles whose tokens fit one workgroup with
    # all six heads of a KV head, so the table is written that narrow (the launch then deals no heads to separate
    # work items)
    assert (n_tiles.value, n_groups.value) == (5, 2)
    assert table[:10].tolist() == [0] + [MAX] * 4 + [1] + [MAX] * 4
    # a group of six tiles is wider than that: the full width, 16 tiles of two heads each
    rows = np.array([[t, 0, 64] for t in range(6)], np.uint32).reshape(-1)
    tiles = np.array([[8 * t, 8 * t + 8] for t in range(6)], np.uint32).reshape(-1)
    slots = np.zeros(48, np.uint32)
    assert lib.psi_hip_split_kv_tiled_q_group_rows(ctypes.byref(cfg), 8, p(rows), 6, p(tiles), 6, p(slots), p(table),
                                                   32, ctypes.byref(n_tiles), ctypes.byref(n_groups)) == 0
    assert (n_tiles.value, n_groups.value) == (16, 1)
    assert table[:16].tolist() == list(range(6)) + [MAX] * 10


# ------------------------------------------------------------------ the whole plan in one call


@pytest.mark.parametrize("seed", range(12))
def test_single_call_prepare_equals_the_step_by_step_plan(psi, seed):
    """psi_hip_gqa_layer_prepare (variant selection, metadata update and dispatch plan in one host call) writes,
    array for array, what the separate entry points write: the reference's exact plan, the fixed-partition plan,
    and the three dispatch plans on top of it."""
    import importlib

    L = importlib.import_module("psi-dec_amd._lib")
    rng = np.random.default_rng(500 + seed)
    n = int(rng.integers(1, 9))
    q_len = int(rng.choice([1, 1, 2, 4, 11]))
    q_lens = np.full(n, q_len) if rng.random() < 0.6 else rng.integers(1, 12, size=n)
    starts = rng.integers(0, 5000, size=n).astype(np.uint32)
    slots = rng.permutation(16)[:n].astype(np.uint32)
    cu = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.uint32)
    core = psi.GQACore(0, 24 * 256, 256, 24, 4, 0.0625)
    gqa = psi.GQA(None, core, psi.GQAMetalConfig(65536, 64, 1e-6, 1e6))
    max_tokens, max_splits, workers = 128, 2048, 8

    def arrays(md):
        s = md.replay_shape()
        out = dict(shape=s, variant=md.split_kv_variant(), slots=md.h_req_slots[:s.num_tokens].tolist(),
                   pos=md.h_flat_token_indices[:s.num_tokens].tolist(),
                   tiles=md.h_q_token_tiles[:2 * s.num_q_token_tiles].tolist() if md.split_kv_variant().is_tiled() else None,
                   splits=md.h_kv_splits[:3 * s.num_total_sdpa_map_task_templates].tolist(),
                   cu=md.h_cu_kv_splits[:(s.num_q_token_tiles if md.split_kv_variant().is_tiled() else s.num_tokens) + 1].tolist(),
                   index=None if md.h_partial_row_index is None else md.h_partial_row_index[:s.num_sdpa_map_task_templates].tolist(),
                   workers=None if md.h_worker_cu is None else md.h_worker_cu.tolist(),
                   groups=None if md.h_row_groups is None or not md.num_row_groups else
                   (md.group_tiles, md.h_row_groups[:md.group_tiles * md.num_row_groups].tolist()))
        return out

    variant = psi.select_split_kv_variant(gqa.split_kv, max_tokens, None, starts.tolist(), cu.tolist())
    # the reference's plan
    a = psi.GQAMetadataBuffers(None, max_tokens)
    a.update(slots, starts, cu, variant)
    b = psi.GQAMetadataBuffers(None, max_tokens)
    assert gqa.prepare(b, slots, starts, cu) == a.replay_shape()
    assert arrays(a) == arrays(b)
    for dispatch in ("plan", "longest", "balanced", "groups"):
        a = psi.GQAMetadataBuffers(None, max_tokens, max_kv_splits=max_splits, max_workers=workers)
        a.update_fixed_partition(slots, starts, cu, variant, 256)
        if dispatch == "longest":
            a.order_longest_first()
        elif dispatch == "balanced" or (dispatch == "groups" and not variant.is_tiled()):
            a.balance(workers)
        elif dispatch == "groups":
            cfg = psi.GQASplitKVTiledQConfig(24, 4, 256, variant.q_head_tile_size, variant.q_token_tile_size,
                                             variant.kv_token_tile_size, 0.0625, 65536, psi.Dtype.Bfloat16, None)
            a.group_rows(cfg)
        b = psi.GQAMetadataBuffers(None, max_tokens, max_kv_splits=max_splits, max_workers=workers)
        b.prepare(gqa.struct(), slots, starts, cu, capacity_mode=L.CAPACITY_FIXED_PARTITION, partition_tokens=256,
                  dispatch={"plan": L.DISPATCH_PLAN_ORDER, "longest": L.DISPATCH_LONGEST_FIRST,
                            "balanced": L.DISPATCH_BALANCED, "groups": L.DISPATCH_ROW_GROUPS}[dispatch],
                  num_workers=workers)
        assert arrays(a) == arrays(b), dispatch
        if variant.is_tiled():
            assert b.max_active_q_tile_tokens == min(int(q_lens.max()), variant.q_token_tile_size)


@pytest.mark.parametrize("hq,q_lens,expect_groups", [
    (24, [1, 1, 1], False),        # decode: SingleQ, balanced
    (24, [4, 2, 4], False),        # one tile of up to 24 columns per request: the multi-query pipeline, balanced
    (24, [8, 8, 8], False),        # 48 columns: still the pipeline
    (24, [8, 9, 8], True),         # one request with a second Q-token tile: row groups
    (32, [8, 8, 3], True),         # 64 columns per tile: row groups
    (28, [7, 2, 1], True),         # 49 columns
    (28, [6, 6, 6], False),        # 42
    (24, [300, 1, 2], True),       # a prefill chunk among decode-sized requests
])
def test_prepare_picks_the_dispatch_by_the_batch(psi, hq, q_lens, expect_groups):
    """PSI_HIP_DISPATCH_AUTO: row groups over the planner's partition when a request brings more than one Q-token
    tile or a tile more than 48 query columns, the balanced plan over the caller's partition otherwise - and either
    way exactly what the explicit dispatch writes."""
    import importlib

    L = importlib.import_module("psi-dec_amd._lib")
    core = psi.GQACore(0, hq * 256, 256, hq, 4, 0.0625)
    gqa = psi.GQA(None, core, psi.GQAMetalConfig(65536, 64, 1e-6, 1e6))
    q_lens = np.array(q_lens)
    starts = np.array([5000, 300, 12000], np.uint32)
    slots = np.array([2, 0, 1], np.uint32)
    cu = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.uint32)
    variant = psi.select_split_kv_variant(gqa.split_kv, 512, None, starts.tolist(), cu.tolist())
    assert variant.is_tiled() == (int(q_lens.max()) > 1)

    def arrays(md):
        s = md.replay_shape()
        return dict(shape=s, splits=md.h_kv_splits[:3 * s.num_total_sdpa_map_task_templates].tolist(),
                    workers=None if md.h_worker_cu is None else md.h_worker_cu.tolist(),
                    groups=None if md.h_row_groups is None or not md.num_row_groups else
                    (md.group_tiles, md.h_row_groups[:md.group_tiles * md.num_row_groups].tolist()))

    auto = psi.GQAMetadataBuffers(None, 512, max_kv_splits=2048, max_workers=8)
    gqa.prepare_fixed_partition(auto, slots, starts, cu, 512, auto=True, num_workers=8)
    assert (auto.num_row_groups > 0) == expect_groups
    explicit = psi.GQAMetadataBuffers(None, 512, max_kv_splits=2048, max_workers=8)
    if expect_groups:
        planned = psi.chunk_partition_tokens(gqa.split_kv.config, variant.q_token_tile_size, starts.tolist(), cu.tolist())
        assert planned > 0
        gqa.prepare_fixed_partition(explicit, slots, starts, cu, planned, grouped=True)
        assert arrays(auto) == arrays(explicit)
        # a partition length of 0 asks for the planner's, too
        gqa.prepare_fixed_partition(explicit, slots, starts, cu, 0, grouped=True)
        assert arrays(auto) == arrays(explicit)
    else:
        gqa.prepare_fixed_partition(explicit, slots, starts, cu, 512, balanced=True, num_workers=8)
        assert auto.num_workers == 8 and arrays(auto) == arrays(explicit)


@pytest.mark.parametrize("dispatch_name", ["plan", "balanced", "groups"])
def test_prepare_buckets_the_dispatch_plans_capacities(psi, dispatch_name):
    """With `bucket_capacities` the one-call preparation rounds the recorded capacities - tokens, Q-token tiles,
    KV splits (the re-cut rows of a balanced plan) and row groups - up to `ReplayBucketPolicy` buckets
    (crates/inference-executor-core/src/replay.rs:4-87) and pads the tables with the sentinel up to them: many
    different batches then share few (capacity) keys, and the active part of every array is what the unbucketed
    preparation writes."""
    import importlib

    L = importlib.import_module("psi-dec_amd._lib")
    MAX = 0xFFFFFFFF
    core = psi.GQACore(0, 24 * 256, 256, 24, 4, 0.0625)
    gqa = psi.GQA(None, core, psi.GQAMetalConfig(65536, 64, 1e-6, 1e6))
    max_tokens, max_splits, workers = 256, 512, 8
    dispatch = {"plan": L.DISPATCH_PLAN_ORDER, "balanced": L.DISPATCH_BALANCED, "groups": L.DISPATCH_ROW_GROUPS}[dispatch_name]
    tiled = dispatch_name == "groups"
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, 6) if tiled else psi.GQASplitKVVariant.SingleQ(256, 256, 6)
    token_policy, split_policy = psi.ReplayBucketPolicy(max_tokens), psi.ReplayBucketPolicy(max_splits + workers)
    rng = np.random.default_rng(77)
    keys, exact_keys = set(), set()
    for _ in range(40):
        n = int(rng.integers(1, 12))
        q_lens = rng.integers(9, 20, size=n) if tiled else np.ones(n, dtype=np.int64)
        starts = rng.integers(0, 3000, size=n).astype(np.uint32)
        slots = rng.permutation(16)[:n].astype(np.uint32)
        cu = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.uint32)
        plain = psi.GQAMetadataBuffers(None, max_tokens, max_kv_splits=max_splits, max_workers=workers)
        plain.prepare(gqa.struct(), slots, starts, cu, capacity_mode=L.CAPACITY_FIXED_PARTITION, partition_tokens=256,
                      dispatch=dispatch, num_workers=workers, variant=variant)
        md = psi.GQAMetadataBuffers(None, max_tokens, max_kv_splits=max_splits, max_workers=workers)
        md.h_kv_splits[:] = 0x5A5A5A5A
        s = md.prepare(gqa.struct(), slots, starts, cu, capacity_mode=L.CAPACITY_FIXED_PARTITION, partition_tokens=256,
                       dispatch=dispatch, num_workers=workers, variant=variant, bucket_capacities=True)
        e = plain.replay_shape()
        assert (s.num_tokens, s.num_q_token_tiles, s.num_sdpa_map_task_templates) == \
               (e.num_tokens, e.num_q_token_tiles, e.num_sdpa_map_task_templates)
        assert s.num_total_tokens == token_policy.capacity(s.num_tokens)
        assert s.num_total_q_token_tiles == token_policy.capacity(s.num_q_token_tiles)
        assert s.num_total_sdpa_map_task_templates == split_policy.capacity(s.num_sdpa_map_task_templates)
        rows, total = s.num_sdpa_map_task_templates, s.num_total_sdpa_map_task_templates
        assert md._h_kv_splits_all[:3 * rows].tolist() == plain._h_kv_splits_all[:3 * rows].tolist()
        assert (md._h_kv_splits_all[3 * rows:3 * total] == MAX).all()
        if tiled:
            assert md.num_row_groups >= plain.num_row_groups > 0 and md.group_tiles == plain.group_tiles
            used = plain.num_row_groups * plain.group_tiles
            assert md.h_row_groups[:used].tolist() == plain.h_row_groups[:used].tolist()
            assert (md.h_row_groups[used:md.num_row_groups * md.group_tiles] == MAX).all()
        keys.add((s.num_total_tokens, s.num_total_q_token_tiles, total, md.num_row_groups))
        exact_keys.add((e.num_total_tokens, e.num_total_q_token_tiles, e.num_total_sdpa_map_task_templates,
                        plain.num_row_groups))
    assert len(keys) < len(exact_keys) and (tiled or len(keys) <= 20), (len(keys), len(exact_keys))


@pytest.mark.parametrize("balanced", [False, True])
def test_advance_decode_equals_a_fresh_preparation(psi, balanced):
    """psi_hip_gqa_layer_advance_decode moves a decode batch's plan on by one token per sequence in place.  Over 60
    decode steps of six sequences: whenever it says it advanced, every array equals what a fresh preparation of
    the grown contexts writes; it declines exactly when some sequence starts a new 16-token tile; and it declines
    for plans it is not meant for (a row index, several tokens per request, the reference's greedy capacities)."""
    core = psi.GQACore(0, 24 * 256, 256, 24, 4, 0.0625)
    gqa = psi.GQA(None, core, psi.GQAMetalConfig(65536, 64, 1e-6, 1e6))
    variant = psi.GQASplitKVVariant.SingleQ(16, 256, 6)
    rng = np.random.default_rng(77)
    n, workers = 6, 8
    ctx = rng.integers(1, 1500, size=n).astype(np.int64)
    ctx[0] = 510  # crosses a 512-token partition on the way
    slots = rng.permutation(16)[:n].astype(np.uint32)
    cu = np.arange(n + 1, dtype=np.uint32)

    def prepared(contexts):
        md = psi.GQAMetadataBuffers(None, 8, max_kv_splits=64, max_workers=workers)
        gqa.prepare_fixed_partition(md, slots, (contexts - 1).astype(np.uint32), cu, 512, balanced=balanced,
                                    variant=variant, num_workers=workers)
        return md

    def arrays(md):
        s = md.replay_shape()
        return (s, md.h_req_slots[:n].tolist(), md.h_flat_token_indices[:n].tolist(),
                md.h_kv_splits[:3 * s.num_total_sdpa_map_task_templates].tolist(), md.h_cu_kv_splits[:n + 1].tolist(),
                None if md.h_worker_cu is None else np.array(md.h_worker_cu).tolist())

    md = prepared(ctx)
    advanced = declined = 0
    for step in range(60):
        starts_a_tile = bool((ctx % 16 == 0).any())
        ok = md.advance_decode()
        ctx = ctx + 1
        assert ok != starts_a_tile, (step, ctx.tolist())
        if ok:
            advanced += 1
            assert arrays(md) == arrays(prepared(ctx)), step
        else:
            declined += 1
            md = prepared(ctx)
    assert advanced > 10 and declined > 10

    # plans it leaves alone
    md = psi.GQAMetadataBuffers(None, 8, max_kv_splits=64, max_workers=workers)
    gqa.prepare_fixed_partition(md, slots, (ctx - 1).astype(np.uint32), cu, 512, balanced=False, variant=variant)
    md.order_longest_first()
    md._last_prepare[2].value |= 1  # the row index is now in use
    assert not md.advance_decode()
    md = psi.GQAMetadataBuffers(None, 16, max_kv_splits=64, max_workers=workers)
    gqa.prepare_fixed_partition(md, slots[:2], np.array([100, 200], np.uint32), np.array([0, 2, 3], np.uint32), 512,
                                balanced=balanced, variant=variant, num_workers=workers)   # two tokens of one request
    assert not md.advance_decode()
    md = psi.GQAMetadataBuffers(None, 8)
    gqa.prepare(md, slots, (ctx - 1).astype(np.uint32), cu)  # the reference's greedy plan
    kept = arrays(md)
    assert not md.advance_decode() and arrays(md) == kept
