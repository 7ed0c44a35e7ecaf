"""GPU parity of the split-KV decode path (append -> map -> combine) against the CPU oracle, through
the C ABI.  Tolerance: 2e-3 max-abs and 1e-3 relative-RMS on the f32-accumulated outputs; page
contents bit-exact."""
import numpy as np
import pytest

from parity_util import importlib_workloads, run_and_check

pytestmark = pytest.mark.gpu


def test_c1_single_sequence_fp16(psi, oracle, device):
    """Batch 1, context 512, 16 Q / 2 KV heads, D=256, fp16, 16-token pages, one appended token."""
    wl = importlib_workloads(psi)
    w = wl.config_c1(seed=1)
    assert w.num_pages == 32 and w.context_lens[0] == 512
    stats, dw = run_and_check(psi, oracle, device, w, "C1")
    print("C1 max_abs %.3e rel_rms %.3e" % stats, dw.variant, dw.shape)


@pytest.mark.parametrize("partition", [None, 512])
def test_c2_shape_small_batch_bf16(psi, oracle, device, partition):
    """C2's geometry (24 Q / 4 KV, D=256, bf16, 16-token pages, shuffled pool) at a batch the
    oracle finishes in seconds; contexts straddle page and partition boundaries."""
    wl = importlib_workloads(psi)
    ctx = [1025, 1536, 2047, 3000, 17, 1, 16, 513]
    w = wl.make_workload(7, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16)
    stats, dw = run_and_check(psi, oracle, device, w, "C2-small", partition_tokens=partition, max_tokens=64)
    print("C2-small partition", partition, "max_abs %.3e rel_rms %.3e" % stats, dw.shape)


@pytest.mark.parametrize("dtype_name,hq,hkv,d,p", [
    ("Bfloat16", 32, 8, 128, 16),
    ("Float16", 8, 8, 128, 32),
    ("Bfloat16", 16, 2, 256, 16),
    ("Bfloat16", 5, 1, 256, 64),
    ("Bfloat16", 6, 2, 256, 16),
    ("Float16", 14, 2, 256, 16),
    ("Bfloat16", 24, 4, 256, 8),   # 8-token pages: every 16-token tile spans two pages
    ("Bfloat16", 32, 4, 128, 8),
    ("Float16", 12, 2, 256, 8),
])
def test_fast_path_geometries(psi, oracle, device, dtype_name, hq, hkv, d, p):
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(11, [700, 33, 1200, 64], hq, hkv, d, dtype, p)
    run_and_check(psi, oracle, device, w, f"{dtype_name} {hq}/{hkv}/{d} P={p}", max_tokens=32)


@pytest.mark.parametrize("dtype_name,hq,hkv,d,p", [
    ("Float32", 4, 2, 2, 4),
    ("Float32", 6, 2, 64, 8),
    ("Bfloat16", 8, 2, 96, 4),
    ("Bfloat16", 24, 4, 256, 8),
    ("Float16", 4, 1, 192, 3),
])
def test_generic_path_geometries(psi, oracle, device, dtype_name, hq, hkv, d, p):
    """Shapes outside the fast kernels' domain (f32, odd head_dim, small or non-power-of-two pages)."""
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(13, [70, 5, 129, 1], hq, hkv, d, dtype, p, num_page_ids_per_block=2)
    run_and_check(psi, oracle, device, w, f"generic {dtype_name} {hq}/{hkv}/{d} P={p}", max_tokens=16)


def test_fast_and_generic_variants_agree(psi, oracle, device):
    """Variant cross-check: the gfx950 kernels and the shape-generic kernels on one workload."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(17, [900, 2048, 77], 24, 4, 256, psi.Dtype.Bfloat16, 16)
    fast = wl.DeviceWorkload(device, w, partition_tokens=512, f32_output=True)
    fast.step()
    a = fast.output_f32()
    device.force_generic(True)
    try:
        slow = wl.DeviceWorkload(device, w, partition_tokens=512, f32_output=True)
        slow.step()
        b = slow.output_f32()
    finally:
        device.force_generic(False)
    assert np.abs(a - b).max() < 1e-5


def test_balanced_plan_matches_oracle(psi, oracle, device):
    """Equal-work worker plan: rows re-cut at tile boundaries, several rows per workgroup."""
    wl = importlib_workloads(psi)
    ctx = [3000, 17, 1025, 2048, 700, 1]
    w = wl.make_workload(29, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16)
    stats, dw = run_and_check(psi, oracle, device, w, "balanced", partition_tokens=512, balanced=True)
    m = dw.meta
    rows = m.h_kv_splits[: dw.shape.num_sdpa_map_task_templates * 3].reshape(-1, 3)
    tiles = (rows[:, 2] + 15) // 16 - rows[:, 1] // 16
    per_worker = [int(tiles[m.h_worker_cu[i]:m.h_worker_cu[i + 1]].sum()) for i in range(m.num_workers)]
    assert sum(per_worker) == sum(-(-c // 16) for c in ctx)
    cost = [t + 10 * int(m.h_worker_cu[i + 1] - m.h_worker_cu[i]) for i, t in enumerate(per_worker)]
    busy = [c for c in cost if c]  # the last busy worker takes what is left
    assert max(busy[:-1]) - min(busy[:-1]) <= 10 and busy[-1] <= max(busy[:-1])


@pytest.mark.parametrize("q_len", [1, 3])
def test_longest_first_dispatch_order(psi, oracle, device, q_len):
    """Rows re-ordered for dispatch (longest first): the combine follows them through its row index,
    and the result is bit-identical to the plan-order launch."""
    wl = importlib_workloads(psi)
    ctx = [3000, 17, 1025, 2048, 700, 5, 513]
    w = wl.make_workload(37, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    stats, dw = run_and_check(psi, oracle, device, w, "longest first", partition_tokens=512, longest_first=True)
    m = dw.meta
    n = dw.shape.num_sdpa_map_task_templates
    rows = m.h_kv_splits[: n * 3].reshape(-1, 3).astype(np.int64)
    lengths = rows[:, 2] - rows[:, 1]
    assert (np.diff(lengths) <= 0).all() and lengths[0] == 512
    assert sorted(m.h_partial_row_index[:n].tolist()) == list(range(n))
    plain = wl.DeviceWorkload(device, w, partition_tokens=512, f32_output=True)
    plain.step()
    assert np.array_equal(plain.output_f32(), dw.output_f32())


@pytest.mark.parametrize("longest_first", [False, True])
def test_long_split_lists_use_the_wide_combine(psi, oracle, device, longest_first):
    """Two sequences of 6000 and 3000 tokens cut into 16-token partitions: 375 and 188 rows per token,
    merged by the workgroup-per-row combine; one-token and many-token partitions must agree too."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(77, [6000, 3000], 16, 2, 256, psi.Dtype.Bfloat16, 16)
    variant = psi.GQASplitKVVariant.SingleQ(16, 256, 8)
    stats, dw = run_and_check(psi, oracle, device, w, "wide combine", partition_tokens=16, variant=variant,
                              longest_first=longest_first)
    assert dw.shape.num_sdpa_map_task_templates == 375 + 188
    _, dw2 = run_and_check(psi, oracle, device, w, "narrow combine", partition_tokens=1024, variant=variant)
    assert np.abs(dw.output_f32() - dw2.output_f32()).max() < 2e-5


@pytest.mark.parametrize("dtype_name,hq,hkv,d,p,q_lens,partition", [
    ("Bfloat16", 24, 4, 256, 16, 1, 512),                       # the decode batch of the headline configuration
    ("Bfloat16", 24, 4, 256, 16, 1, None),                      # the reference's greedy plan
    ("Float16", 16, 2, 256, 16, 1, 256),
    ("Bfloat16", 32, 8, 128, 16, 1, 512),
    ("Bfloat16", 24, 4, 256, 8, 1, 512),                        # 8-token pages
    ("Bfloat16", 24, 4, 256, 16, [3, 1, 2, 1, 4, 1, 2], 512),   # several new tokens per request, each its own row set
    ("Bfloat16", 16, 2, 256, 16, [20, 1, 17, 1, 1, 1, 1], 256),  # more than one tile of new tokens in a row
    ("Float32", 6, 2, 64, 8, 1, None),                          # outside the MFMA kernel: two launches inside
])
def test_append_folded_into_the_map(psi, oracle, device, dtype_name, hq, hkv, d, p, q_lens, partition):
    """The append and the map in one launch: the page arena equals the oracle's (and the append-then-map step's)
    bit for bit; outputs are within tolerance of the oracle and differ from the two-launch step only by the order
    of summation (the new tokens are folded in after the paged ones).  Contexts put new tokens at
    the start of a page, at its end, across a partition boundary (513 = 512 + 1) and in a one-token context."""
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    ctx = [3000, 17, 1025, 2048, 700, 32, 513] if partition else [300, 17, 129, 256, 70, 32, 65]
    if not np.isscalar(q_lens):
        ctx = [max(c, q) for c, q in zip(ctx, q_lens)]
    w = wl.make_workload(41, ctx, hq, hkv, d, dtype, p, q_lens=q_lens)
    variant = psi.GQASplitKVVariant.SingleQ(256, 256, min(hq // hkv, 8))
    what = f"append in map {dtype_name} {hq}/{hkv}/{d} P={p} q={q_lens}"
    stats, dw = run_and_check(psi, oracle, device, w, what, partition_tokens=partition, variant=variant,
                              fused_append=True, max_tokens=64)
    assert dw.fused_append
    plain = wl.DeviceWorkload(device, w, partition_tokens=partition, variant=variant, f32_output=True, max_tokens=64)
    plain.step()
    assert np.abs(plain.output_f32() - dw.output_f32()).max() < 2e-5
    assert np.array_equal(plain.pages_host(), dw.pages_host())


def test_append_folded_into_the_map_single_token_context(psi, oracle, device):
    """A request whose whole context is the token being appended: the row has no paged part at all."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(43, [1, 1, 2, 16, 17], 24, 4, 256, psi.Dtype.Bfloat16, 16)
    run_and_check(psi, oracle, device, w, "append in map, one-token contexts", partition_tokens=512, fused_append=True)


@pytest.mark.parametrize("dtype_name,hq,hkv,d,p,q_lens,fused_append", [
    ("Bfloat16", 24, 4, 256, 16, 1, False),
    ("Bfloat16", 24, 4, 256, 16, 1, True),                      # the default decode step of the bench
    ("Float16", 16, 2, 256, 16, 1, True),
    ("Bfloat16", 32, 8, 128, 8, 1, True),                       # 8-token pages
    ("Bfloat16", 24, 4, 256, 16, [3, 1, 2, 1, 4, 1, 2], True),  # several new tokens per request
    ("Float32", 6, 2, 64, 8, 1, True),                          # generic kernels: row per workgroup, two launches
])
def test_balanced_plan_with_merged_rows(psi, oracle, device, dtype_name, hq, hkv, d, p, q_lens, fused_append):
    """One workgroup per compute unit over equal shares of the tiles, a token's adjacent pieces inside a share
    merged into one row; with and without the append folded into the launch.  Contexts from one token to several
    shares long."""
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    ctx = [30000, 17, 1025, 9000, 700, 1, 513]
    if not np.isscalar(q_lens):
        ctx = [max(c, q) for c, q in zip(ctx, q_lens)]
    w = wl.make_workload(47, ctx, hq, hkv, d, dtype, p, q_lens=q_lens)
    variant = psi.GQASplitKVVariant.SingleQ(256, 256, min(hq // hkv, 8))
    what = f"balanced {dtype_name} {hq}/{hkv}/{d} P={p} q={q_lens} fused={fused_append}"
    stats, dw = run_and_check(psi, oracle, device, w, what, partition_tokens=512, variant=variant, balanced=True,
                              fused_append=fused_append, max_tokens=64)
    assert dw.balanced and dw.fused_append == fused_append
    m = dw.meta
    n = dw.shape.num_sdpa_map_task_templates
    assert n <= m.num_workers + w.num_tokens
    plain = wl.DeviceWorkload(device, w, partition_tokens=512, variant=variant, f32_output=True, max_tokens=64)
    plain.step()
    assert np.abs(plain.output_f32() - dw.output_f32()).max() < 2e-5
    assert np.array_equal(plain.pages_host(), dw.pages_host())
