"""Full-size workloads, checked through properties that do not need the scalar oracle to finish:
  * split-count invariance: any partition of [0, ctx) gives the same attention output;
  * page-placement invariance: moving pages in the arena and rewriting the table changes nothing,
    bit for bit;
  * a sampled oracle check: a few requests of the full batch recomputed on the CPU.
Plus the long-context / large-magnitude-K case at a length the oracle still covers."""
import numpy as np
import pytest

from parity_util import assert_outputs_close, importlib_workloads, layout_tuple, oracle_dtype, run_and_check

pytestmark = pytest.mark.gpu


def _full_c2(psi, device, partition, f32_output=True, seed=2, **how):
    wl = importlib_workloads(psi)
    w = wl.config_c2(seed=seed, batch=32, host_pages=False)
    return wl, w, wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=f32_output, **how)


def test_c2_full_batch_split_count_invariance(psi, device):
    """Batch 32, contexts 1024..8192 (592 MB of K/V): 512-, 2048-token partitions and one split per
    token must agree to f32 rounding."""
    outs = []
    for partition in (512, 2048, 1 << 20):
        _, w, dw = _full_c2(psi, device, partition)
        dw.step()
        outs.append(dw.output_f32())
        del dw
    assert np.isfinite(outs[0]).all()
    scale = np.sqrt((outs[2] ** 2).mean())
    assert np.abs(outs[0] - outs[2]).max() < 2e-5 and np.abs(outs[1] - outs[2]).max() < 2e-5
    assert np.sqrt(((outs[0] - outs[2]) ** 2).mean()) / scale < 1e-5


def test_c2_full_batch_page_placement_invariance(psi, device):
    import torch

    wl, w, dw = _full_c2(psi, device, 512, f32_output=False)
    dw.step()
    base = dw.output.clone()
    # move every page: new arena[perm[i]] = old arena[i], table entries follow
    page_elems = 2 * w.num_kv_heads * w.tokens_per_page * w.head_dim
    gen = torch.Generator(device="cpu")
    gen.manual_seed(5)
    perm = torch.randperm(w.num_pages, generator=gen).to(device.torch_device)
    moved = torch.empty_like(dw.pages)
    moved.view(w.num_pages, page_elems)[perm] = dw.pages.view(w.num_pages, page_elems)
    dw.pages = moved
    dw.page_ids = perm[dw.page_ids.long()].to(torch.int32)
    dw.output.zero_()
    dw.map()
    dw.reduce()
    device.sync()
    assert torch.equal(dw.output.view(torch.int16), base.view(torch.int16))


@pytest.mark.parametrize("how", [{}, {"balanced": True, "fused_append": True}], ids=["row per workgroup", "bench default"])
def test_c2_full_batch_sampled_against_oracle(psi, oracle, device, how):
    """Three of the 32 requests (shortest, median, longest context) recomputed by the scalar oracle
    from the device's own pages.  `bench default`: the balanced worker plan with the append folded into the
    map launch, as `bench.py` runs the step."""
    wl, w, dw = _full_c2(psi, device, 512, **how)
    dw.step()
    if how:
        plain = _full_c2(psi, device, 512)[2]
        plain.step()
        assert np.abs(plain.output_f32() - dw.output_f32()).max() < 2e-5
        assert np.array_equal(plain.pages_host(), dw.pages_host())
        assert dw.shape.num_sdpa_map_task_templates <= dw.meta.num_workers + 32
        del plain
    got = dw.output_f32().reshape(32, w.num_q_heads * w.head_dim)
    pages = dw.pages_host()
    order = np.argsort(w.context_lens)
    picks = [int(order[0]), int(order[16]), int(order[-1])]
    dt = oracle_dtype(oracle, w)
    exp = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout_tuple(w),
                           w.layer, w.req_slots[picks], w.token_indices[picks], np.arange(4, dtype=np.uint32),
                           w.q.reshape(32, -1)[picks].reshape(-1), pages, w.page_ids, num_threads=16)
    assert_outputs_close(got[picks].reshape(-1), exp, "C2 sampled")


def test_long_context_with_large_keys(psi, oracle, device):
    """C3's geometry (16 Q / 2 KV, D=256, bf16) with K outliers of 8 sigma at rate 1e-4, partitions
    from 4096 down to 256 tokens, at 16384 tokens per sequence (the oracle's reach)."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(3, [16384, 16384], 16, 2, 256, psi.Dtype.Bfloat16, 16, outlier_rate=1e-4, outlier_sigma=8.0)
    first = None
    for partition in (4096, 512, 256):
        stats, dw = run_and_check(psi, oracle, device, w, f"long ctx partition {partition}",
                                  partition_tokens=partition, check_rounded=False)
        out = dw.output_f32()
        if first is None:
            first = out
        assert np.abs(out - first).max() < 2e-5


def test_c3_full_length_split_invariance(psi, device):
    """4 x 131072 tokens (1.07 GB of K/V), 32 vs 256 partitions per sequence."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(33, [131072] * 4, 16, 2, 256, psi.Dtype.Bfloat16, 16, host_pages=False)
    outs = []
    for partition in (4096, 512):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True)
        dw.step()
        outs.append(dw.output_f32())
        del dw
    assert np.isfinite(outs[0]).all()
    assert np.abs(outs[0] - outs[1]).max() < 2e-5


def test_verify_full_batch_split_and_placement(psi, device):
    """C4's batch (64 sequences, contexts 2048..16384, 2 tokens each): partition invariance of the
    multi-query kernels at full size."""
    wl = importlib_workloads(psi)
    ctx = wl.config_c2_context_lens(4, 64, 2048, 16384) + 2
    w = wl.make_workload(4, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=2, host_pages=False)
    outs = []
    for partition in (512, 4096):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True)
        assert dw.variant.is_tiled()
        dw.step()
        outs.append(dw.output_f32())
        del dw
    assert np.isfinite(outs[0]).all()
    assert np.abs(outs[0] - outs[1]).max() < 2e-5


def test_c5_prefill_chunk_full_size(psi, oracle, device):
    """C5's chunk: 2048 new tokens on a 4096-token prefix, 24 Q / 4 KV heads.  The row-group map and
    the plain multi-query map agree to rounding on the whole chunk, partition lengths do not matter,
    and sampled query tokens (first, a partition boundary, middle, last) match the scalar oracle run
    on the device's own pages."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(5, [4096 + 2048], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=2048, host_pages=False)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, 6)
    outs = {}
    for name, partition, grouped in (("grouped 2048", 2048, True), ("grouped 512", 512, True), ("plain 2048", 2048, False)):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True, grouped=grouped, variant=variant)
        assert (dw.meta.num_row_groups > 0) == grouped
        dw.step()
        outs[name] = dw.output_f32().reshape(2048, -1)
        if name == "grouped 2048":
            pages = dw.pages_host()
        del dw
    assert np.isfinite(outs["grouped 2048"]).all()
    assert np.abs(outs["grouped 2048"] - outs["grouped 512"]).max() < 1e-4
    assert np.abs(outs["grouped 2048"] - outs["plain 2048"]).max() < 1e-4
    picks = np.array([0, 1, 511, 512, 1023, 2040, 2047])
    dt = oracle_dtype(oracle, w)
    exp = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout_tuple(w),
                           w.layer, np.repeat(w.req_slots, len(picks)), (w.token_indices[0] + picks).astype(np.uint32),
                           np.arange(len(picks) + 1, dtype=np.uint32), w.q.reshape(2048, -1)[picks].reshape(-1), pages,
                           w.page_ids, num_threads=16)
    assert_outputs_close(outs["grouped 2048"][picks].reshape(-1), exp, "C5 chunk sampled")


def test_c5_decode_batch_full_size(psi, device):
    """C5's decode side: 128 sequences with contexts 512..32768 (about 8.7 GB of K/V), split-count
    invariance between 512- and 4096-token partitions."""
    wl = importlib_workloads(psi)
    ctx = wl.config_c2_context_lens(55, 128, 512, 32768)
    w = wl.make_workload(55, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, host_pages=False)
    outs = []
    for partition in (512, 4096):
        dw = wl.DeviceWorkload(device, w, partition_tokens=partition, f32_output=True)
        dw.step()
        outs.append(dw.output_f32())
        del dw
    assert np.isfinite(outs[0]).all()
    assert np.abs(outs[0] - outs[1]).max() < 2e-5
