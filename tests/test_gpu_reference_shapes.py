"""The shapes the reference itself times, at full size against the CPU oracle (they are small enough for it):

  * its Criterion bench of the decode kernels: 32 Q / 8 KV heads, head_dim 128, bf16, 16-token pages, one request
    with context 128 / 1024 / 2048 / 4096, and the ragged batch 7 x 128 + 1 x 4096
    (crates/inference-backend-metal/benches/gqa/split_kv.rs:19-27,44);
  * the eight-row GQA diagnostic behind its published 0.319 ms: 40 Q / 8 KV heads, head_dim 128, 32 KiB pages of
    eight tokens, one request with eight new tokens on 128 cached ones (docs/qwen3_dspark_design_draft.md:1453-1477);
  * the same geometry as a prefill chunk through the row-group map (the (128, 8) TiledQ profile of
    crates/inference-backend-metal/src/components/gqa_split_kv_tiled_q.rs:66-76).
Pages bit-exact, outputs within 2e-3 max-abs / 1e-3 relative RMS, through the launch modes `bench.py` uses."""
import pytest

from parity_util import importlib_workloads, run_and_check

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("ctxs", [[128], [1024], [2048], [4096], [128] * 7 + [4096]],
                         ids=["ctx128", "ctx1024", "ctx2048", "ctx4096", "ragged-7x128-1x4096"])
@pytest.mark.parametrize("how", [dict(), dict(balanced=True, fused_append=True)], ids=["row per workgroup", "bench default"])
def test_criterion_decode_shapes(psi, oracle, device, ctxs, how):
    wl = importlib_workloads(psi)
    w = wl.make_workload(8, ctxs, 32, 8, 128, psi.Dtype.Bfloat16, 16)
    stats, dw = run_and_check(psi, oracle, device, w, f"criterion {ctxs}", partition_tokens=512, **how)
    assert not dw.variant.is_tiled()
    print("criterion", ctxs[-1], len(ctxs), "max_abs %.3e rel_rms %.3e" % stats)


@pytest.mark.parametrize("balanced", [False, True])
def test_eight_row_tiled_q_diagnostic_shape(psi, oracle, device, balanced):
    wl = importlib_workloads(psi)
    w = wl.make_workload(7, [128 + 8], 40, 8, 128, psi.Dtype.Bfloat16, 8, q_lens=8)
    assert w.page_bytes == 32 * 1024
    stats, dw = run_and_check(psi, oracle, device, w, "eight rows on 128", partition_tokens=512, balanced=balanced,
                              variant=psi.GQASplitKVVariant.TiledQ(8, 16, 5))
    assert dw.variant.is_tiled() and dw.variant.q_head_tile_size == 5
    print("eight-row max_abs %.3e rel_rms %.3e" % stats)


@pytest.mark.parametrize("hq", [40, 32])
def test_prefill_chunk_at_the_references_geometry(psi, oracle, device, hq):
    """A 300-token chunk on 900 cached tokens, head_dim 128 on 8-token pages, 5 and 4 query heads per KV head."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(9, [1200, 77], hq, 8, 128, psi.Dtype.Bfloat16, 8, q_lens=[300, 3])
    stats, dw = run_and_check(psi, oracle, device, w, f"chunk {hq}/8/128 P=8", partition_tokens=512, max_tokens=512,
                              grouped=True, variant=psi.GQASplitKVVariant.TiledQ(8, 16, hq // 8))
    assert dw.grouped and dw.meta.num_row_groups > 0
    print("chunk d128 p8 max_abs %.3e rel_rms %.3e" % stats)
