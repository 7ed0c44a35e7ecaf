"""psi_hip_gqa_layer_record_static_scratch: the layer entry for callers that cannot allocate, with the partial
states in the library's built-in device array.  Called through the C ABI on two batches in a row, the second
smaller than the first, and compared bit for bit with psi_hip_gqa_layer_record on a caller-owned buffer."""
import numpy as np
import pytest

from parity_util import assert_outputs_close, importlib_workloads, oracle_step

pytestmark = pytest.mark.gpu


def _layer_step(psi, device, w, static, how):
    """(arena, f32 output) of one decode / verify layer-step through either entry point."""
    import torch

    wl = importlib_workloads(psi)
    dw = wl.DeviceWorkload(device, w, partition_tokens=512, f32_output=True, **how)
    inp = dw.layer_input()
    if static:
        class _NoBuffer:  # the caller passes inputs and outputs only
            qgkv = None
            q_norm_rope = None
            sdpa_partial = None
            attention_output = dw.output

        inp.scratch = _NoBuffer
    free_before = torch.cuda.mem_get_info()[0]
    device.f32_output(True)
    try:
        (dw.gqa.record_static_scratch if static else dw.gqa.record)(inp)
    finally:
        device.f32_output(False)
    device.sync()
    assert not static or torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated inside the call"
    return dw.pages_host().copy(), dw.output_f32()


@pytest.mark.parametrize("q_len,how", [(1, dict(balanced=True, fused_append=True)), (1, dict(fused_append=True)),
                                       (3, dict(balanced=True))])
def test_two_calls_in_a_row_match_the_allocating_entry(psi, oracle, device, q_len, how):
    wl = importlib_workloads(psi)
    big = wl.make_workload(151, [3000, 17, 1025, 2048, 700, 513, 90], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    small = wl.make_workload(152, [600, 47], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    for w in (big, small):  # the second call finds the first call's partial states in the buffer
        exp_pages, exp_out = _layer_step(psi, device, w, False, how)
        got_pages, got_out = _layer_step(psi, device, w, True, how)
        assert np.array_equal(got_pages, exp_pages)
        assert np.array_equal(got_out, exp_out), "static-scratch entry differs from the allocating entry"
        assert_outputs_close(got_out, oracle_step(oracle, w)[1], "static scratch vs oracle")


def test_sizes_beyond_the_built_in_buffer_are_rejected(psi, device):
    wl = importlib_workloads(psi)
    gqa_mod = importlib_gqa(psi)
    # 16-token partitions over 40000 tokens: 2500 rows x 24 heads x 258 floats = 62 MB of partial states
    w = wl.make_workload(153, [40000], 24, 4, 256, psi.Dtype.Bfloat16, 16, host_pages=False)
    dw = wl.DeviceWorkload(device, w, partition_tokens=16, variant=psi.GQASplitKVVariant.SingleQ(16, 256, 6),
                           fused_append=True)
    assert dw.scratch.bytes > gqa_mod.STATIC_SCRATCH_BYTES
    with pytest.raises(psi.PsiHipError) as err:
        dw.gqa.record_static_scratch(dw.layer_input())
    assert "built-in scratch holds" in str(err.value) and err.value.code == -1


def importlib_gqa(psi):
    import importlib

    return importlib.import_module(psi.__name__ + ".gqa")
