"""What a kernel could not compute reaches the host: the device error words of a context.

Two conditions, neither of which the reference has (its Metal kernels have no waits between simdgroups, and they
multiply V in the storage type):
  * a wave's bounded wait on another wave of its workgroup runs out (multi-query map; the prefill-chunk map's
    waves meet at barriers only).  The test forces it from the host (the loading waves never say that a tile has
    landed), so that every kernel still runs to its end;
  * the prefill-chunk map multiplies V as f16 and meets a bf16 value that f16 cannot hold.
Either way `sync()` must fail, `take_device_error()` must name the condition and clear it, no stale or half
computed row may reach the output, and the same batch must then run clean."""
import importlib

import numpy as np
import pytest

from parity_util import assert_outputs_close, importlib_workloads, oracle_step

pytestmark = pytest.mark.gpu


def _lib(psi):
    return importlib.import_module(psi.__name__ + "._lib")


def _verify_workload(psi, wl):
    return wl.make_workload(91, [700, 333, 64, 1200], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[3, 4, 2, 4])


def _chunk_workload(psi, wl, seed=92):
    return wl.make_workload(seed, [650, 40], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[150, 2])


def test_a_wait_that_runs_out_is_reported(psi, oracle, device):
    import torch

    L = _lib(psi)
    wl = importlib_workloads(psi)
    kind = "multi-query"
    w = _verify_workload(psi, wl)
    dw = wl.DeviceWorkload(device, w, f32_output=True, max_tokens=64)
    assert dw.variant.is_tiled()
    _, exp = oracle_step(oracle, w)
    assert device.take_device_error() == 0
    dw.scratch.buffer.view(torch.float32).fill_(7.0)  # stale partial states: finite, plausible
    device.mute_loaders(True)
    try:
        dw.step()
        with pytest.raises(psi.PsiHipError, match="bounded wait"):
            device.sync()
        assert device.take_device_error() & L.DEVICE_ERR_WAIT_GAVE_UP
    finally:
        device.mute_loaders(False)
    device.sync()  # taken: clean again
    got = dw.output_f32().reshape(w.num_tokens, -1)
    assert np.isfinite(got).all()
    # a row either came through whole (its waves never had to wait) or is an empty state: an output row is the
    # oracle's, or a merge of fewer partitions of it - never the stale 7.0s
    exp = exp.reshape(w.num_tokens, -1)
    assert np.abs(got).max() < 6.5 and not (got == 7.0).any()  # V is N(0, 1): no convex combination reaches 6.5
    # the same batch at the default limit
    dw.step()
    assert_outputs_close(dw.output_f32(), exp, f"{kind} after the error was taken")
    assert device.take_device_error() == 0


def test_the_chunk_map_has_no_waits_to_run_out(psi, oracle, device):
    """Its waves meet at workgroup barriers only: the harness switch that starves the multi-query map's waits leaves
    the prefill-chunk map's results as they are, and no error is reported."""
    wl = importlib_workloads(psi)
    w = _chunk_workload(psi, wl)
    _, exp = oracle_step(oracle, w)
    dw = wl.DeviceWorkload(device, w, partition_tokens=256, max_tokens=512, grouped=True, f32_output=True)
    assert dw.grouped
    device.mute_loaders(True)
    try:
        dw.step()
        got = dw.output_f32()
        assert device.take_device_error() == 0
    finally:
        device.mute_loaders(False)
    assert_outputs_close(got, exp, "chunk map under the harness switch")


def _set_v(w, psi, wl, request, position, kv_head, dim, value):
    """Overwrites one V element of the cached history (a host-side arena)."""
    lay = w.layout
    per_slot = lay.num_gqa_layers * lay.num_blocks * lay.num_page_ids_per_block
    page = w.page_ids[int(w.req_slots[request]) * per_slot + position // w.tokens_per_page]
    w.pages[page, 1, kv_head, position % w.tokens_per_page, dim] = wl.to_storage(np.float32([value]), w.dtype)[0]


def test_chunk_map_reports_v_beyond_f16(psi, oracle, device):
    """A bf16 cache may hold |v| > 65504; f16 cannot.  The chunk map must say so instead of clamping, and the
    multi-query map, which multiplies V as bf16, must give the oracle's result on the same batch."""
    L = _lib(psi)
    wl = importlib_workloads(psi)
    w = _chunk_workload(psi, wl, seed=93)
    _set_v(w, psi, wl, 0, 37, 1, 5, 1.0e5)
    _set_v(w, psi, wl, 0, 301, 2, 200, -3.0e7)
    _, exp = oracle_step(oracle, w)
    dw = wl.DeviceWorkload(device, w, partition_tokens=256, max_tokens=512, grouped=True, f32_output=True)
    assert dw.grouped
    dw.step()
    with pytest.raises(psi.PsiHipError, match="f16 range"):
        device.sync()
    assert device.take_device_error() == L.DEVICE_ERR_V_RANGE
    # the route the error message names
    plain = wl.DeviceWorkload(device, w, partition_tokens=256, max_tokens=512, grouped=False, f32_output=True)
    plain.step()
    got = plain.output_f32()
    assert device.take_device_error() == 0
    # outputs now reach 3e7 / context: the bar applies relative to that size
    exp = np.asarray(exp, dtype=np.float64).ravel()
    err = np.abs(got.ravel() - exp)
    assert np.sqrt((err ** 2).sum() / (exp ** 2).sum()) <= 1e-3
    assert (err <= 2e-3 * np.maximum(1.0, np.abs(exp))).all()


def test_wide_tiles_report_v_beyond_f16_and_the_generic_kernels_take_it(psi, oracle, device):
    """Tiles of more than 48 query columns (8 tokens x 8 heads per KV head) go to the row-group kernel through every
    entry point, so a V element beyond f16 is reported there too; the shape-generic kernels, which multiply in f32,
    give the oracle's result on the same batch."""
    L = _lib(psi)
    wl = importlib_workloads(psi)
    w = wl.make_workload(95, [700, 40, 1300], 16, 2, 256, psi.Dtype.Bfloat16, 16, q_lens=8, host_pages=True)
    _set_v(w, psi, wl, 0, 37, 1, 5, 1.0e5)
    _set_v(w, psi, wl, 2, 901, 0, 200, -3.0e7)
    _, exp = oracle_step(oracle, w)
    for how in (dict(balanced=True), dict()):
        dw = wl.DeviceWorkload(device, w, partition_tokens=256, max_tokens=64, f32_output=True, **how)
        dw.step()
        with pytest.raises(psi.PsiHipError, match="f16 range"):
            device.sync()
        assert device.take_device_error() == L.DEVICE_ERR_V_RANGE
    device.force_generic(True)
    try:
        slow = wl.DeviceWorkload(device, w, partition_tokens=256, max_tokens=64, f32_output=True)
        slow.step()
        got = slow.output_f32()
        assert device.take_device_error() == 0
    finally:
        device.force_generic(False)
    exp = np.asarray(exp, dtype=np.float64).ravel()
    err = np.abs(got.ravel() - exp)
    assert np.sqrt((err ** 2).sum() / (exp ** 2).sum()) <= 1e-3
    assert (err <= 2e-3 * np.maximum(1.0, np.abs(exp))).all()


def test_chunk_map_keeps_small_v(psi, oracle, device):
    """V magnitudes around 1e-6 lie below f16's normal range (6.1e-5): as f16 they keep an absolute spacing of
    6e-8, so each output element, a convex combination of them, is within 3e-8 of the oracle's - far inside the
    absolute bar, which is the one that applies to outputs of that size - and no error is reported."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(94, [650, 40], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[150, 2])
    tiny = wl.to_storage((np.random.default_rng(5).standard_normal(w.pages[:, 1].shape) * 1e-6).astype(np.float32),
                         w.dtype)
    w.pages[:, 1] = tiny.reshape(w.pages[:, 1].shape)
    w.flat_v[...] = wl.to_storage((np.random.default_rng(6).standard_normal(w.flat_v.shape) * 1e-6).astype(np.float32),
                                  w.dtype)
    _, exp = oracle_step(oracle, w)
    dw = wl.DeviceWorkload(device, w, partition_tokens=256, max_tokens=512, grouped=True, f32_output=True)
    dw.step()
    got = dw.output_f32()
    assert device.take_device_error() == 0
    err = np.abs(got.ravel().astype(np.float64) - np.asarray(exp, dtype=np.float64).ravel())
    assert err.max() <= 4e-8, err.max()
    assert np.abs(got).max() > 1e-8  # and they are not flushed to zero
