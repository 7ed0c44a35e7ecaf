"""Shared helpers of the GPU parity tests: run one layer-step through the C ABI and check it
against the CPU oracle on the same inputs."""
import numpy as np

# Output tolerance of the path against the f32-accumulating scalar oracle.
MAX_ABS_TOL = 2e-3
REL_RMS_TOL = 1e-3


def oracle_dtype(oracle, w):
    return {0: oracle.F32, 1: oracle.BF16, 2: oracle.F16}[int(w.dtype)]


def layout_tuple(w):
    l = w.layout
    return (l.num_req_slots, l.num_gqa_layers, l.num_blocks, l.num_page_ids_per_block)


def oracle_step(oracle, w, num_threads=8):
    """Append + attention on the CPU.  Returns (pages after the append, f32 outputs)."""
    pages = w.pages.copy()
    flat_slots = np.repeat(w.req_slots, np.diff(w.cu_tokens))
    flat_pos = np.concatenate([w.token_indices[r] + np.arange(n, dtype=np.uint32)
                               for r, n in enumerate(np.diff(w.cu_tokens))]).astype(np.uint32)
    dt = oracle_dtype(oracle, w)
    oracle.kv_page_write(pages, w.flat_k, w.flat_v, flat_slots, flat_pos, w.page_ids, w.num_tokens, w.layer,
                         layout_tuple(w), w.num_kv_heads, w.head_dim, w.page_bytes, dt)
    out = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout_tuple(w),
                           w.layer, w.req_slots, w.token_indices, w.cu_tokens, w.q, pages, w.page_ids,
                           num_threads=num_threads)
    return pages, out


def assert_outputs_close(actual, expected, what=""):
    actual = np.asarray(actual, dtype=np.float64).ravel()
    expected = np.asarray(expected, dtype=np.float64).ravel()
    assert actual.shape == expected.shape
    assert np.isfinite(actual).all(), f"{what}: non-finite outputs"
    max_abs = np.abs(actual - expected).max()
    rel_rms = np.sqrt(((actual - expected) ** 2).sum() / max((expected ** 2).sum(), 1e-30))
    assert max_abs <= MAX_ABS_TOL, f"{what}: max-abs {max_abs:.3e} > {MAX_ABS_TOL}"
    assert rel_rms <= REL_RMS_TOL, f"{what}: rel-RMS {rel_rms:.3e} > {REL_RMS_TOL}"
    return max_abs, rel_rms


def run_and_check(psi, oracle, device, w, what, partition_tokens=None, max_tokens=None, variant=None,
                  check_rounded=True, balanced=False, longest_first=False, grouped=False, fused_append=False):
    """GPU layer-step vs oracle: pages bit-exact, f32 outputs within tolerance, io-dtype outputs
    equal to the f32 outputs rounded once."""
    wl = importlib_workloads(psi)
    dw = wl.DeviceWorkload(device, w, partition_tokens=partition_tokens, max_tokens=max_tokens, variant=variant,
                           f32_output=True, balanced=balanced, longest_first=longest_first, grouped=grouped,
                           fused_append=fused_append)
    dw.step()
    got = dw.output_f32()
    exp_pages, exp = oracle_step(oracle, w)
    got_pages = dw.pages_host().reshape(exp_pages.shape)
    if exp_pages.dtype == np.float32:
        assert np.array_equal(got_pages.view(np.uint32), exp_pages.view(np.uint32)), f"{what}: pages differ"
    else:
        assert np.array_equal(got_pages, exp_pages), f"{what}: pages differ"
    stats = assert_outputs_close(got, exp, what)
    if check_rounded and int(w.dtype) != 0:
        dw2 = wl.DeviceWorkload(device, w, partition_tokens=partition_tokens, max_tokens=max_tokens,
                                variant=variant, f32_output=False, balanced=balanced, longest_first=longest_first,
                                grouped=grouped, fused_append=fused_append)
        dw2.step()
        rounded = dw2.output_f32()
        ref = oracle.to_f32(oracle.from_f32(got, oracle_dtype(oracle, w)), oracle_dtype(oracle, w))
        assert np.array_equal(rounded, ref), f"{what}: io-dtype output is not the rounded f32 output"
    return stats, dw


def importlib_workloads(psi):
    import importlib

    return importlib.import_module(psi.__name__ + ".workloads")
