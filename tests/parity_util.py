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
                  check_rounded=True, balanced=False, longest_first=False, grouped=False, fused_append=False,
                  **more):
    """GPU layer-step vs oracle: pages bit-exact, f32 outputs within tolerance, io-dtype outputs
    equal to the f32 outputs rounded once."""
    wl = importlib_workloads(psi)
    dw = wl.DeviceWorkload(device, w, partition_tokens=partition_tokens, max_tokens=max_tokens, variant=variant,
                           f32_output=True, balanced=balanced, longest_first=longest_first, grouped=grouped,
                           fused_append=fused_append, **more)
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
                                grouped=grouped, fused_append=fused_append, **more)
        dw2.step()
        rounded = dw2.output_f32()
        ref = oracle.to_f32(oracle.from_f32(got, oracle_dtype(oracle, w)), oracle_dtype(oracle, w))
        assert np.array_equal(rounded, ref), f"{what}: io-dtype output is not the rounded f32 output"
    return stats, dw


def importlib_workloads(psi):
    import importlib

    return importlib.import_module(psi.__name__ + ".workloads")


def oracle_sample(oracle, dw, picks, num_threads=16):
    """Attention of the requests `picks` of a device workload recomputed by the scalar oracle from the device's
    own pages (after the step's append): the picked requests' pages are gathered on the device into a compact
    arena with a table of its own, so that a multi-gigabyte arena never crosses to the host.  Returns the f32
    outputs [tokens of the picks][Hq * D] in pick order."""
    import torch

    w = dw.w
    lay = w.layout
    assert lay.num_page_ids_per_block == 1
    per_slot = lay.num_gqa_layers * lay.num_blocks
    page_elems = 2 * w.num_kv_heads * w.tokens_per_page * w.head_dim
    table = dw.page_ids.cpu().numpy().view(np.uint32)
    ctx = w.context_lens
    counts = [-(-int(ctx[r]) // w.tokens_per_page) for r in picks]
    blocks = max(counts)
    ids, sub_table, cursor = [], np.zeros(len(picks) * blocks, np.uint32), 0
    for i, (r, n) in enumerate(zip(picks, counts)):
        start = int(w.req_slots[r]) * per_slot + w.layer * lay.num_blocks
        ids.append(table[start:start + n].astype(np.int64))
        sub_table[i * blocks:i * blocks + n] = np.arange(cursor, cursor + n)
        cursor += n
    index = torch.from_numpy(np.concatenate(ids)).to(dw.pages.device)
    sub_pages = dw.pages.view(w.num_pages, page_elems).index_select(0, index)
    dw.device.sync()
    if sub_pages.dtype in (torch.bfloat16, torch.float16):
        sub_pages = sub_pages.view(torch.int16).cpu().numpy().view(np.uint16)
    else:
        sub_pages = sub_pages.cpu().numpy()
    q_lens = np.diff(w.cu_tokens)
    rows = np.concatenate([np.arange(w.cu_tokens[r], w.cu_tokens[r + 1]) for r in picks])
    q = w.q.reshape(w.num_tokens, -1)[rows].reshape(-1)
    cu = np.concatenate([[0], np.cumsum([q_lens[r] for r in picks])]).astype(np.uint32)
    out = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, oracle_dtype(oracle, w),
                           (len(picks), 1, blocks, 1), 0, np.arange(len(picks), dtype=np.uint32),
                           w.token_indices[list(picks)], cu, q, sub_pages.reshape(-1), sub_table,
                           num_threads=num_threads)
    return np.asarray(out).reshape(len(rows), -1), rows


def assert_appended_lines(dw):
    """Every K / V line of this step's new tokens sits in its page slot, bit for bit (checked on the device:
    the arena does not cross to the host)."""
    import torch

    w = dw.w
    lay = w.layout
    assert lay.num_page_ids_per_block == 1
    per_slot = lay.num_gqa_layers * lay.num_blocks
    q_lens = np.diff(w.cu_tokens)
    slots = np.repeat(w.req_slots, q_lens).astype(np.int64)
    pos = np.concatenate([w.token_indices[r] + np.arange(n) for r, n in enumerate(q_lens)]).astype(np.int64)
    table = dw.page_ids.cpu().numpy().view(np.uint32).astype(np.int64)
    page = table[slots * per_slot + w.layer * lay.num_blocks + pos // w.tokens_per_page]
    dev = dw.pages.device
    arena = dw.pages.view(w.num_pages, 2, w.num_kv_heads, w.tokens_per_page, w.head_dim)
    page_t, off_t = torch.from_numpy(page).to(dev), torch.from_numpy(pos % w.tokens_per_page).to(dev)
    for kind, flat in ((0, dw.flat_k), (1, dw.flat_v)):
        got = arena[page_t, kind, :, off_t, :]  # [tokens, Hkv, D]
        exp = flat.view(w.num_tokens, w.num_kv_heads, w.head_dim)
        assert torch.equal(got.view(torch.int16) if got.element_size() == 2 else got,
                           exp.view(torch.int16) if exp.element_size() == 2 else exp), "appended lines differ"
