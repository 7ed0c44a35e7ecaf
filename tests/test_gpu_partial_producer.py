"""A second producer of partial results: each token's split list ends in a row the map skips (all fields
0xFFFFFFFF), another attention task fills that row, and the combine merges it with the history rows.  This is
how the reference's block attention joins the SingleQ reduce (metal/gqa_block_sdpa.metal:47-76 writes the slot,
metal/gqa_split_kv_single_q_map.metal:49-53 leaves it alone; the split table is laid out as in
crates/inference-executor-metal/src/attn/dspark/metadata.rs:172-212).

Here the other producer is numpy: it attends the last `block` keys of each context in f64 and hands over
(exp sum, max logit, normalised output) in the reference's form.  Expected: softmax attention over the whole
context -- the closed form the merge must reproduce -- from the CPU oracle on the same pages, plus an f64 merge
that rounds the producer's output through the IO dtype exactly as the hand-over does."""
import ctypes

import numpy as np
import pytest

from parity_util import assert_outputs_close, importlib_workloads, layout_tuple, oracle_dtype, oracle_step

pytestmark = pytest.mark.gpu

SENTINEL = 0xFFFFFFFF


def _dspark_like_plan(context_lens, blocks, partition):
    """Per token: history rows of `partition` keys over [0, ctx - block), then the reserved row."""
    rows, cu, slots = [], [0], []
    for t, (ctx, block) in enumerate(zip(context_lens, blocks)):
        history = int(ctx) - int(block)
        for begin in range(0, history, partition):
            rows.append((t, begin, min(begin + partition, history)))
        slots.append(len(rows))
        rows.append((SENTINEL,) * 3)
        cu.append(len(rows))
    active = len(rows)
    total = 1 << (active - 1).bit_length()
    rows += [(SENTINEL,) * 3] * (total - active)
    return (np.asarray(rows, np.uint32).reshape(-1), np.asarray(cu, np.uint32), np.asarray(slots, np.uint32), active,
            total)


@pytest.mark.parametrize("dtype_name,longest_first", [("Bfloat16", False), ("Bfloat16", True), ("Float16", False),
                                                       ("Float32", True)])
def test_reserved_row_filled_by_another_producer(psi, oracle, device, dtype_name, longest_first):
    import torch

    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    hq, hkv, d = 24, 4, 256
    ctx = [700, 33, 1500, 64, 300, 8]
    blocks = [7, 1, 4, 7, 2, 7]  # the last request's history is a single key
    w = wl.make_workload(131, ctx, hq, hkv, d, dtype, 16)
    odt = oracle_dtype(oracle, w)
    exp_pages, exp_full = oracle_step(oracle, w)
    n = w.num_tokens
    assert n == len(ctx) and (w.context_lens == np.asarray(ctx)).all()

    # the other producer, and the f64 merge of its (rounded) result with the history
    q = oracle.to_f32(w.q, odt).reshape(n, hq, d).astype(np.float64)
    sums = np.zeros((n, hq), np.float32)
    maxes = np.zeros((n, hq), np.float32)
    outs = np.zeros((n, hq, d), np.float32)
    merged = np.zeros((n, hq, d))
    group = hq // hkv
    for t in range(n):
        k, v = oracle.gather_context(exp_pages, w.page_ids, int(w.req_slots[t]), w.layer, ctx[t], layout_tuple(w),
                                     hkv, d, w.page_bytes, odt)
        k, v = k.reshape(ctx[t], hkv, d).astype(np.float64), v.reshape(ctx[t], hkv, d).astype(np.float64)
        cut = ctx[t] - blocks[t]
        for h in range(hq):
            logits = (k[:, h // group] @ q[t, h]) * w.scale
            m_b = logits[cut:].max()
            p_b = np.exp(logits[cut:] - m_b)
            sums[t, h], maxes[t, h] = p_b.sum(), m_b
            outs[t, h] = (p_b @ v[cut:, h // group]) / p_b.sum()
            handed = oracle.to_f32(oracle.from_f32(outs[t, h], odt), odt).astype(np.float64)
            m_h = logits[:cut].max()
            p_h = np.exp(logits[:cut] - m_h)
            top = max(m_h, float(maxes[t, h]))
            w_h, w_b = np.exp(m_h - top), np.exp(float(maxes[t, h]) - top) * float(sums[t, h])
            merged[t, h] = (w_h * (p_h @ v[:cut, h // group]) + w_b * handed) / (w_h * p_h.sum() + w_b)

    splits, cu, slots, active, total = _dspark_like_plan(ctx, blocks, 256)
    row_index = None
    if longest_first:
        row_index = np.arange(total, dtype=np.uint32)
        u32p = ctypes.POINTER(ctypes.c_uint32)
        lib = device.lib
        assert lib.psi_hip_split_kv_order_longest_first(splits.ctypes.data_as(u32p), active,
                                                        row_index.ctypes.data_as(u32p)) == 0
        assert (splits.reshape(-1, 3)[:3, 2] - splits.reshape(-1, 3)[:3, 1] == 256).all()

    dw = wl.DeviceWorkload(device, w, partition_tokens=256, f32_output=True)  # arena, table, inputs, append
    kshape = psi.GQASplitKVSingleQShape(n, total)
    kernels = psi.GQASplitKVSingleQKernels(device, dw.cfg, kshape)
    scratch = psi.GQASplitKVSingleQScratch(device, dw.cfg, kshape)
    scratch.buffer.view(torch.int32).fill_(0x7FC00000)  # NaN everywhere: an unfilled row would poison the merge
    d_splits, d_cu, d_slots = (device.from_numpy(a) for a in (splits, cu, slots))
    d_rows = device.from_numpy(row_index) if row_index is not None else None
    d_sums, d_maxes = device.from_numpy(sums.reshape(-1)), device.from_numpy(maxes.reshape(-1))
    d_outs = device.from_numpy(oracle.from_f32(outs.reshape(-1), odt))
    out = torch.zeros(n * hq * d, dtype=torch.float32, device=device.torch_device)

    dw.append()
    kernels.invoke_map_bucketed(dw.q, dw.pages, dw.meta.d_req_slots, dw.page_ids, d_splits, scratch, w.layer, n,
                                active)
    kernels.invoke_store_partials(scratch, d_slots, d_sums, d_maxes, d_outs, n, partial_row_index=d_rows)
    device.f32_output(True)
    try:
        kernels.invoke_reduce_bucketed(scratch, d_cu, out, n, partial_row_index=d_rows)
    finally:
        device.f32_output(False)
    device.sync()
    got = out.cpu().numpy().reshape(n, hq, d)
    assert_outputs_close(got, merged, f"{dtype_name} merge with the handed-over rows")
    if dtype_name == "Float32":  # nothing is rounded on the way: the merge is attention over the whole context
        assert_outputs_close(got, exp_full, "whole-context attention")
    else:
        full = np.asarray(exp_full, np.float64).reshape(n, hq, d)
        assert np.abs(got - full).max() < 8e-3  # the hand-over rounds the block's output to the IO dtype


def test_tokens_without_a_reserved_row_and_empty_results(psi, oracle, device):
    """slot_rows[t] >= the split capacity: nothing is stored for the token.  A result with max = -inf (no
    visible key) enters as an empty row and the combine ignores it."""
    import torch

    wl = importlib_workloads(psi)
    hq, hkv, d = 24, 4, 256
    ctx = [100, 260]
    w = wl.make_workload(137, ctx, hq, hkv, d, psi.Dtype.Bfloat16, 16)
    odt = oracle_dtype(oracle, w)
    _, exp_full = oracle_step(oracle, w)
    n = 2
    # token 0: plain rows only; token 1: its rows, then a reserved row that receives an empty result
    rows = [(0, 0, 100), (1, 0, 256), (1, 256, 260), (SENTINEL,) * 3]
    splits = np.asarray(rows, np.uint32).reshape(-1)
    cu = np.asarray([0, 1, 4], np.uint32)
    slots = np.asarray([SENTINEL, 3], np.uint32)
    dw = wl.DeviceWorkload(device, w, partition_tokens=256, f32_output=True)
    kshape = psi.GQASplitKVSingleQShape(n, 4)
    kernels = psi.GQASplitKVSingleQKernels(device, dw.cfg, kshape)
    scratch = psi.GQASplitKVSingleQScratch(device, dw.cfg, kshape)
    scratch.buffer.view(torch.int32).fill_(0x7FC00000)
    sums = np.zeros((n, hq), np.float32)
    maxes = np.full((n, hq), -np.inf, np.float32)
    outs = np.full((n, hq, d), 5.0, np.float32)  # must not leak into the output
    out = torch.zeros(n * hq * d, dtype=torch.float32, device=device.torch_device)
    dw.append()
    kernels.invoke_map_bucketed(dw.q, dw.pages, dw.meta.d_req_slots, dw.page_ids, device.from_numpy(splits), scratch,
                                w.layer, n, 4)
    kernels.invoke_store_partials(scratch, device.from_numpy(slots), device.from_numpy(sums.reshape(-1)),
                                  device.from_numpy(maxes.reshape(-1)),
                                  device.from_numpy(oracle.from_f32(outs.reshape(-1), odt)), n)
    device.f32_output(True)
    try:
        kernels.invoke_reduce_bucketed(scratch, device.from_numpy(cu), out, n)
    finally:
        device.f32_output(False)
    device.sync()
    assert_outputs_close(out.cpu().numpy(), exp_full, "empty reserved row")


def test_store_partials_rejects_bad_arguments(psi, device):
    wl = importlib_workloads(psi)
    w = wl.make_workload(139, [40], 24, 4, 256, psi.Dtype.Bfloat16, 16)
    dw = wl.DeviceWorkload(device, w, partition_tokens=256)
    kernels = psi.GQASplitKVSingleQKernels(device, dw.cfg, psi.GQASplitKVSingleQShape(1, 2))
    scratch = psi.GQASplitKVSingleQScratch(device, dw.cfg, psi.GQASplitKVSingleQShape(1, 2))
    z = device.from_numpy(np.zeros(24 * 256, np.float32))
    slots = device.from_numpy(np.zeros(1, np.uint32))
    with pytest.raises(psi.PsiHipError, match="must not be null"):
        kernels.invoke_store_partials(scratch, None, z, z, z, 1)
    with pytest.raises(psi.PsiHipError, match="active token count exceeds recorded capacity"):
        kernels.invoke_store_partials(scratch, slots, z, z, z, 2)
    small = psi.GQASplitKVSingleQScratch(device, dw.cfg, psi.GQASplitKVSingleQShape(1, 1))
    with pytest.raises(psi.PsiHipError, match="scratch too small"):
        kernels.invoke_store_partials(small, slots, z, z, z, 1)
