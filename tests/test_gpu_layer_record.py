"""The attention layer behind one call (`GQA.record`, psi_hip_gqa_layer_record) and the per-bucket program
cache (`GQAReplayCache`, psi_hip_gqa_replay_cache_*), against the CPU oracle.

The oracle pipeline for a gated layer is the reference's operator sequence restated on the CPU:
qgkv split -> RMSNorm + RoPE of q and k -> KV page write -> paged attention -> sigmoid gate."""
import dataclasses

import numpy as np
import pytest

from parity_util import assert_outputs_close, importlib_workloads, layout_tuple, oracle_dtype, oracle_step

pytestmark = pytest.mark.gpu

ROPE_DIM, EPS, THETA = 64, 1e-6, 1e7


def _layer(psi, device, w, gated):
    core = psi.GQACore(0, w.num_q_heads * w.head_dim, w.head_dim, w.num_q_heads, w.num_kv_heads, w.scale)
    return psi.GQA.new(device, core, psi.GQAMetalConfig(w.page_bytes, ROPE_DIM, EPS, THETA, io_dtype=w.dtype), gated)


def _assert_rows_close(oracle, got_bits, exp_bits, d, what):
    """2-byte rows after RMSNorm + RoPE: at most 2 % of the elements differ, and none by more than one unit in the
    last place of the row's largest element (a last-place flip of a large element before the rotation shows as
    several last places of a small rotated one)."""
    diff = got_bits != exp_bits
    assert diff.mean() <= 0.02, f"{what}: {diff.mean():.4f} of the elements differ"
    got = oracle.to_f32(got_bits.reshape(-1), oracle.BF16).reshape(-1, d)
    exp = oracle.to_f32(exp_bits.reshape(-1), oracle.BF16).reshape(-1, d)
    bound = np.abs(exp).max(axis=1, keepdims=True) * 2.0 ** -7
    assert (np.abs(got - exp) <= bound).all(), what


def _oracle_layer(oracle, w, qgkv, wq, wk, gated):
    """(pages after the append, f32 attention output, gates or None, normalised q, normalised k) on the CPU."""
    hq, hkv, d, t = w.num_q_heads, w.num_kv_heads, w.head_dim, w.num_tokens
    dt = oracle_dtype(oracle, w)
    if gated:
        q, g, k, v = oracle.qgkv_split(qgkv, t, hq, hkv, d, dt)
    else:
        rows = qgkv.reshape(t, (hq + 2 * hkv) * d)
        q, k, v = (rows[:, :hq * d].reshape(-1).copy(), rows[:, hq * d:(hq + hkv) * d].reshape(-1).copy(),
                   rows[:, (hq + hkv) * d:].reshape(-1).copy())
        g = None
    q_lens = np.diff(w.cu_tokens)
    flat_pos = np.concatenate([w.token_indices[r] + np.arange(n, dtype=np.uint32) for r, n in enumerate(q_lens)])
    inv, factor, _ = oracle.rope_parameters(ROPE_DIM, THETA)
    qn = oracle.rms_norm_rope(q, wq, flat_pos, hq, d, ROPE_DIM, EPS, inv, factor, dt)
    kn = oracle.rms_norm_rope(k, wk, flat_pos, hkv, d, ROPE_DIM, EPS, inv, factor, dt)
    pages = w.pages.copy()
    flat_slots = np.repeat(w.req_slots, q_lens)
    oracle.kv_page_write(pages, kn, v, flat_slots, flat_pos.astype(np.uint32), w.page_ids, t, w.layer, layout_tuple(w),
                         hkv, d, w.page_bytes, dt)
    attn = oracle.paged_gqa(hq, hkv, d, w.scale, w.page_bytes, dt, layout_tuple(w), w.layer, w.req_slots,
                            w.token_indices, w.cu_tokens, qn, pages, w.page_ids, num_threads=8)
    return pages, attn, g, qn, kn


@pytest.mark.parametrize("gated,q_lens,partition,balanced", [
    (True, 1, 512, True),      # the decode batch of the headline shape as a gated layer, bench-default plan
    (True, 1, None, False),    # the reference's greedy plan, one workgroup per row
    (False, 1, 512, True),     # ungated layer
    (True, 2, 512, True),      # one-draft verify step through the multi-query kernels
    (True, [4, 1, 3, 4, 2, 4], 256, False),
])
def test_layer_from_projection_output_to_layer_output(psi, oracle, device, gated, q_lens, partition, balanced):
    """Raw projection rows in, (gated) attention output out, in one call.  Checked against the CPU pipeline:
    V lines and untouched pages bit-exact, K lines within one unit in the last place on < 2 % of the elements
    (sin / cos implementations differ), f32 outputs within the attention bar of the oracle's attention times the
    exact sigmoid; and bit for bit, arena and 2-byte output, against the same step issued operator by operator
    through the component entry points."""
    import torch

    wl = importlib_workloads(psi)
    ctx = [3000, 17, 1025, 2048, 700, 513]
    w = wl.make_workload(61, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_lens)
    hq, hkv, d, t = w.num_q_heads, w.num_kv_heads, w.head_dim, w.num_tokens
    rng = np.random.default_rng(62)
    width = (2 * (hq + hkv) if gated else hq + 2 * hkv) * d
    qgkv = oracle.from_f32(rng.normal(0, 1, t * width).astype(np.float32), oracle.BF16)
    wq = oracle.from_f32(rng.uniform(0.5, 1.5, d).astype(np.float32), oracle.BF16)
    wk = oracle.from_f32(rng.uniform(0.5, 1.5, d).astype(np.float32), oracle.BF16)
    exp_pages, exp_attn, gates, exp_q, _ = _oracle_layer(oracle, w, qgkv, wq, wk, gated)

    gqa = _layer(psi, device, w, gated)
    splits_cap = sum(-(-c // (partition or 16)) for c in ctx) * (4 if q_lens != 1 else 1) + 8
    meta = psi.GQAMetadataBuffers(device, 64, max_kv_splits=max(splits_cap, 64))
    if partition:
        shape = gqa.prepare_fixed_partition(meta, w.req_slots, w.token_indices, w.cu_tokens, partition, balanced=balanced)
    else:
        shape = gqa.prepare(meta, w.req_slots, w.token_indices, w.cu_tokens)
    assert meta.split_kv_variant().is_tiled() == (q_lens != 1)
    scratch = gqa.new_scratch(shape.num_total_tokens, shape.num_total_sdpa_map_task_templates)
    scratch.qgkv[:t * width].copy_(device.from_numpy(qgkv).view(torch.bfloat16))
    pages = device.from_numpy(w.pages.reshape(-1)).view(torch.bfloat16)
    page_ids = device.from_numpy(w.page_ids)
    weights = psi.GQAWeights(device.from_numpy(wq), device.from_numpy(wk))

    def run(f32_output):
        pages.copy_(device.from_numpy(w.pages.reshape(-1)).view(torch.bfloat16))
        out = torch.zeros(shape.num_total_tokens * hq * d, dtype=torch.float32 if f32_output else torch.bfloat16,
                          device=device.torch_device)
        inp = psi.GQAInput(w.layout, w.layer, meta, psi.GQAKVCacheBindings(pages, page_ids), scratch, weights,
                           psi.GQAReplayMode.Exact if shape.num_tokens == shape.num_total_tokens and
                           shape.num_q_token_tiles == shape.num_total_q_token_tiles else psi.GQAReplayMode.Bucketed,
                           output=out)
        device.f32_output(f32_output)
        try:
            assert gqa.record(inp) is out
        finally:
            device.f32_output(False)
        device.sync()
        return out

    out32 = run(True).cpu().numpy()[:t * hq * d]
    got_pages = pages.view(torch.int16).cpu().numpy().view(np.uint16).reshape(exp_pages.shape)
    # V halves of every page and every page the step does not touch: bit-exact
    assert np.array_equal(got_pages[:, 1], exp_pages[:, 1])
    assert (got_pages[:, 0] != exp_pages[:, 0]).sum() <= 0.02 * t * hkv * d
    _assert_rows_close(oracle, got_pages[:, 0], exp_pages[:, 0], d, "K lines")
    touched = np.zeros(w.num_pages, bool)
    flat_slots = np.repeat(w.req_slots, np.diff(w.cu_tokens))
    flat_pos = np.concatenate([w.token_indices[r] + np.arange(n) for r, n in enumerate(np.diff(w.cu_tokens))])
    per_slot = w.layout.num_blocks * w.layout.num_page_ids_per_block * w.layout.num_gqa_layers
    for slot, pos in zip(flat_slots, flat_pos):
        touched[w.page_ids[int(slot) * per_slot + int(pos) // 16]] = True
    assert np.array_equal(got_pages[~touched], exp_pages[~touched])
    # normalised queries: one unit in the last place on < 2 % of the elements
    got_q = scratch.q_norm_rope.view(torch.int16).cpu().numpy().view(np.uint16)[:t * hq * d]
    _assert_rows_close(oracle, got_q, exp_q, d, "normalised queries")
    expected = exp_attn.reshape(-1).astype(np.float64)
    if gated:
        expected = expected * (1.0 / (1.0 + np.exp(-oracle.to_f32(gates, oracle.BF16).astype(np.float64))))
    assert_outputs_close(out32, expected, "layer record f32 output")

    # the same step, operator by operator (bf16 outputs)
    fused_out = run(False).view(torch.int16).cpu().numpy().copy()
    fused_pages = pages.view(torch.int16).cpu().numpy().copy()
    pages.copy_(device.from_numpy(w.pages.reshape(-1)).view(torch.bfloat16))
    i16 = dict(dtype=torch.int16, device=device.torch_device)
    q, g, k, v = (torch.zeros(t * hq * d, **i16), torch.zeros(t * hq * d, **i16), torch.zeros(t * hkv * d, **i16),
                  torch.zeros(t * hkv * d, **i16))
    src = scratch.qgkv.view(torch.int16)
    if gated:
        psi.GQAQGKVSplitKernel(device, hq, hkv, d, w.dtype).invoke_bucketed(t, src, q, g, k, v, t)
    else:
        rows = src[:t * width].view(t, width)
        q, k, v = (rows[:, :hq * d].reshape(-1).contiguous(), rows[:, hq * d:(hq + hkv) * d].reshape(-1).contiguous(),
                   rows[:, (hq + hkv) * d:].reshape(-1).contiguous())
    qn, kn = torch.zeros_like(q), torch.zeros_like(k)
    psi.RMSNormRopeKernel(device, psi.RMSNormRopeConfig(hq, d, ROPE_DIM, EPS, THETA, w.dtype)).invoke_bucketed(
        t, q, weights.q_norm_weight, meta.d_flat_token_indices, qn, t)
    psi.RMSNormRopeKernel(device, psi.RMSNormRopeConfig(hkv, d, ROPE_DIM, EPS, THETA, w.dtype)).invoke_bucketed(
        t, k, weights.k_norm_weight, meta.d_flat_token_indices, kn, t)
    write = psi.GQAKVPageWrite(device, psi.GQAKVPageWriteConfig(hkv, d, w.page_bytes, w.dtype))
    write.invoke_bucketed(psi.GQAKVPageWriteShape(shape.num_total_tokens, w.layout),
                          psi.GQAKVPageWriteBuffers(pages, kn, v, meta.d_req_slots, meta.d_flat_token_indices, page_ids),
                          t, w.layer)
    variant = meta.split_kv_variant()
    attn = torch.zeros(shape.num_total_tokens * hq * d, **i16)
    if variant.is_tiled():
        cfg = psi.GQASplitKVTiledQConfig(hq, hkv, d, variant.q_head_tile_size, variant.q_token_tile_size,
                                         variant.kv_token_tile_size, w.scale, w.page_bytes, w.dtype, w.layout)
        kshape = psi.GQASplitKVTiledQShape(shape.num_total_tokens, shape.num_total_q_token_tiles,
                                           shape.num_total_sdpa_map_task_templates)
        kernels, part = psi.GQASplitKVTiledQKernels(device, cfg, kshape), psi.GQASplitKVTiledQScratch(device, cfg, kshape)
        kernels.invoke_map_bucketed(qn, pages, meta.d_req_slots, page_ids, meta.d_flat_token_indices,
                                    meta.d_q_token_tiles, meta.d_kv_splits, part, w.layer, shape.num_tokens,
                                    shape.num_q_token_tiles, shape.num_sdpa_map_task_templates,
                                    meta.max_active_q_tile_tokens)
        kernels.invoke_reduce_bucketed(part, meta.d_q_token_tiles, meta.d_cu_kv_splits, attn, shape.num_q_token_tiles)
    else:
        cfg = psi.GQASplitKVSingleQConfig(hq, hkv, d, w.scale, w.page_bytes, w.layout, variant.kv_token_tile_size,
                                          variant.num_threads_per_threadblock, variant.q_head_tile_size, w.dtype)
        kshape = psi.GQASplitKVSingleQShape(shape.num_total_tokens, shape.num_total_sdpa_map_task_templates)
        kernels, part = psi.GQASplitKVSingleQKernels(device, cfg, kshape), psi.GQASplitKVSingleQScratch(device, cfg, kshape)
        kernels.invoke_map_bucketed(qn, pages, meta.d_req_slots, page_ids, meta.d_kv_splits, part, w.layer,
                                    shape.num_tokens, shape.num_sdpa_map_task_templates)
        kernels.invoke_reduce_bucketed(part, meta.d_cu_kv_splits, attn, shape.num_tokens)
    final = attn
    if gated:
        final = torch.zeros_like(attn)
        psi.GQAActivationGateKernel(device, hq, d, w.dtype).invoke_bucketed(shape.num_total_tokens, attn, g, final, t)
    device.sync()
    assert np.array_equal(pages.view(torch.int16).cpu().numpy(), fused_pages)
    # same rows, same order of summation inside a row: the outputs agree bit for bit
    assert np.array_equal(fused_out[:t * hq * d], final.cpu().numpy()[:t * hq * d])


def test_layer_input_validation(psi, device):
    """`GQA::validate_input` / `GQAReplayShape::validate`: exact replay needs active counts equal to the
    capacities, the layer index must lie inside the table, buffers must be there."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(63, [100, 40], 24, 4, 256, psi.Dtype.Bfloat16, 16)
    dw = wl.DeviceWorkload(device, w, partition_tokens=512, fused_append=True)
    inp = dw.layer_input()
    inp.shape = psi.GQAReplayShape(2, 4, 2, 4, 2, 4, True)
    inp.replay_mode = psi.GQAReplayMode.Exact
    with pytest.raises(psi.PsiHipError) as err:
        dw.gqa.record(inp)
    assert "exact replay requires active counts equal" in str(err.value)
    inp.shape, inp.replay_mode = None, psi.GQAReplayMode.Bucketed
    inp.gqa_layer_index = 1
    with pytest.raises(psi.PsiHipError) as err:
        dw.gqa.record(inp)
    assert "page-table index exceeds layer count" in str(err.value)
    inp.gqa_layer_index = 0
    inp.k = None
    with pytest.raises(psi.PsiHipError) as err:
        dw.gqa.record(inp)
    assert "split q / k / v rows" in str(err.value)


@pytest.mark.parametrize("q_len,counts_uploaded", [(1, False), (2, False), (1, True), (2, True)])
def test_replay_cache_serves_buckets_and_matches_oracle(psi, oracle, device, q_len, counts_uploaded):
    """One recorded program per (variant, token / tile / split capacities): batches of 5, 3, 1 and 4 of five
    requests are submitted twice through the cache with the capacities `ReplayBucketPolicy` gives them.  Every
    submission matches the CPU oracle on that batch (pages bit-exact, outputs within the bar), rows beyond the
    active tokens keep their canary, the second round records nothing, and the number of programs equals the
    number of distinct capacity keys.  q_len 2: the multi-query kernels.  counts_uploaded: the active counts reach
    the device with the metadata upload and a submission is the program's launch alone."""
    import torch

    wl = importlib_workloads(psi)
    ctx = [700, 33, 1500, 512, 64]
    w = wl.make_workload(141 + q_len, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    hq, hkv, d = w.num_q_heads, w.num_kv_heads, w.head_dim
    row, kv_row = hq * d, hkv * d
    max_tokens, workers = 16, 8
    gqa = _layer(psi, device, w, gated=False)
    token_policy = psi.ReplayBucketPolicy(max_tokens)
    split_policy = psi.ReplayBucketPolicy(64)
    meta = psi.GQAMetadataBuffers(device, max_tokens, max_kv_splits=64, max_workers=workers)
    scratch = gqa.new_scratch(max_tokens, 64 + workers)
    bf = dict(dtype=torch.bfloat16, device=device.torch_device)
    q, k, v = torch.zeros(max_tokens * row, **bf), torch.zeros(max_tokens * kv_row, **bf), torch.zeros(max_tokens * kv_row, **bf)
    out = torch.zeros(max_tokens * row, dtype=torch.float32, device=device.torch_device)
    pristine = device.from_numpy(w.pages.reshape(-1)).view(torch.bfloat16)
    pages = pristine.clone()
    page_ids = device.from_numpy(w.page_ids)
    side, main = torch.cuda.Stream(), device.stream
    keys = set()
    device.use_stream(side)
    device.f32_output(True)
    try:
        cache = psi.GQAReplayCache(device, gqa)
        for round_ in range(2):
            for picks in ([0, 1, 2, 3, 4], [2, 0, 4], [3], [4, 3, 1, 0]):
                n = len(picks) * q_len
                sub = dataclasses.replace(w, req_slots=w.req_slots[picks], token_indices=w.token_indices[picks],
                                          cu_tokens=np.arange(len(picks) + 1, dtype=np.uint32) * q_len,
                                          q=w.q.reshape(-1, q_len * row)[picks].reshape(-1),
                                          flat_k=w.flat_k.reshape(-1, q_len * kv_row)[picks].reshape(-1),
                                          flat_v=w.flat_v.reshape(-1, q_len * kv_row)[picks].reshape(-1))
                with torch.cuda.stream(side):
                    shape = gqa.prepare_fixed_partition(meta, sub.req_slots, sub.token_indices, sub.cu_tokens, 512,
                                                        balanced=False)
                    shape = meta.balance(workers)
                    caps = psi.GQAReplayShape(
                        shape.num_tokens, token_policy.capacity(shape.num_tokens), shape.num_q_token_tiles,
                        token_policy.capacity(shape.num_q_token_tiles), shape.num_sdpa_map_task_templates,
                        split_policy.capacity(shape.num_sdpa_map_task_templates), True)
                    key = (caps.num_total_tokens, caps.num_total_q_token_tiles, caps.num_total_sdpa_map_task_templates)
                    new_key = key not in keys
                    keys.add(key)
                    for dst, src in ((q, sub.q), (k, sub.flat_k), (v, sub.flat_v)):
                        dst.zero_()
                        dst[:src.size].copy_(device.from_numpy(src).view(torch.bfloat16))
                    pages.copy_(pristine)
                    out.fill_(-768.0)
                    inp = psi.GQAInput(w.layout, w.layer, meta, psi.GQAKVCacheBindings(pages, page_ids), scratch,
                                       q=q, k=k, v=v, output=out, shape=caps, counts_uploaded=counts_uploaded)
                    recorded = cache.submit(inp)
                    side.synchronize()
                assert recorded == new_key and (round_ == 0 or not recorded), (round_, picks)
                exp_pages, exp = oracle_step(oracle, sub)
                got = out.cpu().numpy()
                assert_outputs_close(got[:n * row], exp, f"replay {picks}")
                assert (got[n * row:] == -768.0).all(), "rows beyond the active tokens were written"
                assert np.array_equal(pages.view(torch.int16).cpu().numpy().view(np.uint16).reshape(exp_pages.shape),
                                      exp_pages)
                _ = (out * 2).sum().item()  # eager work of the program between replays
        programs, recordings, replays = cache.stats()
        assert programs == recordings == len(keys) and replays == 8
        cache.close()
    finally:
        device.f32_output(False)
        device.use_stream(main)


def test_prepare_with_bucketed_capacities_feeds_the_replay_cache(psi, oracle, device):
    """The one-call preparation with `bucket_capacities` gives the balanced plan's re-cut rows a bucketed capacity,
    so that decode batches of varying size and length share recorded programs: twelve different batches, far fewer
    recordings, every replay equal to the CPU oracle on its batch."""
    import torch

    wl = importlib_workloads(psi)
    rng = np.random.default_rng(7)
    ctx = rng.integers(30, 2500, size=10).tolist()
    w = wl.make_workload(171, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16)
    hq, hkv, d = w.num_q_heads, w.num_kv_heads, w.head_dim
    row, kv_row = hq * d, hkv * d
    max_tokens, max_splits, workers = 16, 96, 8
    gqa = _layer(psi, device, w, gated=False)
    meta = psi.GQAMetadataBuffers(device, max_tokens, max_kv_splits=max_splits, max_workers=workers)
    scratch = gqa.new_scratch(max_tokens, max_splits + workers)
    bf = dict(dtype=torch.bfloat16, device=device.torch_device)
    q, k, v = torch.zeros(max_tokens * row, **bf), torch.zeros(max_tokens * kv_row, **bf), torch.zeros(max_tokens * kv_row, **bf)
    out = torch.zeros(max_tokens * row, dtype=torch.float32, device=device.torch_device)
    pristine = device.from_numpy(w.pages.reshape(-1)).view(torch.bfloat16)
    pages = pristine.clone()
    page_ids = device.from_numpy(w.page_ids)
    side, main = torch.cuda.Stream(), device.stream
    device.use_stream(side)
    device.f32_output(True)
    batches = 12
    try:
        cache = psi.GQAReplayCache(device, gqa)
        for b in range(batches):
            picks = sorted(rng.choice(len(ctx), size=int(rng.integers(1, len(ctx) + 1)), replace=False).tolist())
            n = len(picks)
            sub = dataclasses.replace(w, req_slots=w.req_slots[picks], token_indices=w.token_indices[picks],
                                      cu_tokens=np.arange(n + 1, dtype=np.uint32),
                                      q=w.q.reshape(-1, row)[picks].reshape(-1),
                                      flat_k=w.flat_k.reshape(-1, kv_row)[picks].reshape(-1),
                                      flat_v=w.flat_v.reshape(-1, kv_row)[picks].reshape(-1))
            with torch.cuda.stream(side):
                shape = gqa.prepare_fixed_partition(meta, sub.req_slots, sub.token_indices, sub.cu_tokens, 512,
                                                    balanced=True, num_workers=workers, bucket_capacities=True)
                assert shape.num_total_sdpa_map_task_templates >= shape.num_sdpa_map_task_templates
                for dst, src in ((q, sub.q), (k, sub.flat_k), (v, sub.flat_v)):
                    dst.zero_()
                    dst[:src.size].copy_(device.from_numpy(src).view(torch.bfloat16))
                pages.copy_(pristine)
                out.fill_(-768.0)
                inp = psi.GQAInput(w.layout, w.layer, meta, psi.GQAKVCacheBindings(pages, page_ids), scratch,
                                   q=q, k=k, v=v, output=out)
                cache.submit(inp)
                side.synchronize()
            exp_pages, exp = oracle_step(oracle, sub)
            got = out.cpu().numpy()
            assert_outputs_close(got[:n * row], exp, f"bucketed batch {b} {picks}")
            assert (got[n * row:] == -768.0).all(), "rows beyond the active tokens were written"
            assert np.array_equal(pages.view(torch.int16).cpu().numpy().view(np.uint16).reshape(exp_pages.shape), exp_pages)
        programs, recordings, replays = cache.stats()
        assert replays == batches and recordings == programs and recordings <= batches // 2, (recordings, batches)
        cache.close()
    finally:
        device.f32_output(False)
        device.use_stream(main)


def test_replay_cache_records_again_when_a_context_flag_changes(psi, oracle, device):
    """The output type of the combine (context flag F32_OUTPUT) is baked into a recorded program's arguments: a
    submission after the flag has changed must record a new program, not replay the old one into a buffer of the
    other element size."""
    import torch

    wl = importlib_workloads(psi)
    w = wl.make_workload(172, [700, 33, 1500], 24, 4, 256, psi.Dtype.Bfloat16, 16)
    row = w.num_q_heads * w.head_dim
    gqa = _layer(psi, device, w, gated=False)
    meta = psi.GQAMetadataBuffers(device, 8, max_kv_splits=32, max_workers=8)
    scratch = gqa.new_scratch(8, 40)
    q, k, v = (device.from_numpy(a.reshape(-1)).view(torch.bfloat16) for a in (w.q, w.flat_k, w.flat_v))
    pages = device.from_numpy(w.pages.reshape(-1)).view(torch.bfloat16)
    page_ids = device.from_numpy(w.page_ids)
    # one buffer for both element sizes: f32 rows fill it, bf16 rows fill its first half
    out = torch.zeros(w.num_tokens * row, dtype=torch.float32, device=device.torch_device)
    side, main = torch.cuda.Stream(), device.stream
    device.use_stream(side)
    try:
        cache = psi.GQAReplayCache(device, gqa)
        _, exp = oracle_step(oracle, w)
        results = []
        for f32 in (True, False, True):
            device.f32_output(f32)
            with torch.cuda.stream(side):
                gqa.prepare_fixed_partition(meta, w.req_slots, w.token_indices, w.cu_tokens, 512, balanced=True,
                                            num_workers=8)
                out.fill_(-768.0)
                inp = psi.GQAInput(w.layout, w.layer, meta, psi.GQAKVCacheBindings(pages, page_ids), scratch,
                                   q=q, k=k, v=v, output=out)
                results.append(cache.submit(inp))
                side.synchronize()
            if f32:
                assert_outputs_close(out.cpu().numpy(), exp, "f32 output")
            else:
                half = out.view(torch.bfloat16)
                got = half[:w.num_tokens * row].to(torch.float32).cpu().numpy()
                assert np.abs(got - exp).max() <= 2e-2
                assert (out[w.num_tokens * row // 2:] == -768.0).all(), "a bf16 program wrote beyond its rows"
        assert results == [True, True, False]
        programs, recordings, replays = cache.stats()
        assert (programs, recordings, replays) == (2, 2, 3)
        cache.close()
    finally:
        device.f32_output(False)
        device.use_stream(main)


@pytest.mark.parametrize("q_lens,ctx", [
    ([200, 50, 1, 1, 3], [500, 300, 700, 33, 64]),   # two chunks, decode requests and a short verify request
    ([1, 1, 2, 1], [600, 47, 1024, 9]),              # no chunk at all: the decode part alone
    ([40, 130], [40, 900]),                          # chunks only
])
def test_mixed_batch_is_one_prepare_and_one_record(psi, oracle, device, q_lens, ctx):
    """A batch of prefill chunks and decode requests behind one planning call and one layer call
    (psi_hip_gqa_layer_prepare_mixed / _record_mixed): pages bit-exact and outputs within the bar of the CPU
    oracle on the whole batch, whichever of the two parts the batch holds."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(181, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_lens)
    exp_pages, exp = oracle_step(oracle, w)
    n_chunk = sum(1 for n in q_lens if n > 8)
    if 0 < n_chunk < len(q_lens):
        step = wl.MixedStep(device, w, decode_partition=512, chunk_partition=256, f32_output=True)
    else:  # MixedStep insists on both parts; the entry points do not
        step = _one_kind_mixed_step(psi, wl, device, w)
    plan = step.mixed_plan
    assert plan.num_chunk_reqs == n_chunk and plan.num_chunk_tokens == sum(n for n in q_lens if n > 8)
    assert plan.has_chunk == (n_chunk > 0) and plan.has_decode == (n_chunk < len(q_lens))
    step.step()
    got = step.output_f32()
    assert device.take_device_error() == 0
    assert np.array_equal(step.pages_host().reshape(exp_pages.shape), exp_pages)
    assert_outputs_close(got, exp, f"mixed batch {q_lens}")


def _one_kind_mixed_step(psi, wl, device, w):
    """`MixedStep` for a batch with only chunks or only decode requests (its constructor asks for both)."""
    import torch

    step = wl.MixedStep.__new__(wl.MixedStep)
    step.device, step.w, step.f32_output = device, w, True
    step.pages, step.page_ids = wl.device_pages(device, w), device.from_numpy(w.page_ids)
    step.q, step.flat_k, step.flat_v = (device.from_numpy(a.reshape(-1)) for a in (w.q, w.flat_k, w.flat_v))
    step.chunk_partition, step.decode_partition, step.chunk_min_tokens = 256, 512, 8
    step.chunk_meta = psi.GQAMetadataBuffers(device, w.num_tokens, max_kv_splits=256)
    step.decode_meta = psi.GQAMetadataBuffers(device, w.num_tokens, max_kv_splits=64)
    step.gqa = _layer(psi, device, w, gated=False)
    step.plan()
    step.scratch = torch.empty(step.gqa.mixed_scratch_bytes(step.mixed_plan), dtype=torch.uint8,
                               device=device.torch_device)
    step.output = torch.zeros(w.num_tokens * w.num_q_heads * w.head_dim, dtype=torch.float32, device=device.torch_device)

    class _Scratch:
        qgkv = None
        q_norm_rope = None
        sdpa_partial = step.scratch
        attention_output = step.output

    step._input = psi.GQAInput(w.layout, w.layer, step.chunk_meta, psi.GQAKVCacheBindings(step.pages, step.page_ids),
                               _Scratch, q=step.q, k=step.flat_k, v=step.flat_v, output=step.output)
    return step


def test_mixed_batch_wants_its_chunks_first(psi, device):
    wl = importlib_workloads(psi)
    w = wl.make_workload(182, [600, 300], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[1, 100])
    gqa = _layer(psi, device, w, gated=False)
    chunk_meta = psi.GQAMetadataBuffers(device, 128, max_kv_splits=64)
    decode_meta = psi.GQAMetadataBuffers(device, 128, max_kv_splits=64)
    with pytest.raises(psi.PsiHipError, match="must come first"):
        gqa.prepare_mixed(chunk_meta, decode_meta, w.req_slots, w.token_indices, w.cu_tokens)
