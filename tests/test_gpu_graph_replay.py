"""A decode layer-step (append -> map -> combine) captured into a HIP graph and replayed: every
replay, with the program's own eager work and synchronisations in between, must reproduce the
eager result bit for bit on the inputs current at replay time.  The library's launches take their
active counts as kernel arguments and use no memset, so a captured step is self-contained."""
import numpy as np
import pytest

from parity_util import assert_outputs_close, importlib_workloads, oracle_step

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("q_len,fused_append", [(1, False), (2, False), (1, True)])
def test_captured_layer_step_replays(psi, oracle, device, q_len, fused_append):
    """`fused_append`: the append rides in the decode map launch (two nodes in the graph instead of three).
    Every replay equals the eager step bit for bit, and the eager step matches the CPU oracle on the inputs of
    that replay."""
    import dataclasses

    import torch

    wl = importlib_workloads(psi)
    w = wl.make_workload(101 + q_len, [700, 33, 1500, 512, 64], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    dw = wl.DeviceWorkload(device, w, partition_tokens=512, fused_append=fused_append, f32_output=True)
    assert dw.fused_append == fused_append
    pristine = dw.pages.clone()
    current = w

    def eager():
        dw.pages.copy_(pristine)
        dw.step()
        device.sync()
        return dw.output.clone()

    base = eager()
    side = torch.cuda.Stream()
    main = device.stream
    graph = torch.cuda.CUDAGraph()
    try:
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            device.use_stream(side)
            dw.pages.copy_(pristine)
            dw.step()  # warm-up on the capture stream
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                dw.step()
    finally:
        device.use_stream(main)
    torch.cuda.synchronize()

    rng = np.random.default_rng(7)
    for replay in range(4):
        # new inputs each time: queries and the new tokens' K/V change, the history is restored
        dw.pages.copy_(pristine)
        if replay:
            fresh = {}
            for name, t in (("q", dw.q), ("flat_k", dw.flat_k), ("flat_v", dw.flat_v)):
                fresh[name] = wl.to_storage(rng.standard_normal(t.numel(), dtype=np.float32), w.dtype)
                t.copy_(device.from_numpy(fresh[name]))
            current = dataclasses.replace(w, **fresh)
        expected = eager()
        n = w.num_tokens * w.num_q_heads * w.head_dim
        assert_outputs_close(expected[:n].cpu().numpy(), oracle_step(oracle, current)[1], f"eager step of replay {replay}")
        dw.pages.copy_(pristine)
        dw.output.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dw.output.view(torch.int32), expected.view(torch.int32)), f"replay {replay}"
        if replay == 0:
            assert torch.equal(dw.output.view(torch.int32), base.view(torch.int32))
        # eager work of the program between replays
        _ = (dw.output.float() * 2).sum().item()


@pytest.mark.parametrize("balanced", [False, True])
def test_one_captured_step_serves_every_batch_of_its_bucket(psi, oracle, device, balanced):
    """Device-side active counts (`ReplayU32::Parameter` of the reference): a decode step captured once at the
    capacity of its bucket (5 tokens, 16 splits) with the counts bound, then replayed for batches of 5, 3, 1 and
    4 requests after refreshing only the metadata arrays, the inputs and the 16-byte count block.  Each replay
    equals the eager step with by-value counts, bit for bit, in the output rows (f32, before output rounding) and
    in the page arena, and that eager step matches the CPU oracle on the batch; rows beyond the active count keep
    a canary.  `balanced`: the plan is re-cut into equal worker shares on the host
    for every batch and the append rides in the map launch; the grid (workers x KV heads) is the same for all."""
    import torch

    wl = importlib_workloads(psi)
    ctx_lens = [700, 33, 1500, 512, 64]
    w = wl.make_workload(111, ctx_lens, 24, 4, 256, psi.Dtype.Bfloat16, 16)
    workers = 8
    cap_tokens, cap_splits = 5, 16 + (workers if balanced else 0)
    dw = wl.DeviceWorkload(device, w, partition_tokens=512)  # owns pages, page table, q, flat_k, flat_v
    pristine = dw.pages.clone()
    variant = dw.variant
    cfg = dw.cfg
    kernels = psi.GQASplitKVSingleQKernels(device, cfg, psi.GQASplitKVSingleQShape(cap_tokens, cap_splits))
    scratch = psi.GQASplitKVSingleQScratch(device, cfg, psi.GQASplitKVSingleQShape(cap_tokens, cap_splits))
    write_shape = psi.GQAKVPageWriteShape(cap_tokens, w.layout)
    row = w.num_q_heads * w.head_dim
    kv_row = w.num_kv_heads * w.head_dim
    i32 = dict(dtype=torch.int32, device=device.torch_device)
    d_slots, d_pos = torch.zeros(cap_tokens, **i32), torch.zeros(cap_tokens, **i32)
    d_splits, d_cu = torch.zeros(cap_splits * 3, **i32), torch.zeros(cap_tokens + 1, **i32)
    d_counts = torch.zeros(4, **i32)
    d_workers = torch.zeros(workers + 1, **i32)
    q, fk, fv = torch.zeros_like(dw.q), torch.zeros_like(dw.flat_k), torch.zeros_like(dw.flat_v)
    out = torch.zeros(cap_tokens * row, dtype=torch.float32, device=device.torch_device)
    host_meta = psi.GQAMetadataBuffers(None, cap_tokens, max_kv_splits=cap_splits)
    device.f32_output(True)  # taken when a combine is launched or captured

    def load_batch(picks):
        n = len(picks)
        shape = host_meta.update_fixed_partition(w.req_slots[picks], w.token_indices[picks], list(range(n + 1)), variant,
                                                 512)
        if balanced:
            shape = host_meta.balance(workers)
            d_workers.copy_(device.from_numpy(host_meta.h_worker_cu.copy()))
            d_splits.fill_(-1)
            d_splits.copy_(device.from_numpy(host_meta.h_kv_splits[:cap_splits * 3].copy()))
            d_slots.copy_(device.from_numpy(host_meta.h_req_slots.copy()))
            d_pos.copy_(device.from_numpy(host_meta.h_flat_token_indices.copy()))
            d_cu.copy_(device.from_numpy(host_meta.h_cu_kv_splits.copy()))
        if not balanced:
            for dst, src in ((d_slots, host_meta.h_req_slots), (d_pos, host_meta.h_flat_token_indices),
                             (d_splits, host_meta.h_kv_splits[:cap_splits * 3]), (d_cu, host_meta.h_cu_kv_splits)):
                dst.copy_(device.from_numpy(src.copy()))
        for dst, src, width in ((q, dw.q, row), (fk, dw.flat_k, kv_row), (fv, dw.flat_v, kv_row)):
            dst.zero_()
            for i, r in enumerate(picks):
                dst[i * width:(i + 1) * width] = src[r * width:(r + 1) * width]
        d_counts.copy_(torch.tensor([shape.num_tokens, shape.num_q_token_tiles, shape.num_sdpa_map_task_templates, 0],
                                    dtype=torch.int32))
        return shape

    def step(active_tokens, active_splits):
        if balanced:
            kernels.invoke_append_map_bucketed(q, dw.pages, fk, fv, d_slots, d_pos, dw.page_ids, d_splits, scratch,
                                               w.layer, active_tokens, active_splits, worker_cu=d_workers,
                                               num_workers=workers)
        else:
            bufs = psi.GQAKVPageWriteBuffers(dw.pages, fk, fv, d_slots, d_pos, dw.page_ids)
            dw.write.invoke_bucketed(write_shape, bufs, active_tokens, w.layer)
            kernels.invoke_map_bucketed(q, dw.pages, d_slots, dw.page_ids, d_splits, scratch, w.layer, active_tokens,
                                        active_splits)
        kernels.invoke_reduce_bucketed(scratch, d_cu, out, active_tokens)

    # capture at capacity with the count block bound
    load_batch([0, 1, 2, 3, 4])
    side, main = torch.cuda.Stream(), device.stream
    graph = torch.cuda.CUDAGraph()
    try:
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            device.use_stream(side)
            device.bind_replay_counts(d_counts)
            step(cap_tokens, cap_splits)  # warm-up on the capture stream
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                step(cap_tokens, cap_splits)
    finally:
        device.bind_replay_counts(None)
        device.use_stream(main)
        device.f32_output(False)
    torch.cuda.synchronize()

    import dataclasses

    for picks in ([0, 1, 2, 3, 4], [2, 0, 4], [3], [4, 3, 1, 0]):
        shape = load_batch(picks)
        n = shape.num_tokens
        dw.pages.copy_(pristine)
        out.fill_(-768.0)
        device.f32_output(True)
        step(shape.num_tokens, shape.num_sdpa_map_task_templates)  # eager, counts by value
        device.f32_output(False)
        device.sync()
        eager_out, eager_pages = out.clone(), dw.pages.clone()
        sub = dataclasses.replace(w, req_slots=w.req_slots[picks], token_indices=w.token_indices[picks],
                                  cu_tokens=np.arange(len(picks) + 1, dtype=np.uint32),
                                  q=w.q.reshape(-1, row)[picks].reshape(-1),
                                  flat_k=w.flat_k.reshape(-1, kv_row)[picks].reshape(-1),
                                  flat_v=w.flat_v.reshape(-1, kv_row)[picks].reshape(-1))
        exp_pages, exp = oracle_step(oracle, sub)
        assert_outputs_close(eager_out[:n * row].cpu().numpy(), exp, f"eager step {picks}")
        assert np.array_equal(eager_pages.view(torch.int16).cpu().numpy().view(np.uint16).reshape(exp_pages.shape), exp_pages)
        dw.pages.copy_(pristine)
        out.fill_(-768.0)
        scratch.buffer.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int32), eager_out.view(torch.int32)), picks
        assert torch.equal(dw.pages.view(torch.int16), eager_pages.view(torch.int16)), picks
        assert (out[n * row:] == -768.0).all() and (out[:n * row] != -768.0).any()
        _ = out.float().sum().item()  # eager work between replays


def test_one_captured_step_serves_every_layer_of_the_table(psi, device):
    """The page-table layer as a device-side parameter (`qwen3.5.mtp.gqa_layer_index` of the reference: one
    recorded program serves every MTP step).  A step captured once against a 3-layer table with the count
    block bound is replayed with word 3 = 1, 2, 3; each replay equals the eager step of that layer with the
    layer passed by value, bit for bit, and only that layer's pages change.  Word 3 = 0 keeps the by-value
    layer of the capture."""
    import torch

    wl = importlib_workloads(psi)
    import dataclasses

    ctx_lens = [300, 33, 700]
    layers = 3
    needed = sum(-(-c // 16) for c in ctx_lens)
    w0 = wl.make_workload(121, ctx_lens, 24, 4, 256, psi.Dtype.Bfloat16, 16, num_gqa_layers=layers, layer=0,
                          spare_pages=2 * needed + 3)
    # layers 1 and 2 get pages of their own from the spare part of the pool
    lay = w0.layout
    table = w0.page_ids.reshape(lay.num_req_slots, layers, lay.num_blocks * lay.num_page_ids_per_block).copy()
    free = [p for p in range(w0.num_pages) if p not in set(table[:, 0].ravel().tolist())]
    for layer in (1, 2):
        for r, c in enumerate(ctx_lens):
            n = -(-c // 16)
            table[int(w0.req_slots[r]), layer, :n] = [free.pop() for _ in range(n)]
    ws = [dataclasses.replace(w0, page_ids=table.reshape(-1), layer=l) for l in range(layers)]
    dws = [wl.DeviceWorkload(device, w, partition_tokens=256) for w in ws]
    pristine = dws[0].pages.clone()
    eager = []
    for dw in dws:  # same inputs, same arena contents, layer by value
        dw.pages.copy_(pristine)
        dw.step()
        device.sync()
        eager.append((dw.output.clone(), dw.pages.clone()))
    assert not torch.equal(eager[0][0], eager[1][0]) and not torch.equal(eager[0][1], eager[2][1])

    dw = dws[1]  # captured with layer 1 by value
    counts = torch.tensor([dw.shape.num_tokens, dw.shape.num_q_token_tiles, dw.shape.num_sdpa_map_task_templates, 0],
                          dtype=torch.int32, device=device.torch_device)
    side, main = torch.cuda.Stream(), device.stream
    graph = torch.cuda.CUDAGraph()
    try:
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            device.use_stream(side)
            device.bind_replay_counts(counts)
            dw.step()  # warm-up on the capture stream
            side.synchronize()
            with torch.cuda.graph(graph, stream=side):
                dw.step()
    finally:
        device.bind_replay_counts(None)
        device.use_stream(main)
    torch.cuda.synchronize()

    for word, layer in ((1, 0), (3, 2), (0, 1), (2, 1), (1, 0)):
        counts[3] = word
        dw.pages.copy_(pristine)
        dw.output.fill_(-768.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dw.output.view(torch.int16), eager[layer][0].view(torch.int16)), (word, layer)
        assert torch.equal(dw.pages.view(torch.int16), eager[layer][1].view(torch.int16)), (word, layer)
        _ = dw.output.float().sum().item()  # eager work between replays


def test_wide_combine_leaves_inactive_tokens_alone(psi, oracle, device):
    """Device-side counts below the capacity on a split list long enough for the workgroup-per-row combine
    (40 rows per token of capacity): the batch holds one of two tokens, the metadata beyond it is what the
    previous, full batch left behind.  The active token matches the oracle; the inactive token's output row
    keeps its canary and the map writes no partial row beyond the active splits."""
    import torch

    from parity_util import assert_outputs_close, layout_tuple, oracle_dtype

    wl = importlib_workloads(psi)
    w = wl.make_workload(131, [3000, 2000], 16, 2, 256, psi.Dtype.Bfloat16, 16)
    variant = psi.GQASplitKVVariant.SingleQ(16, 256, 8)
    dw = wl.DeviceWorkload(device, w, partition_tokens=64, variant=variant, f32_output=True)
    s = dw.shape
    rows_first = -(-3000 // 64)
    assert s.num_sdpa_map_task_templates == rows_first + -(-2000 // 64)
    assert s.num_total_sdpa_map_task_templates // s.num_total_tokens >= 32  # the wide combine's domain
    dw.step()  # the full batch: leaves its rows in the scratch and its entries in cu_kv_splits
    full = dw.output_f32().reshape(2, -1)
    row = w.num_q_heads * w.head_dim
    counts = torch.tensor([1, 1, rows_first, 0], dtype=torch.int32, device=device.torch_device)
    dw.output.fill_(-768.0)
    scratch_before = dw.scratch.buffer.clone()
    device.bind_replay_counts(counts)
    try:
        dw.step()  # by-value counts stay at the capacity (2 tokens, all rows)
        device.sync()
    finally:
        device.bind_replay_counts(None)
    got = dw.output.float().cpu().numpy().reshape(2, row)
    assert (got[1] == -768.0).all(), "the combine wrote the output row of an inactive token"
    assert np.array_equal(got[0], full[0])
    # partial rows of the inactive token are untouched
    acc_rows = dw.scratch.buffer.view(torch.float32)[-s.num_total_sdpa_map_task_templates * row:].view(-1, row)
    acc_before = scratch_before.view(torch.float32)[-s.num_total_sdpa_map_task_templates * row:].view(-1, row)
    assert torch.equal(acc_rows[rows_first:], acc_before[rows_first:])
    dt = oracle_dtype(oracle, w)
    exp = oracle.paged_gqa(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes, dt, layout_tuple(w),
                           w.layer, w.req_slots[:1], w.token_indices[:1], np.arange(2, dtype=np.uint32),
                           w.q.reshape(2, -1)[:1].reshape(-1), dw.pages_host(), w.page_ids, num_threads=8)
    assert_outputs_close(got[0], exp, "wide combine under device-side counts")


def test_a_stream_switch_keeps_the_contexts_launches_in_order(psi, oracle, device):
    """`psi_hip_ctx_set_stream`: what the context launches on the new stream runs behind what it launched on the old
    one, with no synchronisation by the caller.  The old stream is held busy while a step is queued on it; the step
    queued on the new stream right after must see that step's pages (it appends to the same slots and reads the
    history) and leave the output of its own inputs."""
    import dataclasses

    import torch

    wl = importlib_workloads(psi)
    w = wl.make_workload(77, [900, 40, 2100], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=2)
    dw = wl.DeviceWorkload(device, w, partition_tokens=512, f32_output=True)
    rng = np.random.default_rng(5)
    fresh = {name: wl.to_storage(rng.standard_normal(t.numel(), dtype=np.float32), w.dtype)
             for name, t in (("q", dw.q), ("flat_k", dw.flat_k), ("flat_v", dw.flat_v))}
    staged = {name: device.from_numpy(a) for name, a in fresh.items()}
    second = dataclasses.replace(w, **fresh)
    side, main = torch.cuda.Stream(), device.stream
    torch.cuda.synchronize()
    try:
        torch.cuda._sleep(50_000_000)  # the old stream is busy for tens of milliseconds
        dw.step()                       # first inputs, queued behind the sleep
        for name, t in (("q", dw.q), ("flat_k", dw.flat_k), ("flat_v", dw.flat_v)):
            t.copy_(staged[name])       # second inputs, behind the first step on the old stream
        device.use_stream(side)
        dw.step()                       # on the new stream: must run behind all of the above
        side.synchronize()
    finally:
        device.use_stream(main)
    torch.cuda.synchronize()
    n = w.num_tokens * w.num_q_heads * w.head_dim
    exp_pages, exp = oracle_step(oracle, second)
    assert_outputs_close(dw.output[:n].cpu().numpy(), exp, "the step on the new stream")
    got_pages = dw.pages.view(torch.int16).cpu().numpy().view(np.uint16)
    assert np.array_equal(got_pages.reshape(exp_pages.shape), exp_pages)
