"""GPU parity of the multi-query path (speculative verify with 2 or 4 tokens per sequence, prefill
chunks, mixed batches) against the CPU oracle through the C ABI, and the verify -> accept -> roll
back cycle driven by the library's own token-window bookkeeping.  Same tolerance as the decode
path: 2e-3 max-abs / 1e-3 relative RMS on f32 outputs, pages bit-exact."""
import importlib

import numpy as np
import pytest

from parity_util import assert_outputs_close, importlib_workloads, oracle_step, run_and_check

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("q_len,expected_head_tile", [(2, 3), (4, 6)])
def test_verify_batches(psi, oracle, device, q_len, expected_head_tile):
    """C4's geometry (24 Q / 4 KV, D=256, bf16, 16-token pages) at oracle-sized contexts."""
    wl = importlib_workloads(psi)
    rng = np.random.default_rng(40 + q_len)
    ctx = rng.integers(40, 1500, size=8).tolist() + [q_len, 16, 17, 513]
    w = wl.make_workload(41 + q_len, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_len)
    stats, dw = run_and_check(psi, oracle, device, w, f"verify q_len={q_len}", max_tokens=4 * len(ctx) * q_len)
    assert dw.variant.is_tiled() and dw.variant.q_head_tile_size == expected_head_tile
    print("verify q_len", q_len, "max_abs %.3e rel_rms %.3e" % stats, dw.shape)


@pytest.mark.parametrize("partition", [None, 256])
def test_prefill_chunk_on_prefix(psi, oracle, device, partition):
    """A 200-token chunk on a 300-token prefix next to decode-sized requests, one variant for all."""
    wl = importlib_workloads(psi)
    q_lens = [200, 1, 1, 3, 8, 9]
    ctx = [500, 700, 33, 64, 8, 40]
    w = wl.make_workload(51, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_lens)
    stats, dw = run_and_check(psi, oracle, device, w, "prefill chunk", partition_tokens=partition, max_tokens=512)
    assert dw.variant.is_tiled()
    print("prefill chunk max_abs %.3e rel_rms %.3e" % stats, dw.shape)


@pytest.mark.parametrize("dtype_name,hq,hkv,d,p,q_len", [
    ("Bfloat16", 32, 4, 128, 8, 4),
    ("Bfloat16", 12, 2, 256, 8, 2),
    ("Float16", 16, 2, 256, 16, 5),
    ("Bfloat16", 4, 4, 256, 16, 8),
    ("Float32", 4, 2, 64, 4, 3),
    ("Bfloat16", 24, 4, 256, 8, 8),  # the reference's (256, 8) profile, full tiles
    ("Float16", 8, 1, 128, 8, 3),
    ("Float16", 16, 2, 256, 16, 8),   # 8 heads per KV head, full tiles: 64 columns: the row-group kernel, a row per group
    ("Bfloat16", 16, 2, 256, 16, 7),  # 56 columns
])
def test_tiled_geometries(psi, oracle, device, dtype_name, hq, hkv, d, p, q_len):
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(61, [300, 31, 129, q_len], hq, hkv, d, dtype, p, q_lens=q_len, num_page_ids_per_block=2)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16 if p >= 8 else 4, min(hq // hkv, 8))
    run_and_check(psi, oracle, device, w, f"tiled {dtype_name} {hq}/{hkv}/{d} P={p} q={q_len}", max_tokens=64,
                  variant=variant)


@pytest.mark.parametrize("scale", [1.0, 0.25, 1.0 / 256.0])
@pytest.mark.parametrize("dtype_name", ["Bfloat16", "Float16"])
def test_sharp_and_flat_softmax(psi, oracle, device, scale, dtype_name):
    """Logits from very peaked (scale 1: log2-domain spread of tens of units, a new maximum every few
    tiles) to almost flat (1/256).  The maps move a column's reference maximum only when a tile
    exceeds it by more than 2^8 and carry probabilities up to that size as 2-byte matrix operands;
    the outputs must stay inside the tolerance either way - through the multi-query map (short
    tiles) and through the chunk map (a 150-token chunk in row groups)."""
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(81, [700, 333, 64, 1200], 24, 4, 256, dtype, 16, q_lens=[3, 4, 2, 1], scale=scale)
    run_and_check(psi, oracle, device, w, f"verify scale {scale} {dtype_name}", max_tokens=64)
    w = wl.make_workload(82, [650, 40], 24, 4, 256, dtype, 16, q_lens=[150, 2], scale=scale)
    stats, dw = run_and_check(psi, oracle, device, w, f"chunk scale {scale} {dtype_name}", partition_tokens=256,
                              max_tokens=512, grouped=True)
    assert dw.grouped


def test_sentinel_split_rows_are_skipped(psi, oracle, device):
    """The split list is padded to its capacity with 0xFFFFFFFF rows; they must not touch anything:
    the scratch behind the active rows keeps its fill pattern."""
    import torch

    wl = importlib_workloads(psi)
    w = wl.make_workload(71, [90, 200, 45], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[2, 2, 1])
    dw = wl.DeviceWorkload(device, w, max_tokens=32, f32_output=True,
                           variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6))
    assert dw.shape.num_total_sdpa_map_task_templates > dw.shape.num_sdpa_map_task_templates
    dw.scratch.buffer.view(torch.int32).fill_(0x5A5A5A5A)
    dw.step()
    got = dw.output_f32()
    _, exp = oracle_step(oracle, w)
    assert_outputs_close(got, exp, "padded")
    raw = dw.scratch.buffer.view(torch.int32).cpu().numpy()
    assert (raw == 0x5A5A5A5A).sum() > 0, "padded rows of the scratch were overwritten"


@pytest.mark.parametrize("balanced", [False, True])
def test_tile_wider_than_the_launch_was_sized_for(psi, oracle, device, balanced):
    """`max_active_q_tile_tokens` is a contract: a launch sized for two-token tiles (one column block) that meets a
    four-token tile cannot compute its rows.  It must enter them as empty states over whatever the scratch held,
    so that the combine merges nothing stale and the tile's output is visibly wrong (zeros), while every tile
    within the bound is computed as usual."""
    import torch

    wl = importlib_workloads(psi)
    w = wl.make_workload(73, [300, 90, 1200], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[2, 4, 2])
    dw = wl.DeviceWorkload(device, w, partition_tokens=512, max_tokens=32, f32_output=True, balanced=balanced,
                           variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6))
    dw.scratch.buffer.view(torch.float32).fill_(7.0)   # stale partial states: finite, plausible
    dw.append()
    m, s = dw.meta, dw.shape
    if balanced:
        dw.kernels.invoke_map_balanced(dw.q, dw.pages, m.d_req_slots, dw.page_ids, m.d_flat_token_indices,
                                       m.d_q_token_tiles, m.d_kv_splits, m.d_worker_cu, m.num_workers, dw.scratch,
                                       w.layer, s.num_tokens, s.num_q_token_tiles, s.num_sdpa_map_task_templates, 2)
    else:
        dw.kernels.invoke_map_bucketed(dw.q, dw.pages, m.d_req_slots, dw.page_ids, m.d_flat_token_indices,
                                       m.d_q_token_tiles, m.d_kv_splits, dw.scratch, w.layer, s.num_tokens,
                                       s.num_q_token_tiles, s.num_sdpa_map_task_templates, 2)
    dw.reduce()
    got = dw.output_f32().reshape(w.num_tokens, -1)
    _, exp = oracle_step(oracle, w)
    exp = exp.reshape(w.num_tokens, -1)
    assert_outputs_close(got[:2], exp[:2], "tile within the bound, before the wide one")
    assert_outputs_close(got[6:], exp[6:], "tile within the bound, after the wide one")
    assert (got[2:6] == 0.0).all(), "the wide tile's rows must come out as zeros, not as stale or partial sums"


def test_verify_accept_rollback_cycle(psi, oracle, device):
    """Two verify steps with drafts: step 1 writes K/V for [token, d1, d2, d3]; the host accepts a
    prefix; step 2 starts at the first rejected position and overwrites it.  Attention of step 2
    must see the accepted history only, and the page table / lengths come from the library's
    allocator and token window."""
    import torch

    rt = importlib.import_module("psi-dec_amd.runtime")
    wl = importlib_workloads(psi)
    rng = np.random.default_rng(81)
    hq, hkv, d, p, dtype = 24, 4, 256, 16, psi.Dtype.Bfloat16
    odt = oracle.BF16
    n_req, spec = 5, 3
    prompts = [int(x) for x in rng.integers(20, 200, size=n_req)]
    page_elems = 2 * hkv * p * d
    num_pages = sum(-(-(n + 16) // p) for n in prompts) + 8
    alloc = rt.U32IDAllocator(num_pages)
    max_blocks = max(-(-(n + 16) // p) for n in prompts)
    layout = psi.GQAPageTableLayout(n_req, 1, max_blocks, 1)
    table = psi.GQARequestPageTable(device, layout)
    host_table = np.zeros(layout.num_page_ids(), np.uint32)
    pages = np.zeros(num_pages * page_elems, np.uint16)  # host mirror maintained by the oracle
    dev_pages = device.from_numpy(pages)
    cfg_w = psi.GQAKVPageWriteConfig(hkv, d, page_elems * 2, dtype)
    blocks = []
    # per-token K/V/Q are a pure function of (request, position, token id) so that both sides agree

    def kvq(r, pos, tok):
        g = np.random.default_rng([r, pos, tok])
        return (wl.to_storage(g.standard_normal((hkv, d), dtype=np.float32), dtype),
                wl.to_storage(g.standard_normal((hkv, d), dtype=np.float32), dtype),
                wl.to_storage(g.standard_normal((hq, d), dtype=np.float32), dtype))

    def sync(r, b):
        s = b.prepare_blocks()
        for i, ids in enumerate(s.kv_page_ids[0]):
            table.write_page_ids(r, 0, s.block_index + i, ids, num_cache_pages=num_pages)
            host_table[(r * max_blocks + s.block_index + i)] = ids[0]

    def run_step(queries):
        """queries[r] = (token_index, [token ids incl. drafts]); appends then attends."""
        slots = list(range(n_req))
        starts = [q[0] for q in queries]
        cu = np.concatenate([[0], np.cumsum([len(q[1]) for q in queries])]).astype(np.uint32)
        fk, fv, fq = [], [], []
        for r, (start, toks) in enumerate(queries):
            for i, t in enumerate(toks):
                k, v, q = kvq(r, start + i, t)
                fk.append(k), fv.append(v), fq.append(q)
        fk, fv, fq = np.stack(fk), np.stack(fv), np.stack(fq)
        total = int(cu[-1])
        split = psi.GQASplitKV.new(psi.GQASplitKVConfig(dtype, page_elems * 2, hq, hkv, d))
        variant = split.select(total, n_req)
        assert variant.is_tiled()
        meta = psi.GQAMetadataBuffers(device, 64)
        shape = meta.update(slots, starts, cu.tolist(), variant)
        write = psi.GQAKVPageWrite(device, cfg_w)
        write.invoke_bucketed(psi.GQAKVPageWriteShape(shape.num_total_tokens, layout),
                              psi.GQAKVPageWriteBuffers(dev_pages, device.from_numpy(fk.reshape(-1)),
                                                        device.from_numpy(fv.reshape(-1)), meta.d_req_slots,
                                                        meta.d_flat_token_indices, table.page_ids_buffer()),
                              shape.num_tokens, 0)
        cfg = psi.GQASplitKVTiledQConfig(hq, hkv, d, variant.q_head_tile_size, variant.q_token_tile_size,
                                         variant.kv_token_tile_size, 1.0 / 16.0, page_elems * 2, dtype, layout)
        kshape = psi.GQASplitKVTiledQShape(shape.num_total_tokens, shape.num_total_q_token_tiles,
                                           shape.num_total_sdpa_map_task_templates)
        kern = psi.GQASplitKVTiledQKernels(device, cfg, kshape)
        scratch = psi.GQASplitKVTiledQScratch(device, cfg, kshape)
        out = torch.zeros(shape.num_total_tokens * hq * d, dtype=torch.float32, device=device.torch_device)
        kern.invoke_map_bucketed(device.from_numpy(fq.reshape(-1)), dev_pages, meta.d_req_slots,
                                 table.page_ids_buffer(), meta.d_flat_token_indices, meta.d_q_token_tiles,
                                 meta.d_kv_splits, scratch, 0, shape.num_tokens, shape.num_q_token_tiles,
                                 shape.num_sdpa_map_task_templates)
        device.f32_output(True)
        kern.invoke_reduce_bucketed(scratch, meta.d_q_token_tiles, meta.d_cu_kv_splits, out,
                                    shape.num_q_token_tiles)
        device.f32_output(False)
        device.sync()
        # oracle on the host mirror
        lt = (n_req, 1, max_blocks, 1)
        oracle.kv_page_write(pages, fk.reshape(-1), fv.reshape(-1), meta.h_req_slots[:total],
                             meta.h_flat_token_indices[:total], host_table, total, 0, lt, hkv, d, page_elems * 2, odt)
        exp = oracle.paged_gqa(hq, hkv, d, 1.0 / 16.0, page_elems * 2, odt, lt, 0, slots, starts, cu, fq.reshape(-1),
                               pages, host_table, num_threads=8)
        got = out[:total * hq * d].cpu().numpy()
        assert_outputs_close(got, exp, "verify step")
        assert np.array_equal(dev_pages.view(torch.int16).cpu().numpy().view(np.uint16), pages)

    # prefill the prompts on the host side of the bookkeeping (K/V history written by the oracle path)
    for r, n in enumerate(prompts):
        toks = [1000 * r + i for i in range(n)]
        b = rt.DecoderBlocks(alloc, p, 1, 1, toks)
        blocks.append(b)
        while b.ready_token_slots() < n - 1:
            assert b.init_block_once() != "ResourceLimitExceeded"
        q = b.prepare(n - 1)  # everything but the last prompt token
        assert q.kind == "Prefill" and q.token_index == 0
        sync(r, b)
        fk = np.stack([kvq(r, i, toks[i])[0] for i in range(n - 1)])
        fv = np.stack([kvq(r, i, toks[i])[1] for i in range(n - 1)])
        oracle.kv_page_write(pages, fk.reshape(-1), fv.reshape(-1), [r] * (n - 1), list(range(n - 1)), host_table,
                             n - 1, 0, (n_req, 1, max_blocks, 1), hkv, d, page_elems * 2, odt)
        b.commit(q, rt.SampledTokens.prefill(q.epoch))
        b.set_spec_tokens([50000 + 10 * r + j for j in range(spec)])
    dev_pages.copy_(device.from_numpy(pages))

    accepted_total = 0
    for step in range(2):
        queries, prepared = [], []
        for r, b in enumerate(blocks):
            budget = len(b.ready_tokens()) + len(b.queued_tokens()) + len(b.spec_tokens())
            while b.ready_token_slots() < budget:
                assert b.init_block_once() != "ResourceLimitExceeded"
            budget = len(b.ready_tokens()) + len(b.queued_tokens()) + len(b.spec_tokens())
            q = b.prepare(budget)
            assert q.kind == "Decode" and len(q.tokens) == 1 and len(q.spec_tokens) == spec
            assert q.token_index == len(b.cached_tokens())
            sync(r, b)
            prepared.append(q)
            queries.append((q.token_index, q.tokens + q.spec_tokens))
        run_step(queries)
        for r, (b, q) in enumerate(zip(blocks, prepared)):
            accept = int(rng.integers(0, spec + 1))  # seeded Bernoulli-prefix accept mask
            accepted_total += accept
            before = len(b.cached_tokens())
            b.commit(q, rt.SampledTokens.decode(q.epoch, q.spec_tokens[:accept], 70000 + 100 * step + r,
                                                [60000 + 100 * step + 10 * r + j for j in range(spec)]))
            # the cache advanced by the input token plus the accepted drafts; rejected slots will be rewritten
            assert len(b.cached_tokens()) == before + 1 + accept
    assert 0 < accepted_total < 2 * n_req * spec
    used = alloc.used()
    for b in blocks:
        b.close()
    assert alloc.used() == 0 and used > 0


def test_mfma_and_generic_kernels_agree_but_differ_in_rounding(psi, oracle, device):
    """The gfx950 kernels and the shape-generic kernels on one verify batch: both within tolerance of
    each other, and not bit-identical (which would mean the generic kernels served both runs)."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(91, [900, 2048, 77, 300], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=4)
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
    assert np.abs(a - b).max() < 2e-4
    assert not np.array_equal(a, b)


@pytest.mark.parametrize("partition,prefix,chunk", [(256, 300, 200), (512, 0, 77), (128, 1000, 64), (2048, 37, 300)])
def test_grouped_prefill_chunk(psi, oracle, device, partition, prefix, chunk):
    """The row-group map (K/V tiles staged once in LDS for up to 256 query columns) on a chunk next to
    decode-sized requests: same tolerance against the oracle as every other path."""
    wl = importlib_workloads(psi)
    q_lens = [chunk, 1, 3, 8]
    ctx = [prefix + chunk, 700, 64, 8]
    w = wl.make_workload(91, ctx, 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_lens)
    stats, dw = run_and_check(psi, oracle, device, w, f"grouped chunk {chunk} on {prefix}", partition_tokens=partition,
                              max_tokens=512, grouped=True, variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6))
    assert dw.meta.num_row_groups > 0 and dw.meta.group_tiles == 16
    print("grouped chunk max_abs %.3e rel_rms %.3e" % stats, dw.shape, dw.meta.num_row_groups)


def test_grouped_long_unsplit_range(psi, oracle, device):
    """A chunk against 20000 cached tokens in a single partition: 627 KV tiles go round the row-group map's four LDS
    stages, with its loading waves several tiles ahead of the multiplying ones all the way, and the range neither
    begins nor ends on a tile."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(97, [20000 + 57, 9], 4, 2, 256, psi.Dtype.Bfloat16, 16, q_lens=[57, 9])
    stats, dw = run_and_check(psi, oracle, device, w, "grouped chunk 57 on 20000, one partition", max_tokens=128,
                              variant=psi.GQASplitKVVariant.TiledQ(8, 16, 2), partition_tokens=32768, grouped=True)
    assert dw.meta.num_row_groups > 0
    print("long range max_abs %.3e rel_rms %.3e" % stats, dw.shape, dw.meta.num_row_groups)


@pytest.mark.parametrize("dtype_name,hq,hkv,d,p,q_len", [
    ("Float16", 16, 2, 256, 16, 50),    # 8 heads per KV head: two head subsets of 4, f16 single-term P
    ("Bfloat16", 4, 4, 256, 32, 130),   # one head per KV head: 16 tiles per group, 32-token pages
    ("Bfloat16", 10, 2, 256, 64, 41),   # 5 heads per KV head: one subset, 3 tiles per group
    ("Bfloat16", 14, 2, 256, 16, 23),   # 7 heads: subsets of 4 and 3
    # the reference's TiledQ profiles (crates/inference-backend-metal/src/components/gqa_split_kv_tiled_q.rs:66-76)
    ("Bfloat16", 24, 4, 256, 8, 77),    # (256, 8): a 32-key tile spans four pages
    ("Bfloat16", 32, 8, 128, 8, 90),    # (128, 8), the heads of the reference's Criterion bench
    ("Bfloat16", 40, 8, 128, 8, 61),    # (128, 8), the heads of its published timing: 5 per KV head
    ("Bfloat16", 32, 8, 128, 16, 130),  # head_dim 128 on 16-token pages
    ("Float16", 16, 2, 128, 32, 35),    # head_dim 128, f16, 8 heads per KV head
])
def test_grouped_geometries(psi, oracle, device, dtype_name, hq, hkv, d, p, q_len):
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    w = wl.make_workload(93, [300, 31 + q_len, q_len], hq, hkv, d, dtype, p, q_lens=[q_len, q_len, q_len],
                         num_page_ids_per_block=2)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, min(hq // hkv, 8))
    _, dw = run_and_check(psi, oracle, device, w, f"grouped {dtype_name} {hq}/{hkv}/{d} P={p} q={q_len}",
                          max_tokens=512, variant=variant, partition_tokens=128, grouped=True)
    assert dw.meta.num_row_groups > 0


@pytest.mark.parametrize("hq,hkv,d,p,q_lens,width", [
    (32, 4, 256, 16, [8, 8, 5, 8, 1], 4),   # verify steps at 8 heads per KV head: 64 columns, all heads in one item
    (28, 4, 256, 16, [8, 1, 8], 4),         # 7 heads: 56 columns
    (24, 4, 128, 8, [8, 8, 40], 5),         # 6 heads: a chunk of five tiles still fits (240 columns)
    (16, 2, 128, 16, [32, 8], 4),           # 8 heads x 32 tokens: all 256 columns of one item
    (16, 2, 256, 32, [33, 8], 8),           # one token more: back to two head subsets, tables 8 tiles wide
])
def test_grouped_short_chunks_walk_their_range_once_for_all_heads(psi, oracle, device, hq, hkv, d, p, q_lens, width):
    """With more than five heads per KV head a row group's heads are dealt to two or three work items - unless no
    group of the batch is wider than what fits one workgroup with all the heads: then the table is written that
    narrow and a work item serves every head of its KV head, reading the KV range once."""
    wl = importlib_workloads(psi)
    prefixes = [700, 64, 1500, 0, 333][:len(q_lens)]
    ctx = [a + b for a, b in zip(prefixes, q_lens)]
    w = wl.make_workload(411, ctx, hq, hkv, d, psi.Dtype.Bfloat16, p, q_lens=q_lens)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, hq // hkv)
    _, dw = run_and_check(psi, oracle, device, w, f"grouped short chunks {hq}/{hkv}/{d} q={q_lens}", max_tokens=256,
                          variant=variant, partition_tokens=512, grouped=True)
    assert dw.meta.num_row_groups > 0 and dw.meta.group_tiles == width


@pytest.mark.parametrize("hq,q_lens,expect_groups", [
    (24, [8, 3, 8, 1], False),      # single tiles of up to 48 columns: the multi-query pipeline over a balanced plan
    (24, [8, 16, 8, 1], True),      # a request with two Q-token tiles
    (32, [8, 8, 2, 8], True),       # 64 columns per tile
    (24, [1, 1, 1, 1], False),      # decode
    (24, [200, 1, 2, 8], True),     # a prefill chunk among decode-sized requests
])
def test_the_library_picks_the_dispatch(psi, oracle, device, hq, q_lens, expect_groups):
    """PSI_HIP_DISPATCH_AUTO through the one-call preparation: whichever launch it picks, the step matches the
    oracle."""
    wl = importlib_workloads(psi)
    prefixes = [3000, 700, 1025, 64]
    ctx = [a + b for a, b in zip(prefixes, q_lens)]
    w = wl.make_workload(433, ctx, hq, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=q_lens)
    _, dw = run_and_check(psi, oracle, device, w, f"auto dispatch {hq} heads q={q_lens}", partition_tokens=512,
                          max_tokens=512, auto=True)
    assert dw.grouped == expect_groups and dw.balanced != expect_groups
    assert (dw.meta.num_row_groups > 0) == expect_groups and (dw.meta.num_workers > 0) != expect_groups


@pytest.mark.parametrize("seed", range(16))
def test_grouped_random_batches(psi, oracle, device, seed):
    """Seeded random batches through the row-group map against the oracle: head groups 1..8, both head dims, pages
    of 8..64 tokens, both 16-bit types, partitions that do and do not divide the contexts, chunks from one token to
    a few hundred next to decode-sized requests, contexts that end inside a tile, on a tile boundary and inside
    the first tile."""
    rng = np.random.default_rng(7000 + seed)
    wl = importlib_workloads(psi)
    group = int(rng.choice([1, 2, 4, 5, 6, 7, 8]))
    hkv = int(rng.choice([1, 2, 4]))
    d = int(rng.choice([128, 256]))
    p = int(rng.choice([8, 16, 32, 64]))
    dtype = psi.Dtype.Bfloat16 if rng.random() < 0.7 else psi.Dtype.Float16
    n = int(rng.integers(1, 5))
    q_lens = [int(rng.choice([1, 2, 7, 8, 9, 33, 64, 100, 257])) for _ in range(n)]
    prefixes = [int(rng.choice([0, 1, 15, 31, 32, 33, 200, 511, 777])) for _ in range(n)]
    ctx = [a + b for a, b in zip(prefixes, q_lens)]
    partition = int(rng.choice([64, 128, 256, 2048]))
    w = wl.make_workload(7100 + seed, ctx, group * hkv, hkv, d, dtype, p, q_lens=q_lens,
                         num_page_ids_per_block=int(rng.choice([1, 2])))
    variant = psi.GQASplitKVVariant.TiledQ(8, 16, group)
    _, dw = run_and_check(psi, oracle, device, w,
                          f"grouped random {seed}: G={group} Hkv={hkv} D={d} P={p} q={q_lens} on {prefixes} part={partition}",
                          max_tokens=1024, variant=variant, partition_tokens=partition, grouped=True)
    assert dw.meta.num_row_groups > 0


@pytest.mark.parametrize("prefix,chunk", [(0, 700), (1500, 300), (37, 64)])
def test_grouped_with_the_planned_partition(psi, oracle, device, prefix, chunk):
    """The partition length that the library's planner picks for the batch (psi_hip_split_kv_chunk_partition_tokens)
    instead of a given one: a multiple of 256 tokens, and the same outputs against the oracle as with any other."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(99, [prefix + chunk, 40], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[chunk, 5])
    _, dw = run_and_check(psi, oracle, device, w, f"grouped chunk {chunk} on {prefix}, planned partition",
                          max_tokens=1024, variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6), partition_tokens="auto",
                          grouped=True, check_rounded=False)
    assert dw.partition_tokens % 256 == 0 and 256 <= dw.partition_tokens <= (prefix + chunk + 255) // 256 * 256
    assert dw.meta.num_row_groups > 0


def test_grouped_more_items_than_workgroups(psi, oracle, device):
    """The row-group map runs one workgroup per compute unit, and a workgroup that is through with its item takes the
    next from a counter that the launch leaves at zero.  Here the launch has several times as many items as the GPU
    has compute units, of one to four KV tiles each; the outputs match the oracle, and a second and a third
    step on the same context, the third after a small launch in between, repeat the first bit for bit."""
    wl = importlib_workloads(psi)
    w = wl.make_workload(95, [1100, 40], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[900, 40])
    _, dw = run_and_check(psi, oracle, device, w, "grouped chunk 900 on 200, 128-token partitions", max_tokens=1024,
                          variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6), partition_tokens=128, grouped=True,
                          check_rounded=False)
    items = dw.meta.num_row_groups * 4 * 3  # KV heads x head subsets
    assert items > 512, items
    first = dw.output_f32().copy()
    dw.step()
    assert np.array_equal(dw.output_f32(), first)
    small = wl.make_workload(96, [70], 24, 4, 256, psi.Dtype.Bfloat16, 16, q_lens=[9])
    run_and_check(psi, oracle, device, small, "grouped chunk 9 on 61", max_tokens=64,
                  variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6), partition_tokens=256, grouped=True, check_rounded=False)
    dw.step()
    assert np.array_equal(dw.output_f32(), first)


def test_grouped_and_plain_maps_agree(psi, oracle, device):
    """Same plan through both maps: the outputs differ only in rounding, the grouped table falls
    back to the plain map where the geometry has no grouped kernel (head_dim 64)."""
    wl = importlib_workloads(psi)
    for d, p, expect_groups in [(256, 16, True), (256, 8, True), (128, 8, True), (64, 16, False)]:
        w = wl.make_workload(95, [900, 450], 24, 4, d, psi.Dtype.Bfloat16, p, q_lens=[300, 450])
        outs = []
        for grouped in (False, True):
            dw = wl.DeviceWorkload(device, w, partition_tokens=256, max_tokens=1024, f32_output=True, grouped=grouped,
                                   variant=psi.GQASplitKVVariant.TiledQ(8, 16, 6))
            dw.step()
            outs.append(dw.output_f32())
            if grouped:
                assert (dw.meta.num_row_groups > 0) == expect_groups
        diff = np.abs(outs[0] - outs[1]).max()
        assert diff < 1e-3, diff
        if not expect_groups:
            assert diff == 0.0


@pytest.mark.parametrize("dtype_name,hq,hkv,d,p,q_lens", [
    ("Bfloat16", 24, 4, 256, 16, 2),                        # one-draft verify: one column block
    ("Bfloat16", 24, 4, 256, 16, 4),                        # three drafts: two column blocks
    ("Bfloat16", 24, 4, 256, 16, [8, 3, 1, 8, 5, 2, 7]),    # full tiles: three column blocks, the loading wave takes one
    ("Bfloat16", 16, 2, 256, 16, [8, 2, 8, 1, 8, 3, 8]),    # 64 columns: the row-group kernel, a row per group
    ("Float16", 16, 2, 256, 8, 3),                          # 8-token pages
    ("Bfloat16", 32, 8, 128, 16, [20, 1, 9, 2, 1, 1, 12]),  # several Q-token tiles per request
    ("Float32", 6, 2, 64, 8, 2),                            # generic kernels: one workgroup per row
])
def test_balanced_plan_for_multi_query_rows(psi, oracle, device, dtype_name, hq, hkv, d, p, q_lens):
    """The multi-query map over equal worker shares (one workgroup per compute unit), a tile's adjacent pieces
    inside a share merged into one row: outputs within tolerance of the oracle and, up to the order of
    summation, equal to the row-per-workgroup launch; pages bit-exact."""
    wl = importlib_workloads(psi)
    dtype = getattr(psi.Dtype, dtype_name)
    ctx = [30000, 40, 1025, 9000, 700, 33, 513]
    w = wl.make_workload(53, ctx, hq, hkv, d, dtype, p, q_lens=q_lens)
    variant = psi.GQASplitKVVariant.TiledQ(8, 16 if p >= 8 else 4, min(hq // hkv, 8))
    what = f"balanced tiled {dtype_name} {hq}/{hkv}/{d} P={p} q={q_lens}"
    stats, dw = run_and_check(psi, oracle, device, w, what, partition_tokens=512, variant=variant, balanced=True,
                              max_tokens=64)
    assert dw.balanced and dw.shape.num_sdpa_map_task_templates <= dw.meta.num_workers + dw.shape.num_q_token_tiles
    plain = wl.DeviceWorkload(device, w, partition_tokens=512, variant=variant, f32_output=True, max_tokens=64)
    plain.step()
    # f16 probabilities are one 11-bit term: their rounding depends on where the rows are cut (the row-group kernel
    # rounds them to f16 for bf16 K/V, too)
    one_term = dtype_name == "Float16" or hq // hkv * 8 > 48
    assert np.abs(plain.output_f32() - dw.output_f32()).max() < (2e-4 if one_term else 2e-5)
