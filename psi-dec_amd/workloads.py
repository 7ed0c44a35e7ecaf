"""Seeded synthetic workloads for the paged-attention path: page pools, block tables, K/V history,
new-token K/V and queries in the shapes the benchmark configurations name.  Host arrays are numpy;
`DeviceWorkload` uploads them and drives one layer-step (append -> split-KV map -> combine)
through the library.  Nothing here computes attention.
"""
from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

from . import gqa as G


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))
    return (rounded >> np.uint32(16)).astype(np.uint16)


def to_storage(x: np.ndarray, dtype: G.Dtype) -> np.ndarray:
    """f32 values -> the element storage of `dtype` (f32, or uint16 bit patterns)."""
    if dtype == G.Dtype.Float32:
        return np.ascontiguousarray(x, dtype=np.float32)
    if dtype == G.Dtype.Bfloat16:
        return f32_to_bf16_bits(x)
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


@dataclass
class Workload:
    """One layer-step of a batch: `q_lens[r]` new tokens per request on top of `token_indices[r]`
    cached ones.  The page arena holds random history everywhere; the new tokens' K/V arrive in
    flat_k / flat_v and are appended by the step itself."""

    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    dtype: G.Dtype
    scale: float
    tokens_per_page: int
    layout: G.GQAPageTableLayout
    layer: int
    num_pages: int
    req_slots: np.ndarray        # [requests]
    token_indices: np.ndarray    # [requests] position of the first new token
    cu_tokens: np.ndarray        # [requests + 1]
    page_ids: np.ndarray         # the table, flat u32
    pages: Optional[np.ndarray]  # arena storage [num_pages, 2, Hkv, P, D] (None when filled on device)
    q: np.ndarray                # storage [tokens, Hq, D]
    flat_k: np.ndarray           # storage [tokens, Hkv, D]
    flat_v: np.ndarray
    seed: int
    outlier_rate: float = 0.0    # K elements set to +-outlier_sigma * input_scale (applied on the device too)
    outlier_sigma: float = 8.0
    input_scale: float = 1.0

    @property
    def page_bytes(self) -> int:
        return 2 * self.num_kv_heads * self.tokens_per_page * self.head_dim * self.dtype.item_size()

    @property
    def num_tokens(self) -> int:
        return int(self.cu_tokens[-1])

    @property
    def context_lens(self) -> np.ndarray:
        """Context length of each request after the append."""
        return self.token_indices + np.diff(self.cu_tokens)

    def algorithmic_bytes(self) -> int:
        """Bytes one layer-step must move: every visible K and V element once, Q read, O write,
        append read + write."""
        es = self.dtype.item_size()
        kv = int(self.context_lens.astype(np.int64).sum()) * 2 * self.num_kv_heads * self.head_dim * es
        t = self.num_tokens
        qo = 2 * t * self.num_q_heads * self.head_dim * es
        append = t * 2 * self.num_kv_heads * self.head_dim * es * 2
        return kv + qo + append

    def map_algorithmic_bytes(self) -> int:
        """Bytes of the split-KV map kernel alone: visible K and V once plus the Q read."""
        es = self.dtype.item_size()
        q_lens = np.diff(self.cu_tokens).astype(np.int64)
        # with more than one new token per request the tokens share one pass over the context
        kv = int(self.context_lens.astype(np.int64).sum()) * 2 * self.num_kv_heads * self.head_dim * es
        return kv + int(q_lens.sum()) * self.num_q_heads * self.head_dim * es


def make_workload(seed: int, context_lens: Sequence[int], num_q_heads: int, num_kv_heads: int, head_dim: int,
                  dtype: G.Dtype, tokens_per_page: int = 16, q_lens=1, scale: Optional[float] = None,
                  input_scale: float = 1.0, num_gqa_layers: int = 1, layer: int = 0, num_page_ids_per_block: int = 1,
                  spare_pages: int = 3, host_pages: bool = True, outlier_rate: float = 0.0,
                  outlier_sigma: float = 8.0, shuffle_slots: bool = True, shuffle_pages: bool = True) -> Workload:
    """`context_lens[r]` counts the tokens of request r after this step's append."""
    rng = np.random.default_rng(seed)
    context_lens = np.asarray(context_lens, dtype=np.int64)
    batch = len(context_lens)
    q_lens = np.full(batch, q_lens, dtype=np.int64) if np.isscalar(q_lens) else np.asarray(q_lens, dtype=np.int64)
    assert (context_lens >= q_lens).all() and (q_lens >= 1).all()
    token_indices = (context_lens - q_lens).astype(np.uint32)
    cu_tokens = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.uint32)
    pages_per_req = -(-context_lens // tokens_per_page)
    blocks_per_req = -(-pages_per_req // num_page_ids_per_block)
    num_blocks = int(blocks_per_req.max())
    num_req_slots = batch + 1
    layout = G.GQAPageTableLayout(num_req_slots, num_gqa_layers, num_blocks, num_page_ids_per_block)
    req_slots = (rng.permutation(num_req_slots)[:batch] if shuffle_slots else np.arange(batch)).astype(np.uint32)
    num_pages = int(pages_per_req.sum()) + spare_pages
    pool = rng.permutation(num_pages).astype(np.uint32)
    if not shuffle_pages:
        pool = np.arange(num_pages, dtype=np.uint32)  # identity table, as the reference's own benches use
    table = np.zeros(layout.num_page_ids(), dtype=np.uint32)
    # rows of other layers stay zero on purpose: a kernel that walks the wrong layer reads page 0
    cursor = 0
    per_slot = num_gqa_layers * num_blocks * num_page_ids_per_block
    for r in range(batch):
        n = int(pages_per_req[r])
        start = int(req_slots[r]) * per_slot + layer * num_blocks * num_page_ids_per_block
        table[start:start + n] = pool[cursor:cursor + n]
        cursor += n
    total_tokens = int(cu_tokens[-1])
    elems_per_page = 2 * num_kv_heads * tokens_per_page * head_dim

    def normal(shape):
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(input_scale)

    pages = None
    if host_pages:
        values = normal((num_pages, elems_per_page))
        if outlier_rate > 0:
            # large-magnitude K outliers: the K half of each page is [0, elems/2)
            k_part = values[:, :elems_per_page // 2]
            mask = rng.random(k_part.shape) < outlier_rate
            signs = np.where(rng.random(k_part.shape) < 0.5, -1.0, 1.0).astype(np.float32)
            k_part[mask] = (outlier_sigma * input_scale) * signs[mask]
        pages = to_storage(values, dtype).reshape(num_pages, 2, num_kv_heads, tokens_per_page, head_dim)
    q = to_storage(normal((total_tokens, num_q_heads, head_dim)), dtype)
    flat_k = to_storage(normal((total_tokens, num_kv_heads, head_dim)), dtype)
    flat_v = to_storage(normal((total_tokens, num_kv_heads, head_dim)), dtype)
    if scale is None:
        scale = 1.0 / float(np.sqrt(head_dim))
    return Workload(num_q_heads, num_kv_heads, head_dim, dtype, float(scale), tokens_per_page, layout, layer,
                    num_pages, req_slots, token_indices, cu_tokens, table, pages, q, flat_k, flat_v, seed,
                    outlier_rate, outlier_sigma, input_scale)


def device_pages(device: G.Device, w: Workload):
    """The workload's page arena in HBM: uploaded when the workload carries host pages, else drawn on the device
    from the workload's seed (same distribution, K outliers included)."""
    import torch

    dev = device.torch_device
    torch_dtype = w.dtype.torch()
    if w.pages is not None:
        return device.from_numpy(w.pages.reshape(-1))
    n = w.num_pages * 2 * w.num_kv_heads * w.tokens_per_page * w.head_dim
    gen = torch.Generator(device=dev)
    gen.manual_seed(w.seed)
    pages = torch.empty(n, dtype=torch_dtype, device=dev)
    chunk = 1 << 26
    for start in range(0, n, chunk):
        end = min(n, start + chunk)
        pages[start:end] = (torch.randn(end - start, generator=gen, device=dev, dtype=torch.float32) *
                            w.input_scale).to(torch_dtype)
    if w.outlier_rate > 0:
        # large-magnitude K outliers: the K half of each page comes first
        half = w.num_kv_heads * w.tokens_per_page * w.head_dim
        by_page = pages.view(w.num_pages, 2 * half)
        rows = 1 << 12
        for start in range(0, w.num_pages, rows):
            k_part = by_page[start:start + rows, :half]
            draw = torch.rand(k_part.shape, generator=gen, device=dev)
            value = torch.where(draw < w.outlier_rate / 2, w.outlier_sigma * w.input_scale,
                                -w.outlier_sigma * w.input_scale).to(torch_dtype)
            k_part.copy_(torch.where(draw < w.outlier_rate, value, k_part))
    return pages


class DeviceWorkload:
    """A workload resident in HBM plus the metadata and scratch one layer-step needs."""

    def __init__(self, device: G.Device, w: Workload, partition_tokens: Optional[int] = None,
                 max_tokens: Optional[int] = None, variant: Optional[G.GQASplitKVVariant] = None,
                 f32_output: bool = False, balanced: bool = False, longest_first: bool = False,
                 grouped: bool = False, fused_append: bool = False, num_workers: Optional[int] = None,
                 pages=None, page_ids=None, auto: bool = False):
        """`pages` / `page_ids`: an arena and a page table already on the device (shared with another workload
        of the same step) instead of this workload's own.  `auto`: the library picks the dispatch for the batch
        (PSI_HIP_DISPATCH_AUTO): row groups over the planner's partition, or the balanced plan over
        `partition_tokens`."""
        import torch

        self.device, self.w = device, w
        self.torch_dtype = w.dtype.torch()
        dev = device.torch_device
        self.pages = pages if pages is not None else device_pages(device, w)
        self.q = device.from_numpy(w.q.reshape(-1))
        self.flat_k = device.from_numpy(w.flat_k.reshape(-1))
        self.flat_v = device.from_numpy(w.flat_v.reshape(-1))
        self.page_ids = page_ids if page_ids is not None else device.from_numpy(w.page_ids)
        split_kv = G.GQASplitKV.new(G.GQASplitKVConfig(w.dtype, w.page_bytes, w.num_q_heads, w.num_kv_heads,
                                                       w.head_dim))
        q_lens = np.diff(w.cu_tokens)
        if variant is None:
            variant = split_kv.select(w.num_tokens, int(sum(-(-int(n) // 8) for n in q_lens)))
        self.variant = variant
        rows = variant.q_token_tile_size if variant.is_tiled() else 1
        if partition_tokens == "auto":
            # prefill chunks through the row-group map: the partition that the library's model of the launch picks
            assert grouped and variant.is_tiled(), "the partition planner serves the row-group map"
            partition_tokens = G.chunk_partition_tokens(split_kv.config, variant.q_token_tile_size,
                                                        [int(t) for t in w.token_indices],
                                                        [int(c) for c in w.cu_tokens]) or None
        self.partition_tokens = partition_tokens
        self._auto = bool(auto)
        if auto:
            assert partition_tokens is not None and not grouped, "auto dispatch plans over fixed partitions"
            balanced = True
        if partition_tokens is not None:
            if variant.is_tiled():
                tile = variant.q_token_tile_size
                shortest = min(partition_tokens, 256) if auto else partition_tokens  # (the planner's are 256 * k)
                splits_cap = int(sum(-(-int(c) // shortest) * -(-int(n) // tile)
                                     for c, n in zip(w.context_lens, q_lens)))
            else:
                splits_cap = int(sum(-(-(int(t) + i + 1) // partition_tokens)
                                     for t, n in zip(w.token_indices, q_lens) for i in range(int(n))))
            self.meta = G.GQAMetadataBuffers(device, max(w.num_tokens, 1), max_kv_splits=splits_cap)
        else:
            self.meta = G.GQAMetadataBuffers(device, max_tokens or max(w.num_tokens, 1))
        self._partition_tokens, self._longest_first, self._num_workers = partition_tokens, longest_first, num_workers
        self.balanced = bool(balanced) and not grouped  # the prefill-chunk map has its own row grouping
        self.grouped = bool(grouped) and variant.is_tiled()
        self.gqa = G.GQA(device, G.GQACore(0, w.num_q_heads * w.head_dim, w.head_dim, w.num_q_heads, w.num_kv_heads,
                                           w.scale),
                         G.GQAMetalConfig(w.page_bytes, 2, 1e-6, 10000.0, io_dtype=w.dtype), gated=False)
        self._layer_struct = self.gqa.struct()
        self.plan()
        s = self.shape
        self.write = G.GQAKVPageWrite(device, G.GQAKVPageWriteConfig(w.num_kv_heads, w.head_dim, w.page_bytes,
                                                                     w.dtype))
        self.write_shape = G.GQAKVPageWriteShape(s.num_total_tokens, w.layout)
        self.f32_output = f32_output
        out_dtype = torch.float32 if f32_output else self.torch_dtype
        self.output = torch.zeros(s.num_total_tokens * w.num_q_heads * w.head_dim, dtype=out_dtype, device=dev)
        if variant.is_tiled():
            self.cfg = G.GQASplitKVTiledQConfig(w.num_q_heads, w.num_kv_heads, w.head_dim, variant.q_head_tile_size,
                                                variant.q_token_tile_size, variant.kv_token_tile_size, w.scale,
                                                w.page_bytes, w.dtype, w.layout)
            self.kshape = G.GQASplitKVTiledQShape(s.num_total_tokens, s.num_total_q_token_tiles,
                                                  s.num_total_sdpa_map_task_templates)
            self.kernels = G.GQASplitKVTiledQKernels(device, self.cfg, self.kshape)
            self.scratch = G.GQASplitKVTiledQScratch(device, self.cfg, self.kshape)
        else:
            self.cfg = G.GQASplitKVSingleQConfig(w.num_q_heads, w.num_kv_heads, w.head_dim, w.scale, w.page_bytes,
                                                 w.layout, variant.kv_token_tile_size,
                                                 variant.num_threads_per_threadblock, variant.q_head_tile_size,
                                                 w.dtype)
            self.kshape = G.GQASplitKVSingleQShape(s.num_total_tokens, s.num_total_sdpa_map_task_templates)
            self.kernels = G.GQASplitKVSingleQKernels(device, self.cfg, self.kshape)
            self.scratch = G.GQASplitKVSingleQScratch(device, self.cfg, self.kshape)
        self._rows = rows
        # decode only: the append rides in the map launch (one launch fewer per step)
        self.fused_append = bool(fused_append) and not variant.is_tiled()
        self._layer_input = None

    def plan(self):
        """The host side of one step: batch metadata, split plan, dispatch plan (worker shares, row order or row
        groups) in one library call, and one upload into the metadata buffers' fixed device arrays."""
        w = self.w
        L = G.L
        dispatch = (L.DISPATCH_AUTO if self._auto else L.DISPATCH_ROW_GROUPS if self.grouped else
                    L.DISPATCH_BALANCED if self.balanced else
                    L.DISPATCH_LONGEST_FIRST if self._longest_first else L.DISPATCH_PLAN_ORDER)
        fixed = self._partition_tokens is not None
        self.shape = self.meta.prepare(self._layer_struct, w.req_slots, w.token_indices, w.cu_tokens,
                                       capacity_mode=L.CAPACITY_FIXED_PARTITION if fixed else L.CAPACITY_EXACT,
                                       partition_tokens=self._partition_tokens or 0, dispatch=dispatch,
                                       num_workers=self._num_workers or 0, variant=self.variant)
        if self._auto:  # what the library picked
            self.grouped = self.meta.num_row_groups > 0
            self.balanced = not self.grouped
        return self.shape

    def append(self):
        m = self.meta
        self.write.invoke_bucketed(
            self.write_shape,
            G.GQAKVPageWriteBuffers(self.pages, self.flat_k, self.flat_v, m.d_req_slots, m.d_flat_token_indices,
                                    self.page_ids),
            self.shape.num_tokens, self.w.layer)

    def map(self):
        m, s = self.meta, self.shape
        if self.variant.is_tiled() and self.grouped and m.num_row_groups:
            self.kernels.invoke_map_grouped(self.q, self.pages, m.d_req_slots, self.page_ids,
                                            m.d_flat_token_indices, m.d_q_token_tiles, m.d_kv_splits, self.scratch,
                                            self.w.layer, s.num_tokens, s.num_q_token_tiles,
                                            s.num_sdpa_map_task_templates, m.d_row_groups, m.group_tiles,
                                            m.num_row_groups,
                                            min(int(np.diff(self.w.cu_tokens).max()),
                                                self.variant.q_token_tile_size))
        elif self.variant.is_tiled() and self.balanced:
            self.kernels.invoke_map_balanced(self.q, self.pages, m.d_req_slots, self.page_ids,
                                             m.d_flat_token_indices, m.d_q_token_tiles, m.d_kv_splits, m.d_worker_cu,
                                             m.num_workers, self.scratch, self.w.layer, s.num_tokens,
                                             s.num_q_token_tiles, s.num_sdpa_map_task_templates,
                                             min(int(np.diff(self.w.cu_tokens).max()),
                                                 self.variant.q_token_tile_size))
        elif self.variant.is_tiled():
            self.kernels.invoke_map_bucketed(self.q, self.pages, m.d_req_slots, self.page_ids,
                                             m.d_flat_token_indices, m.d_q_token_tiles, m.d_kv_splits, self.scratch,
                                             self.w.layer, s.num_tokens, s.num_q_token_tiles,
                                             s.num_sdpa_map_task_templates,
                                             min(int(np.diff(self.w.cu_tokens).max()),
                                                 self.variant.q_token_tile_size))
        elif self.balanced:
            self.kernels.invoke_map_balanced(self.q, self.pages, m.d_req_slots, self.page_ids, m.d_kv_splits,
                                             m.d_worker_cu, m.num_workers, self.scratch, self.w.layer, s.num_tokens,
                                             s.num_sdpa_map_task_templates)
        else:
            self.kernels.invoke_map_bucketed(self.q, self.pages, m.d_req_slots, self.page_ids, m.d_kv_splits,
                                             self.scratch, self.w.layer, s.num_tokens,
                                             s.num_sdpa_map_task_templates)

    def reduce(self):
        m, s = self.meta, self.shape
        self.device.f32_output(self.f32_output)
        if self.variant.is_tiled():
            self.kernels.invoke_reduce_bucketed(self.scratch, m.d_q_token_tiles, m.d_cu_kv_splits, self.output,
                                                s.num_q_token_tiles, partial_row_index=m.d_partial_row_index)
        else:
            self.kernels.invoke_reduce_bucketed(self.scratch, m.d_cu_kv_splits, self.output, s.num_tokens,
                                                partial_row_index=m.d_partial_row_index)
        self.device.f32_output(False)

    def append_map(self):
        m, s = self.meta, self.shape
        self.kernels.invoke_append_map_bucketed(self.q, self.pages, self.flat_k, self.flat_v, m.d_req_slots,
                                                m.d_flat_token_indices, self.page_ids, m.d_kv_splits, self.scratch,
                                                self.w.layer, s.num_tokens, s.num_sdpa_map_task_templates,
                                                worker_cu=m.d_worker_cu if self.balanced else None,
                                                num_workers=m.num_workers if self.balanced else 0)

    def layer_input(self) -> "G.GQAInput":
        """The step as the layer entry takes it: split, normalised rows in; the workload's own buffers as scratch."""
        if self._layer_input is None:
            w = self.w

            class _Scratch:  # the buffers of `GQAScratch` this path touches
                qgkv = None
                q_norm_rope = None
                sdpa_partial = self.scratch.buffer
                attention_output = self.output

            self._layer_input = G.GQAInput(w.layout, w.layer, self.meta, G.GQAKVCacheBindings(self.pages, self.page_ids),
                                           _Scratch, replay_mode=G.GQAReplayMode.Bucketed, q=self.q, k=self.flat_k,
                                           v=self.flat_v, output=self.output)
        self._layer_input.kv_cache = G.GQAKVCacheBindings(self.pages, self.page_ids)
        return self._layer_input

    def step(self):
        """One layer-step: append the new tokens, then attend (the new tokens see themselves).  Issued through
        the layer entry (`GQA.record`) unless the decode step is asked to launch its append separately, which
        exercises the component entry points one by one."""
        if self.fused_append or self.variant.is_tiled():
            self.device.f32_output(self.f32_output)
            try:
                self.gqa.record(self.layer_input())
            finally:
                self.device.f32_output(False)
            return
        self.append()
        self.map()
        self.reduce()

    def output_f32(self) -> np.ndarray:
        import torch

        self.device.sync()
        n = self.w.num_tokens * self.w.num_q_heads * self.w.head_dim
        return self.output[:n].to(torch.float32).cpu().numpy()

    def pages_host(self) -> np.ndarray:
        """The arena's bytes as the storage dtype (uint16 bit patterns for 2-byte types)."""
        import torch

        self.device.sync()
        t = self.pages
        if t.dtype in (torch.bfloat16, torch.float16, torch.int16):
            return t.view(torch.int16).cpu().numpy().view(np.uint16)
        return t.cpu().numpy()


class MixedStep:
    """A step that holds prefill chunks and decode tokens at once, over one arena and one page table.  The
    reference would run one SplitKV variant for the whole batch; here the requests with more than
    `chunk_min_tokens` new tokens go through the multi-query kernels with the row-group plan and the others
    through the decode kernels (balanced worker plan, append inside the map launch): one planning call
    (`GQA.prepare_mixed`) and one layer call (`GQA.record_mixed`) for the whole batch.  The chunk requests must
    come first in the batch, so that either part's tokens are one contiguous run of the flat q / k / v / output
    rows."""

    def __init__(self, device: G.Device, w: Workload, decode_partition: int = 512,
                 chunk_partition: Optional[int] = None, chunk_min_tokens: int = 8, f32_output: bool = False):
        import torch

        q_lens = np.diff(w.cu_tokens).astype(np.int64)
        is_chunk = q_lens > chunk_min_tokens
        n_chunk = int(is_chunk.sum())
        assert 0 < n_chunk < len(q_lens) and is_chunk[:n_chunk].all(), "chunk requests first, then decode requests"
        self.device, self.w, self.f32_output = device, w, f32_output
        self.pages, self.page_ids = device_pages(device, w), device.from_numpy(w.page_ids)
        self.q = device.from_numpy(w.q.reshape(-1))
        self.flat_k = device.from_numpy(w.flat_k.reshape(-1))
        self.flat_v = device.from_numpy(w.flat_v.reshape(-1))
        n_chunk_tokens = int(w.cu_tokens[n_chunk])
        chunk_ctx = w.context_lens[:n_chunk]
        if chunk_partition is None:
            # what the library's model of the row-group launch picks for these chunks (4096 tokens for a 2048-token
            # chunk over 4096 cached tokens: 192 work items of 128 KV tiles and 192 of 4 to 64)
            config = G.GQASplitKVConfig(w.dtype, w.page_bytes, w.num_q_heads, w.num_kv_heads, w.head_dim)
            chunk_partition = G.chunk_partition_tokens(config, 8, [int(t) for t in w.token_indices[:n_chunk]],
                                                       [int(c) for c in w.cu_tokens[:n_chunk + 1]])
            if chunk_partition == 0:  # no row-group kernel for this geometry: the multi-query map's partitions
                chunk_partition = 512
        self.chunk_partition, self.decode_partition, self.chunk_min_tokens = chunk_partition, decode_partition, chunk_min_tokens
        chunk_rows = int(sum(-(-int(c) // chunk_partition) * -(-int(n) // 8) for c, n in zip(chunk_ctx, q_lens[:n_chunk])))
        decode_rows = int(sum(-(-(int(t) + i + 1) // decode_partition)
                              for t, n in zip(w.token_indices[n_chunk:], q_lens[n_chunk:]) for i in range(int(n))))
        self.chunk_meta = G.GQAMetadataBuffers(device, n_chunk_tokens, max_kv_splits=chunk_rows)
        self.decode_meta = G.GQAMetadataBuffers(device, w.num_tokens - n_chunk_tokens, max_kv_splits=decode_rows)
        self.gqa = G.GQA(device, G.GQACore(0, w.num_q_heads * w.head_dim, w.head_dim, w.num_q_heads, w.num_kv_heads,
                                           w.scale),
                         G.GQAMetalConfig(w.page_bytes, 2, 1e-6, 10000.0, io_dtype=w.dtype), gated=False)
        self.plan()
        self.scratch = torch.empty(self.gqa.mixed_scratch_bytes(self.mixed_plan), dtype=torch.uint8,
                                   device=device.torch_device)
        out_dtype = torch.float32 if f32_output else w.dtype.torch()
        self.output = torch.zeros(w.num_tokens * w.num_q_heads * w.head_dim, dtype=out_dtype, device=device.torch_device)

        class _Scratch:  # the buffers of `GQAScratch` this path touches
            qgkv = None
            q_norm_rope = None
            sdpa_partial = self.scratch
            attention_output = self.output

        self._input = G.GQAInput(w.layout, w.layer, self.chunk_meta, G.GQAKVCacheBindings(self.pages, self.page_ids),
                                 _Scratch, replay_mode=G.GQAReplayMode.Bucketed, q=self.q, k=self.flat_k,
                                 v=self.flat_v, output=self.output)

    def plan(self):
        """The host side of the step: both parts planned by one library call, two uploads."""
        w = self.w
        self.mixed_plan = self.gqa.prepare_mixed(self.chunk_meta, self.decode_meta, w.req_slots, w.token_indices,
                                                 w.cu_tokens, chunk_min_tokens=self.chunk_min_tokens,
                                                 chunk_partition=self.chunk_partition,
                                                 decode_partition=self.decode_partition)
        return self.mixed_plan

    def step(self):
        self.device.f32_output(self.f32_output)
        try:
            self.gqa.record_mixed(self._input, self.mixed_plan)
        finally:
            self.device.f32_output(False)

    def algorithmic_bytes(self) -> int:
        return self.w.algorithmic_bytes()

    def chunk_flops(self) -> int:
        """Matrix flops of the chunk part: 4 * Hq * D per visible (query, key) pair."""
        w, n = self.w, self.mixed_plan.num_chunk_reqs
        q_lens = np.diff(w.cu_tokens).astype(np.int64)
        pairs = sum(int(w.token_indices[r]) * int(q_lens[r]) + int(q_lens[r]) * (int(q_lens[r]) + 1) // 2 for r in range(n))
        return 4 * w.num_q_heads * w.head_dim * pairs

    def decode_map_bytes(self) -> int:
        """Algorithmic bytes of the decode part's map: its visible K and V once plus its Q rows."""
        w, n = self.w, self.mixed_plan.num_chunk_reqs
        es = w.dtype.item_size()
        q_lens = np.diff(w.cu_tokens).astype(np.int64)
        kv = int(w.context_lens[n:].astype(np.int64).sum()) * 2 * w.num_kv_heads * w.head_dim * es
        return kv + int(q_lens[n:].sum()) * w.num_q_heads * w.head_dim * es

    def output_f32(self) -> np.ndarray:
        import torch

        self.device.sync()
        return self.output.to(torch.float32).cpu().numpy()

    def pages_host(self) -> np.ndarray:
        import torch

        self.device.sync()
        return self.pages.view(torch.int16).cpu().numpy().view(np.uint16)


def config_c5(seed: int = 5, chunk: int = 2048, prefix: int = 4096, batch: int = 128, lo: int = 512,
              hi: int = 32768) -> Workload:
    """Mixed chunked-prefill + decode step: one sequence appends `chunk` tokens on a `prefix`-token history, `batch`
    decode sequences with contexts uniform in [lo, hi] append one token each; 24 Q / 4 KV heads, D=256, bf16,
    16-token pages of one shuffled pool."""
    ctx = np.concatenate([[prefix + chunk], config_c2_context_lens(seed, batch, lo, hi) + 1])
    return make_workload(seed, ctx, 24, 4, 256, G.Dtype.Bfloat16, 16, q_lens=[chunk] + [1] * batch,
                         host_pages=False)


def config_c1(seed: int = 1) -> Workload:
    """Single-sequence decode: batch 1, context 512 after the append, 16 Q / 2 KV heads, D=256, fp16,
    16-token pages; inputs N(0,1)/sqrt(256).  Appending position 511 keeps the pool at 32 pages."""
    return make_workload(seed, [512], 16, 2, 256, G.Dtype.Float16, 16, input_scale=1.0 / 16.0, spare_pages=0,
                         shuffle_slots=False)


def config_c2_context_lens(seed: int = 2, batch: int = 32, lo: int = 1024, hi: int = 8192) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.integers(lo, hi + 1, size=batch)


def config_c2(seed: int = 2, batch: int = 32, host_pages: bool = False, lo: int = 1024, hi: int = 8192,
              shuffle_pages: bool = True) -> Workload:
    """Batched ragged decode: contexts uniform in [lo, hi] (before the append), 24 Q / 4 KV heads,
    D=256, bf16, 16-token pages from a shuffled pool; each step appends one token per sequence."""
    ctx = config_c2_context_lens(seed, batch, lo, hi) + 1
    return make_workload(seed, ctx, 24, 4, 256, G.Dtype.Bfloat16, 16, host_pages=host_pages,
                         shuffle_pages=shuffle_pages)
