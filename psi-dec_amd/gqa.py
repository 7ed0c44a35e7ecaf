"""Host-side mirror of the reference's GQA component interface over the C ABI.

Class and method names follow the reference's backend components so that tests read like the
reference's own:

  GQAPageTableLayout, GQAKVPageWriteConfig/Shape/Buffers, GQAKVPageWrite
      crates/inference-backend-metal/src/components/gqa_kv_page_write.rs:15-177
  GQASplitKVConfig, GQASplitKVVariant, GQASplitKV
      crates/inference-backend-metal/src/components/gqa_split_kv.rs:8-156
  GQASplitKVSingleQConfig/Shape/Scratch/Kernels
      crates/inference-backend-metal/src/components/gqa_split_kv_single_q.rs:47-383
  GQASplitKVTiledQConfig/Shape/Kernels
      crates/inference-backend-metal/src/components/gqa_split_kv_tiled_q.rs:46-327
  ReplayBucketPolicy                     crates/inference-executor-core/src/replay.rs:4-87
  GQAReplayBucketPolicy, GQAMetadataBuffers, select_split_kv_variant
      crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:12-346, attn/gqa/mod.rs:64-94
  GQARequestPageTable                    crates/inference-executor-metal/src/attn/gqa/request_page_table.rs:8-122

Where the reference records an `Invocation` into a replay program, the calls here launch on the
device's HIP stream immediately; stream order provides the barriers the reference records.
Device buffers are torch tensors (torch is only the allocator); every launch goes through
libpsi_hip.so and raises `PsiHipError` where the reference panics.
"""
import ctypes
from dataclasses import dataclass, field
from enum import IntEnum
from typing import List, Optional, Sequence

import numpy as np

from . import _lib as L


class Dtype(IntEnum):
    Float32 = L.F32
    Bfloat16 = L.BF16
    Float16 = L.F16

    def item_size(self) -> int:
        return 4 if self == Dtype.Float32 else 2

    def torch(self):
        import torch

        return {Dtype.Float32: torch.float32, Dtype.Bfloat16: torch.bfloat16, Dtype.Float16: torch.float16}[self]


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _nbytes(t):
    return t.numel() * t.element_size()


class Device:
    """One GPU and one stream; replaces `Device::system_default()` + `Stream::new`."""

    def __init__(self, index: int = 0, stream=None):
        import torch

        if not torch.cuda.is_available():
            raise RuntimeError("psi-dec_amd needs a GPU: torch.cuda.is_available() is False")
        self.lib = L.load()
        self.index = index
        self.torch_device = torch.device("cuda", index)
        torch.cuda.set_device(index)
        if stream is None:
            stream = torch.cuda.current_stream(self.torch_device)
        self.stream = stream
        handle = ctypes.c_void_p()
        L.check(self.lib.psi_hip_ctx_create(index, ctypes.c_void_p(stream.cuda_stream), ctypes.byref(handle)))
        self.ctx = handle

    def sync(self):
        L.check(self.lib.psi_hip_sync(self.ctx))

    def use_stream(self, stream):
        """Launch on another torch stream from now on (e.g. the stream a graph is captured on)."""
        self.stream = stream
        L.check(self.lib.psi_hip_ctx_set_stream(self.ctx, ctypes.c_void_p(stream.cuda_stream)))

    def bind_replay_counts(self, counts=None):
        """Device int32[4] = {active tokens, active Q-token tiles, active KV splits, 0} that every
        kernel reads when it runs (graph replay); None restores the by-value counts."""
        self._replay_counts = counts  # keep the tensor alive while it is bound
        L.check(self.lib.psi_hip_ctx_bind_replay_counts(self.ctx, _ptr(counts)))

    def set_timing(self, enabled: bool):
        L.check(self.lib.psi_hip_ctx_set_timing(self.ctx, int(enabled)))

    def reset_timing(self):
        L.check(self.lib.psi_hip_ctx_reset_timing(self.ctx))

    def kernel_time_ms(self, name: str):
        total, launches = ctypes.c_double(), ctypes.c_uint64()
        L.check(self.lib.psi_hip_ctx_kernel_time_ms(self.ctx, name.encode(), ctypes.byref(total),
                                                    ctypes.byref(launches)))
        return total.value, launches.value

    def force_generic(self, on: bool):
        L.check(self.lib.psi_hip_ctx_set_flag(self.ctx, L.FLAG_FORCE_GENERIC, int(on)))

    def f32_output(self, on: bool):
        """Combine kernels then store f32 outputs (for checking the result before output rounding)."""
        L.check(self.lib.psi_hip_ctx_set_flag(self.ctx, L.FLAG_F32_OUTPUT, int(on)))

    def close(self):
        if self.ctx:
            self.lib.psi_hip_ctx_destroy(self.ctx)
            self.ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # allocation helpers
    def zeros(self, shape, dtype):
        import torch

        return torch.zeros(shape, dtype=dtype, device=self.torch_device)

    def from_numpy(self, array: np.ndarray):
        import torch

        if array.dtype == np.uint32:
            return torch.from_numpy(array.view(np.int32).copy()).to(self.torch_device)
        if array.dtype == np.uint16:
            return torch.from_numpy(array.view(np.int16).copy()).to(self.torch_device)
        return torch.from_numpy(np.ascontiguousarray(array)).to(self.torch_device)


@dataclass(frozen=True)
class GQAPageTableLayout:
    num_req_slots: int
    num_gqa_layers: int
    num_blocks: int
    num_page_ids_per_block: int

    def validate(self):
        assert self.num_req_slots > 0 and self.num_blocks > 0
        assert self.num_gqa_layers > 0 and self.num_page_ids_per_block > 0

    def num_page_ids(self) -> int:
        return self.num_req_slots * self.num_gqa_layers * self.num_blocks * self.num_page_ids_per_block

    def bytes(self) -> int:
        return self.num_page_ids() * 4

    def num_physical_pages_per_request(self) -> int:
        return self.num_blocks * self.num_page_ids_per_block

    def struct(self):
        return L.PageTableLayoutStruct(self.num_req_slots, self.num_gqa_layers, self.num_blocks,
                                       self.num_page_ids_per_block)


def _cfg_struct(num_q_heads, num_kv_heads, head_dim, scale, page_bytes, dtype):
    return L.GQAConfigStruct(num_q_heads, num_kv_heads, head_dim, float(scale), page_bytes, int(dtype))


def _tokens_per_page(cfg_struct) -> int:
    out = ctypes.c_uint32()
    L.check(L.load().psi_hip_gqa_tokens_per_page(ctypes.byref(cfg_struct), ctypes.byref(out)))
    return out.value


# ------------------------------------------------------------------ KV append


@dataclass(frozen=True)
class GQAKVPageWriteConfig:
    num_kv_heads: int
    head_dim: int
    page_bytes: int
    dtype: Dtype

    def struct(self):
        # the append ignores the query side of the config
        return _cfg_struct(self.num_kv_heads, self.num_kv_heads, self.head_dim, 1.0, self.page_bytes, self.dtype)

    def num_tokens_per_page(self) -> int:
        return _tokens_per_page(self.struct())


@dataclass(frozen=True)
class GQAKVPageWriteShape:
    num_total_token_writes: int
    page_table_layout: GQAPageTableLayout


@dataclass
class GQAKVPageWriteBuffers:
    pages: object
    flat_k: object
    flat_v: object
    req_slots: object
    flat_token_indices: object
    page_ids: object


class GQAKVPageWrite:
    def __init__(self, device: Device, config: GQAKVPageWriteConfig):
        config.num_tokens_per_page()  # validates
        self.device, self.config = device, config

    def invoke(self, shape: GQAKVPageWriteShape, buffers: GQAKVPageWriteBuffers, page_table_index: int):
        self.invoke_bucketed(shape, buffers, shape.num_total_token_writes, page_table_index)

    def invoke_bucketed(self, shape, buffers, num_active_token_writes: int, page_table_index: int):
        cfg, layout = self.config.struct(), shape.page_table_layout.struct()
        L.check(self.device.lib.psi_hip_kv_page_write(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), _ptr(buffers.pages), _nbytes(buffers.pages),
            _ptr(buffers.flat_k), _ptr(buffers.flat_v), _ptr(buffers.req_slots), _ptr(buffers.flat_token_indices),
            _ptr(buffers.page_ids), shape.num_total_token_writes, num_active_token_writes, page_table_index))

    def invoke_norm_rope_bucketed(self, shape, buffers, norm: "RMSNormRopeConfig", norm_weight,
                                  num_active_token_writes: int, page_table_index: int, k_token_stride: int = 0,
                                  v_token_stride: int = 0):
        """The append with the K-side RMSNorm + RoPE fused in: `buffers.flat_k` holds the raw K rows
        (token strides in elements, 0 = dense), `norm` is the K norm config (num_heads = KV heads)."""
        cfg, layout, ncfg = self.config.struct(), shape.page_table_layout.struct(), norm.struct()
        L.check(self.device.lib.psi_hip_kv_page_write_norm_rope(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), ctypes.byref(ncfg), _ptr(buffers.pages),
            _nbytes(buffers.pages), _ptr(buffers.flat_k), k_token_stride, _ptr(buffers.flat_v), v_token_stride,
            _ptr(norm_weight), _ptr(buffers.req_slots), _ptr(buffers.flat_token_indices), _ptr(buffers.page_ids),
            shape.num_total_token_writes, num_active_token_writes, page_table_index))

    def invoke_prepare_bucketed(self, shape, buffers, attention_config, q_norm: "RMSNormRopeConfig",
                                k_norm: "RMSNormRopeConfig", raw_q, q_norm_weight, q_output, k_norm_weight,
                                num_active_tokens: int, page_table_index: int, q_token_stride: int = 0,
                                q_head_stride: int = 0, k_token_stride: int = 0, v_token_stride: int = 0):
        """Q norm + rope and the fused append in one launch (psi_hip_qk_norm_rope_kv_page_write);
        `attention_config` is the attention's config (it carries the Q head count)."""
        cfg, layout = attention_config.struct(), shape.page_table_layout.struct()
        qc, kc = q_norm.struct(), k_norm.struct()
        L.check(self.device.lib.psi_hip_qk_norm_rope_kv_page_write(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), ctypes.byref(qc), ctypes.byref(kc), _ptr(raw_q),
            q_token_stride, q_head_stride, _ptr(q_norm_weight), _ptr(q_output), _ptr(buffers.pages),
            _nbytes(buffers.pages), _ptr(buffers.flat_k), k_token_stride, _ptr(buffers.flat_v), v_token_stride,
            _ptr(k_norm_weight), _ptr(buffers.req_slots), _ptr(buffers.flat_token_indices), _ptr(buffers.page_ids),
            shape.num_total_token_writes, num_active_tokens, page_table_index))


# ------------------------------------------------------------------ projections around the attention


@dataclass(frozen=True)
class RopeScaling:
    """`RopeScaling::{Default, Yarn}` (components/rms_norm_rope.rs:16-27)."""
    kind: str = "Default"
    factor: float = 1.0
    attention_factor: float = 1.0
    beta_fast: float = 1.0
    beta_slow: float = 1.0
    original_max_position_embeddings: int = 1
    truncate: bool = False

    @staticmethod
    def Yarn(factor, attention_factor, beta_fast, beta_slow, original_max_position_embeddings, truncate):
        return RopeScaling("Yarn", factor, attention_factor, beta_fast, beta_slow, original_max_position_embeddings,
                           truncate)

    def struct(self):
        return L.RopeScalingStruct(1 if self.kind == "Yarn" else 0, self.factor, self.attention_factor, self.beta_fast,
                                   self.beta_slow, self.original_max_position_embeddings, 1 if self.truncate else 0)


@dataclass(frozen=True)
class RMSNormRopeConfig:
    """`RMSNormRopeConfig` (components/rms_norm_rope.rs:40-96)."""
    num_heads: int
    head_dim: int
    rope_dim: int
    eps: float
    rope_theta: float
    dtype: Dtype = Dtype.Bfloat16
    rope_scaling: RopeScaling = RopeScaling()

    def struct(self):
        return L.RMSNormRopeConfigStruct(self.num_heads, self.head_dim, self.rope_dim, self.eps, self.rope_theta,
                                         self.rope_scaling.struct(), int(self.dtype))

    def kernel_parameters(self):
        """(inverse_frequencies f32[rope_dim / 2], attention_factor, (low, high) or None): the host
        values the kernels use (`RopeScaling::kernel_parameters`)."""
        cfg = self.struct()
        inv = np.zeros(max(self.rope_dim // 2, 1), np.float32)
        factor, corr = ctypes.c_float(), (ctypes.c_float * 2)()
        L.check(L.load().psi_hip_rope_parameters(ctypes.byref(cfg), inv.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                                 ctypes.byref(factor), corr))
        return inv, factor.value, ((corr[0], corr[1]) if self.rope_scaling.kind == "Yarn" else None)


class RMSNormRopeKernel:
    """`RMSNormRopeKernel::{invoke, invoke_bucketed}` (components/rms_norm_rope.rs:252-296)."""

    def __init__(self, device: Device, config: RMSNormRopeConfig):
        config.kernel_parameters()  # validates
        self.device, self.config = device, config

    def invoke(self, num_total_tokens: int, input, norm_weight, flat_token_indices, output):
        self.invoke_bucketed(num_total_tokens, input, norm_weight, flat_token_indices, output, num_total_tokens)

    def invoke_bucketed(self, num_total_tokens: int, input, norm_weight, flat_token_indices, output,
                        num_active_tokens: int, input_token_stride: int = 0, input_head_stride: int = 0):
        cfg = self.config.struct()
        L.check(self.device.lib.psi_hip_rms_norm_rope(
            self.device.ctx, ctypes.byref(cfg), _ptr(input), input_token_stride, input_head_stride, _ptr(norm_weight),
            _ptr(flat_token_indices), _ptr(output), num_total_tokens, num_active_tokens))


class GQAQGKVSplitKernel:
    """`GQAQGKVSplitKernel::invoke_bucketed` (components/gqa_qgkv_split.rs)."""

    def __init__(self, device: Device, num_q_heads: int, num_kv_heads: int, head_dim: int, dtype: Dtype):
        self.device, self.shape, self.dtype = device, (num_q_heads, num_kv_heads, head_dim), dtype

    def invoke_bucketed(self, num_total_tokens: int, qgkv, q, g, k, v, num_active_tokens: int):
        hq, hkv, d = self.shape
        L.check(self.device.lib.psi_hip_qgkv_split(self.device.ctx, hq, hkv, d, int(self.dtype), _ptr(qgkv), _ptr(q),
                                                   _ptr(g), _ptr(k), _ptr(v), num_total_tokens, num_active_tokens))


class GQAActivationGateKernel:
    """`GQAActivationGateKernel::invoke_bucketed` (components/gqa_split_kv_single_q.rs:453-543)."""

    def __init__(self, device: Device, num_q_heads: int, head_dim: int, dtype: Dtype):
        self.device, self.shape, self.dtype = device, (num_q_heads, head_dim), dtype

    def invoke_bucketed(self, num_total_tokens: int, attention_output, g, output, num_active_tokens: int):
        hq, d = self.shape
        L.check(self.device.lib.psi_hip_activation_gate(self.device.ctx, hq, d, int(self.dtype), _ptr(attention_output),
                                                        _ptr(g), _ptr(output), num_total_tokens, num_active_tokens))


@dataclass
class OutputGate:
    """Gate operand of the combine: a tensor (or a view into the projection output: pass `offset`
    elements) with element strides per token and head."""
    gates: object
    token_stride: int
    head_stride: int
    offset: int = 0

    def struct(self):
        base = self.gates.data_ptr() + self.offset * self.gates.element_size()
        return L.OutputGateStruct(ctypes.c_void_p(base), self.token_stride, self.head_stride)


def _gate_ref(gate):
    return ctypes.byref(gate.struct()) if gate is not None else None


# ------------------------------------------------------------------ variant selection


@dataclass(frozen=True)
class GQASplitKVVariant:
    kind: str  # "SingleQ" | "TiledQ"
    kv_token_tile_size: int
    q_head_tile_size: int
    num_threads_per_threadblock: int = 0  # SingleQ only
    q_token_tile_size: int = 1  # TiledQ only

    @staticmethod
    def SingleQ(kv_token_tile_size, num_threads_per_threadblock, q_head_tile_size):
        return GQASplitKVVariant("SingleQ", kv_token_tile_size, q_head_tile_size, num_threads_per_threadblock, 1)

    @staticmethod
    def TiledQ(q_token_tile_size, kv_token_tile_size, q_head_tile_size):
        return GQASplitKVVariant("TiledQ", kv_token_tile_size, q_head_tile_size, 0, q_token_tile_size)

    def is_tiled(self) -> bool:
        return self.kind == "TiledQ"

    def struct(self):
        return L.VariantStruct(L.VARIANT_TILED_Q if self.is_tiled() else L.VARIANT_SINGLE_Q, self.q_token_tile_size,
                               self.kv_token_tile_size, self.num_threads_per_threadblock, self.q_head_tile_size)

    @staticmethod
    def from_struct(s):
        if s.kind == L.VARIANT_TILED_Q:
            return GQASplitKVVariant.TiledQ(s.q_token_tile_size, s.kv_token_tile_size, s.q_head_tile_size)
        return GQASplitKVVariant.SingleQ(s.kv_token_tile_size, s.num_threads_per_threadblock, s.q_head_tile_size)


@dataclass(frozen=True)
class GQASplitKVConfig:
    io_dtype: Dtype
    page_bytes: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int

    def struct(self):
        return _cfg_struct(self.num_q_heads, self.num_kv_heads, self.head_dim, 1.0, self.page_bytes, self.io_dtype)

    def validate(self):
        self.num_tokens_per_page()

    def q_heads_per_kv_head(self) -> int:
        return self.num_q_heads // self.num_kv_heads

    def num_tokens_per_page(self) -> int:
        return _tokens_per_page(self.struct())


class GQASplitKV:
    """Backend-owned variant selector (`GQASplitKV::new`, `new_dspark_history`, `select`)."""

    def __init__(self, config: GQASplitKVConfig, dspark_history: bool = False):
        config.validate()
        self.config, self.dspark_history = config, dspark_history

    @staticmethod
    def new(config):
        return GQASplitKV(config, False)

    @staticmethod
    def new_dspark_history(config):
        return GQASplitKV(config, True)

    def tiled_q_token_tile_size(self) -> int:
        return 8

    def max_q_tokens_per_partial_output(self) -> int:
        out, cfg = ctypes.c_uint32(), self.config.struct()
        L.check(L.load().psi_hip_split_kv_max_q_tokens_per_partial_output(ctypes.byref(cfg), int(self.dspark_history),
                                                                          ctypes.byref(out)))
        return out.value

    def select(self, num_tokens: int, num_q_token_tiles: int) -> GQASplitKVVariant:
        out, cfg = L.VariantStruct(), self.config.struct()
        L.check(L.load().psi_hip_split_kv_select(ctypes.byref(cfg), int(self.dspark_history), num_tokens,
                                                 num_q_token_tiles, ctypes.byref(out)))
        return GQASplitKVVariant.from_struct(out)


class ReplayBucketPolicy:
    def __init__(self, max_capacity: int, topology_boundaries: Sequence[int] = ()):
        self._max, self._boundaries = max_capacity, list(topology_boundaries)
        count = ctypes.c_uint32()
        b = L.u32_array(self._boundaries)
        L.check(L.load().psi_hip_replay_buckets(max_capacity, b, len(self._boundaries), None, 0, ctypes.byref(count)))
        out = (ctypes.c_uint32 * count.value)()
        L.check(L.load().psi_hip_replay_buckets(max_capacity, b, len(self._boundaries), out, count.value,
                                                ctypes.byref(count)))
        self._buckets = list(out)

    @staticmethod
    def with_topology_boundaries(max_capacity, topology_boundaries):
        return ReplayBucketPolicy(max_capacity, topology_boundaries)

    def max_capacity(self) -> int:
        return self._max

    def buckets(self) -> List[int]:
        return list(self._buckets)

    def capacity(self, active: int) -> int:
        out, b = ctypes.c_uint32(), L.u32_array(self._boundaries)
        L.check(L.load().psi_hip_replay_bucket_capacity(self._max, b, len(self._boundaries), active,
                                                        ctypes.byref(out)))
        return out.value

    def capacity_allow_zero(self, active: int) -> int:
        return 0 if active == 0 else self.capacity(active)


class GQAReplayBucketPolicy:
    def __init__(self, max_tokens: int, token_topology_boundaries: Sequence[int] = ()):
        self._max_tokens = max_tokens
        self.token_topology_boundaries = list(token_topology_boundaries)
        self.kv_splits = ReplayBucketPolicy(max_tokens)

    def max_tokens(self) -> int:
        return self._max_tokens

    def kv_split_capacity(self, num_kv_splits: int) -> int:
        return self.kv_splits.capacity(num_kv_splits)


def balanced_workers(config: "GQASplitKVConfig") -> int:
    """Decode-map workers per KV head: one workgroup per compute unit over all KV heads."""
    out, cfg = ctypes.c_uint32(), config.struct()
    L.check(L.load().psi_hip_split_kv_balanced_workers(ctypes.byref(cfg), ctypes.byref(out)))
    return out.value


def select_split_kv_variant(split_kv: GQASplitKV, max_tokens: int, replay_policy: Optional[GQAReplayBucketPolicy],
                            token_indices: Sequence[int], cu_tokens: Sequence[int]) -> GQASplitKVVariant:
    """`select_split_kv_variant` (attn/gqa/mod.rs:64-94); the (256, 8) work model applies by itself."""
    out, cfg = L.VariantStruct(), split_kv.config.struct()
    if split_kv.dspark_history:
        return split_kv.select(cu_tokens[-1], cu_tokens[-1])
    L.check(L.load().psi_hip_split_kv_select_batch(
        ctypes.byref(cfg), max_tokens, replay_policy.max_tokens() if replay_policy else 0,
        L.u32_array(token_indices), L.u32_array(cu_tokens), len(token_indices), ctypes.byref(out)))
    return GQASplitKVVariant.from_struct(out)


# ------------------------------------------------------------------ batch metadata


@dataclass(frozen=True)
class GQAReplayShape:
    num_tokens: int
    num_total_tokens: int
    num_q_token_tiles: int
    num_total_q_token_tiles: int
    num_sdpa_map_task_templates: int
    num_total_sdpa_map_task_templates: int
    reduce_sdpa_partial_outputs: bool


class GQAMetadataBuffers:
    """Capacity-sized metadata refreshed per microbatch: host arrays plus device copies."""

    def __init__(self, device: Optional[Device], max_tokens: int, max_kv_splits: Optional[int] = None):
        assert max_tokens > 0, "GQA batch metadata requires tokens"
        self.device, self._max_tokens = device, max_tokens
        self._max_kv_splits = max_kv_splits if max_kv_splits is not None else max_tokens
        self.h_req_slots = np.zeros(max_tokens, np.uint32)
        self.h_flat_token_indices = np.zeros(max_tokens, np.uint32)
        self.h_q_token_tiles = np.zeros(max_tokens * 2, np.uint32)
        self.h_kv_splits = np.zeros(self._max_kv_splits * 3, np.uint32)
        self.h_cu_kv_splits = np.zeros(max_tokens + 1, np.uint32)
        self._shape, self._variant = None, None
        self.d_req_slots = self.d_flat_token_indices = self.d_q_token_tiles = None
        self.d_kv_splits = self.d_cu_kv_splits = None
        self.h_partial_row_index = self.d_partial_row_index = None
        self.h_row_groups = self.d_row_groups = None
        self.group_tiles = self.num_row_groups = 0

    def max_tokens(self) -> int:
        return self._max_tokens

    def _update(self, req_slots, token_indices, cu_tokens, variant, mode, caller_tokens=0, boundaries=(),
                partition_tokens=0):
        assert len(req_slots) == len(token_indices) and len(cu_tokens) == len(req_slots) + 1
        shape = L.ReplayShapeStruct()
        v = variant.struct()

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        L.check(L.load().psi_hip_gqa_metadata_update(
            self._max_tokens, L.u32_array(req_slots), L.u32_array(token_indices), L.u32_array(cu_tokens),
            len(req_slots), ctypes.byref(v), mode, caller_tokens, L.u32_array(boundaries), len(boundaries),
            partition_tokens, self._max_kv_splits, p(self.h_req_slots), p(self.h_flat_token_indices),
            p(self.h_q_token_tiles), p(self.h_kv_splits), p(self.h_cu_kv_splits), ctypes.byref(shape)))
        self._shape = GQAReplayShape(shape.num_tokens, shape.num_total_tokens, shape.num_q_token_tiles,
                                     shape.num_total_q_token_tiles, shape.num_kv_splits, shape.num_total_kv_splits,
                                     bool(shape.reduce_sdpa_partial_outputs))
        self._variant = variant
        self.h_partial_row_index = self.d_partial_row_index = None  # rows are in plan order again
        self.h_row_groups = self.d_row_groups = None
        self.group_tiles = self.num_row_groups = 0
        if self.device is not None:
            self.upload()
        return self._shape

    def upload(self):
        d = self.device
        self.d_req_slots = d.from_numpy(self.h_req_slots)
        self.d_flat_token_indices = d.from_numpy(self.h_flat_token_indices)
        self.d_q_token_tiles = d.from_numpy(self.h_q_token_tiles)
        self.d_kv_splits = d.from_numpy(self.h_kv_splits)
        self.d_cu_kv_splits = d.from_numpy(self.h_cu_kv_splits)

    def update(self, req_slots, token_indices, cu_tokens, split_kv_variant):
        return self._update(req_slots, token_indices, cu_tokens, split_kv_variant, L.CAPACITY_EXACT)

    def update_bucketed(self, req_slots, token_indices, cu_tokens, split_kv_variant, policy: GQAReplayBucketPolicy):
        assert policy.max_tokens() == self._max_tokens, \
            "GQA replay bucket policy must match metadata token capacity"
        return self._update(req_slots, token_indices, cu_tokens, split_kv_variant, L.CAPACITY_BUCKETED,
                            boundaries=policy.token_topology_boundaries)

    def update_bucketed_with_token_capacity(self, req_slots, token_indices, cu_tokens, split_kv_variant, policy,
                                            num_total_tokens: int):
        assert policy.max_tokens() == self._max_tokens, \
            "GQA replay bucket policy must match metadata token capacity"
        return self._update(req_slots, token_indices, cu_tokens, split_kv_variant, L.CAPACITY_CALLER_TOKENS,
                            caller_tokens=num_total_tokens, boundaries=policy.token_topology_boundaries)

    def update_fixed_partition(self, req_slots, token_indices, cu_tokens, split_kv_variant, partition_tokens: int):
        """Fixed-length KV partitions (not in the reference): ceil(ctx / partition) splits per row."""
        return self._update(req_slots, token_indices, cu_tokens, split_kv_variant, L.CAPACITY_FIXED_PARTITION,
                            partition_tokens=partition_tokens)

    def order_longest_first(self):
        """Re-orders the planned rows for dispatch (psi_hip_split_kv_order_longest_first): longest
        rows first.  `d_partial_row_index` must then be passed to the combine."""
        s = self._shape
        n = s.num_sdpa_map_task_templates
        self.h_partial_row_index = np.zeros(max(len(self.h_kv_splits) // 3, 1), np.uint32)
        self.h_partial_row_index[:] = np.arange(len(self.h_partial_row_index), dtype=np.uint32)

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        L.check(L.load().psi_hip_split_kv_order_longest_first(p(self.h_kv_splits), n, p(self.h_partial_row_index)))
        if self.device is not None:
            self.upload()
            self.d_partial_row_index = self.device.from_numpy(self.h_partial_row_index)
        return self.h_partial_row_index

    def group_rows(self, config) -> int:
        """Row groups of the current TiledQ plan for the prefill-chunk map
        (psi_hip_split_kv_tiled_q_group_rows); `config` is the kernels' GQASplitKVTiledQConfig.
        Returns the number of groups, 0 when the geometry has no grouped kernel.  Call after any
        re-ordering of the rows: the table holds row positions."""
        s = self._shape
        assert s is not None and self._variant.is_tiled()
        n = s.num_sdpa_map_task_templates
        table = np.full(max(n, 1) * 32, L.SENTINEL, np.uint32)
        tiles, groups = ctypes.c_uint32(), ctypes.c_uint32()
        cfg = config.struct()

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        L.check(L.load().psi_hip_split_kv_tiled_q_group_rows(
            ctypes.byref(cfg), config.q_token_tile_size, p(self.h_kv_splits), n, p(self.h_q_token_tiles),
            s.num_q_token_tiles, p(self.h_req_slots), p(table), len(table), ctypes.byref(tiles), ctypes.byref(groups)))
        self.group_tiles, self.num_row_groups = tiles.value, groups.value
        self.h_row_groups = table[:max(tiles.value * groups.value, 1)].copy()
        if self.device is not None and groups.value:
            self.d_row_groups = self.device.from_numpy(self.h_row_groups)
        return groups.value

    def balance(self, num_workers: int):
        """Re-cuts the current SingleQ plan into rows grouped for `num_workers` equal-work decode
        workgroups per KV head (psi_hip_split_kv_balance_plan); adjacent pieces of one token inside a group
        become one row.  Returns the new replay shape."""
        s = self._shape
        assert s is not None
        groups = s.num_q_token_tiles if self._variant.is_tiled() else s.num_tokens  # what cu_kv_splits counts
        rows_in = s.num_sdpa_map_task_templates
        cap = max(rows_in + num_workers, self._max_kv_splits)  # the arrays are reused by the next update
        out_splits = np.full(cap * 3, L.SENTINEL, np.uint32)
        out_cu = np.zeros(self._max_tokens + 1, np.uint32)
        worker_cu = np.zeros(num_workers + 1, np.uint32)
        n_out = ctypes.c_uint32()

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        L.check(L.load().psi_hip_split_kv_balance_plan(p(self.h_kv_splits), rows_in, p(self.h_cu_kv_splits),
                                                       groups, num_workers, p(out_splits), cap, p(out_cu),
                                                       p(worker_cu), ctypes.byref(n_out)))
        self.h_kv_splits, self.h_cu_kv_splits, self.h_worker_cu = out_splits, out_cu, worker_cu
        self.num_workers = num_workers
        self._shape = GQAReplayShape(s.num_tokens, s.num_total_tokens, s.num_q_token_tiles,
                                     s.num_total_q_token_tiles, n_out.value, n_out.value, True)
        if self.device is not None:
            self.upload()
            self.d_worker_cu = self.device.from_numpy(worker_cu)
        return self._shape

    def replay_shape(self) -> GQAReplayShape:
        assert self._shape is not None, "GQA batch metadata must be updated before recording"
        return self._shape

    def split_kv_variant(self) -> GQASplitKVVariant:
        assert self._variant is not None, "GQA batch metadata must be updated before recording"
        return self._variant


# ------------------------------------------------------------------ request page table


class GQARequestPageTable:
    def __init__(self, device: Device, layout: GQAPageTableLayout):
        import torch

        layout.validate()
        self.device, self.layout = device, layout
        self.page_ids = torch.zeros(layout.num_page_ids(), dtype=torch.int32, device=device.torch_device)

    def layout_struct(self):
        return self.layout.struct()

    def page_ids_buffer(self):
        return self.page_ids

    def num_req_slots(self):
        return self.layout.num_req_slots

    def num_layers(self):
        return self.layout.num_gqa_layers

    def num_blocks(self):
        return self.layout.num_blocks

    def num_page_ids_per_block(self):
        return self.layout.num_page_ids_per_block

    def start_index(self, req_slot, layer_index, block_index) -> int:
        out, layout = ctypes.c_uint64(), self.layout.struct()
        L.check(self.device.lib.psi_hip_page_table_start_index(ctypes.byref(layout), req_slot, layer_index,
                                                               block_index, ctypes.byref(out)))
        return out.value

    def write_page_ids(self, req_slot, layer_index, block_index, page_ids, num_cache_pages: int = 0):
        layout = self.layout.struct()
        L.check(self.device.lib.psi_hip_page_table_write_page_ids(
            self.device.ctx, ctypes.byref(layout), _ptr(self.page_ids), req_slot, layer_index, block_index,
            L.u32_array(page_ids), len(page_ids), num_cache_pages))

    def read_page_ids(self, req_slot, layer_index, block_index) -> List[int]:
        start = self.start_index(req_slot, layer_index, block_index)
        self.device.sync()
        n = self.layout.num_page_ids_per_block
        return [int(v) & 0xFFFFFFFF for v in self.page_ids[start:start + n].cpu().tolist()]

    def reset_req_slot(self, req_slot):
        layout = self.layout.struct()
        L.check(self.device.lib.psi_hip_page_table_reset_req_slot(self.device.ctx, ctypes.byref(layout),
                                                                  _ptr(self.page_ids), req_slot))

    def reset_req_slots(self, req_slots):
        for s in req_slots:
            self.reset_req_slot(s)


# ------------------------------------------------------------------ SingleQ decode


@dataclass(frozen=True)
class GQASplitKVSingleQConfig:
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    page_bytes: int
    page_table_layout: GQAPageTableLayout
    kv_token_tile_size: int
    num_threads_per_threadblock: int
    q_head_tile_size: int
    dtype: Dtype

    def struct(self):
        return _cfg_struct(self.num_q_heads, self.num_kv_heads, self.head_dim, self.scale, self.page_bytes,
                           self.dtype)

    def num_tokens_per_page(self) -> int:
        return _tokens_per_page(self.struct())

    def q_heads_per_kv_head(self) -> int:
        return self.num_q_heads // self.num_kv_heads

    def num_output_values(self, shape) -> int:
        return shape.num_total_tokens * self.num_q_heads * self.head_dim


@dataclass(frozen=True)
class GQASplitKVSingleQShape:
    num_total_tokens: int
    num_total_sdpa_map_task_templates: int


class GQASplitKVSingleQScratch:
    """Partial-state scratch sized by the library (`GQASplitKVSingleQScratch::new`)."""

    def __init__(self, device: Device, config: GQASplitKVSingleQConfig, shape: GQASplitKVSingleQShape, fill=None):
        import torch

        out, cfg = ctypes.c_uint64(), config.struct()
        L.check(device.lib.psi_hip_split_kv_single_q_scratch_bytes(
            ctypes.byref(cfg), shape.num_total_sdpa_map_task_templates, ctypes.byref(out)))
        self.bytes = out.value
        self.buffer = torch.zeros(self.bytes, dtype=torch.uint8, device=device.torch_device)
        if fill is not None:
            self.buffer.fill_(fill)


class GQASplitKVSingleQKernels:
    def __init__(self, device: Device, config: GQASplitKVSingleQConfig, shape: GQASplitKVSingleQShape):
        config.num_tokens_per_page()
        self.device, self.config, self.shape = device, config, shape

    def invoke_map(self, q, kv_pages, req_slots, page_ids, sdpa_map_task_templates, scratch, page_table_index: int):
        self.invoke_map_bucketed(q, kv_pages, req_slots, page_ids, sdpa_map_task_templates, scratch,
                                 page_table_index, self.shape.num_total_tokens,
                                 self.shape.num_total_sdpa_map_task_templates)

    def invoke_map_bucketed(self, q, kv_pages, req_slots, page_ids, sdpa_map_task_templates, scratch,
                            page_table_index: int, num_active_tokens: int, num_active_kv_splits: int):
        cfg, layout = self.config.struct(), self.config.page_table_layout.struct()
        L.check(self.device.lib.psi_hip_split_kv_single_q_map(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), _ptr(q), _ptr(kv_pages), _nbytes(kv_pages),
            _ptr(req_slots), _ptr(page_ids), _ptr(sdpa_map_task_templates), _ptr(scratch.buffer), scratch.bytes,
            page_table_index, self.shape.num_total_tokens, self.shape.num_total_sdpa_map_task_templates,
            num_active_tokens, num_active_kv_splits))

    def invoke_append_map_bucketed(self, q, kv_pages, flat_k, flat_v, req_slots, flat_token_indices, page_ids,
                                   sdpa_map_task_templates, scratch, page_table_index: int, num_active_tokens: int,
                                   num_active_kv_splits: int, worker_cu=None, num_workers: int = 0):
        """`GQAKVPageWrite.invoke_bucketed` and `invoke_map_bucketed` in one launch: the workgroup whose split row
        ends at a token's position writes the token's K/V lines, and the step's new positions are read from
        `flat_k` / `flat_v`.  Same arena as the two calls bit for bit; partial states equal up to summation order."""
        cfg, layout = self.config.struct(), self.config.page_table_layout.struct()
        L.check(self.device.lib.psi_hip_kv_page_write_split_kv_single_q_map(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), _ptr(q), _ptr(kv_pages), _nbytes(kv_pages),
            _ptr(flat_k), _ptr(flat_v), _ptr(req_slots), _ptr(flat_token_indices), _ptr(page_ids),
            _ptr(sdpa_map_task_templates), _ptr(worker_cu), num_workers, _ptr(scratch.buffer), scratch.bytes,
            page_table_index, self.shape.num_total_tokens, self.shape.num_total_sdpa_map_task_templates,
            num_active_tokens, num_active_kv_splits))

    def invoke_map_balanced(self, q, kv_pages, req_slots, page_ids, sdpa_map_task_templates, worker_cu,
                            num_workers: int, scratch, page_table_index: int, num_active_tokens: int,
                            num_active_kv_splits: int):
        """The map over a balanced plan: one workgroup per (worker, KV head) walks its row range."""
        cfg, layout = self.config.struct(), self.config.page_table_layout.struct()
        L.check(self.device.lib.psi_hip_split_kv_single_q_map_balanced(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), _ptr(q), _ptr(kv_pages), _nbytes(kv_pages),
            _ptr(req_slots), _ptr(page_ids), _ptr(sdpa_map_task_templates), _ptr(worker_cu), num_workers,
            _ptr(scratch.buffer), scratch.bytes, page_table_index, self.shape.num_total_tokens,
            self.shape.num_total_sdpa_map_task_templates, num_active_tokens, num_active_kv_splits))

    def invoke_store_partials(self, scratch, slot_rows, partial_exp_sums, partial_max_logits, partial_output,
                              num_active_tokens: int, partial_row_index=None):
        """Enters another attention task's partial results (one per token and query head, in the form
        `gqa_block_sdpa.metal` writes them) into the split rows the map skips for them; call between the map
        and the reduce.  `slot_rows[t]`: the split row reserved for token t."""
        cfg = self.config.struct()
        L.check(self.device.lib.psi_hip_split_kv_single_q_store_partials(
            self.device.ctx, ctypes.byref(cfg), _ptr(scratch.buffer), scratch.bytes, _ptr(slot_rows),
            _ptr(partial_exp_sums), _ptr(partial_max_logits), _ptr(partial_output), self.shape.num_total_tokens,
            self.shape.num_total_sdpa_map_task_templates, num_active_tokens, _ptr(partial_row_index)))

    def invoke_reduce(self, scratch, cu_sdpa_partial_outputs, output):
        self.invoke_reduce_bucketed(scratch, cu_sdpa_partial_outputs, output, self.shape.num_total_tokens)

    def invoke_reduce_bucketed(self, scratch, cu_sdpa_partial_outputs, output, num_active_tokens: int,
                               partial_row_index=None, gate: Optional["OutputGate"] = None):
        """`gate`: fuses the sigmoid gate of a gated GQA layer into the combine."""
        cfg = self.config.struct()
        L.check(self.device.lib.psi_hip_split_kv_single_q_reduce(
            self.device.ctx, ctypes.byref(cfg), _ptr(scratch.buffer), scratch.bytes, _ptr(cu_sdpa_partial_outputs),
            _ptr(output), self.shape.num_total_tokens, self.shape.num_total_sdpa_map_task_templates,
            num_active_tokens, _ptr(partial_row_index), _gate_ref(gate)))


# ------------------------------------------------------------------ TiledQ verify / prefill


@dataclass(frozen=True)
class GQASplitKVTiledQConfig:
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    q_head_tile_size: int
    q_token_tile_size: int
    kv_token_tile_size: int
    scale: float
    page_bytes: int
    dtype: Dtype
    page_table_layout: GQAPageTableLayout

    def struct(self):
        return _cfg_struct(self.num_q_heads, self.num_kv_heads, self.head_dim, self.scale, self.page_bytes,
                           self.dtype)

    def num_tokens_per_page(self) -> int:
        return _tokens_per_page(self.struct())


@dataclass(frozen=True)
class GQASplitKVTiledQShape:
    num_total_tokens: int
    num_total_q_token_tiles: int
    num_total_sdpa_map_task_templates: int


class GQASplitKVTiledQScratch:
    def __init__(self, device: Device, config: GQASplitKVTiledQConfig, shape: GQASplitKVTiledQShape, fill=None):
        import torch

        out, cfg = ctypes.c_uint64(), config.struct()
        L.check(device.lib.psi_hip_split_kv_tiled_q_scratch_bytes(
            ctypes.byref(cfg), config.q_token_tile_size, shape.num_total_sdpa_map_task_templates, ctypes.byref(out)))
        self.bytes = out.value
        self.buffer = torch.zeros(self.bytes, dtype=torch.uint8, device=device.torch_device)
        if fill is not None:
            self.buffer.fill_(fill)


class GQASplitKVTiledQKernels:
    def __init__(self, device: Device, config: GQASplitKVTiledQConfig, shape: GQASplitKVTiledQShape):
        config.num_tokens_per_page()
        self.device, self.config, self.shape = device, config, shape

    def invoke_map(self, q, kv_pages, req_slots, page_ids, flat_token_indices, q_token_tiles,
                   sdpa_map_task_templates, scratch, page_table_index: int):
        s = self.shape
        self.invoke_map_bucketed(q, kv_pages, req_slots, page_ids, flat_token_indices, q_token_tiles,
                                 sdpa_map_task_templates, scratch, page_table_index, s.num_total_tokens,
                                 s.num_total_q_token_tiles, s.num_total_sdpa_map_task_templates)

    def invoke_map_bucketed(self, q, kv_pages, req_slots, page_ids, flat_token_indices, q_token_tiles,
                            sdpa_map_task_templates, scratch, page_table_index: int, num_active_tokens: int,
                            num_active_q_token_tiles: int, num_active_kv_splits: int,
                            max_active_q_tile_tokens: int = 0):
        """`max_active_q_tile_tokens`: the largest tile of this batch (2 for a one-draft verify step);
        0 = unknown, any tile may be full."""
        cfg, layout, s = self.config.struct(), self.config.page_table_layout.struct(), self.shape
        L.check(self.device.lib.psi_hip_split_kv_tiled_q_map(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), self.config.q_token_tile_size, _ptr(q),
            _ptr(kv_pages), _nbytes(kv_pages), _ptr(req_slots), _ptr(page_ids), _ptr(flat_token_indices),
            _ptr(q_token_tiles), _ptr(sdpa_map_task_templates), _ptr(scratch.buffer), scratch.bytes,
            page_table_index, s.num_total_tokens, s.num_total_q_token_tiles, s.num_total_sdpa_map_task_templates,
            num_active_tokens, num_active_q_token_tiles, num_active_kv_splits, max_active_q_tile_tokens))

    def invoke_map_balanced(self, q, kv_pages, req_slots, page_ids, flat_token_indices, q_token_tiles,
                            sdpa_map_task_templates, worker_cu, num_workers: int, scratch, page_table_index: int,
                            num_active_tokens: int, num_active_q_token_tiles: int, num_active_kv_splits: int,
                            max_active_q_tile_tokens: int = 0):
        """The map over a balanced plan: one workgroup per (worker, KV head) walks its row range."""
        cfg, layout, s = self.config.struct(), self.config.page_table_layout.struct(), self.shape
        L.check(self.device.lib.psi_hip_split_kv_tiled_q_map_balanced(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), self.config.q_token_tile_size, _ptr(q),
            _ptr(kv_pages), _nbytes(kv_pages), _ptr(req_slots), _ptr(page_ids), _ptr(flat_token_indices),
            _ptr(q_token_tiles), _ptr(sdpa_map_task_templates), _ptr(worker_cu), num_workers, _ptr(scratch.buffer),
            scratch.bytes, page_table_index, s.num_total_tokens, s.num_total_q_token_tiles,
            s.num_total_sdpa_map_task_templates, num_active_tokens, num_active_q_token_tiles, num_active_kv_splits,
            max_active_q_tile_tokens))

    def invoke_map_grouped(self, q, kv_pages, req_slots, page_ids, flat_token_indices, q_token_tiles,
                           sdpa_map_task_templates, scratch, page_table_index: int, num_active_tokens: int,
                           num_active_q_token_tiles: int, num_active_kv_splits: int, row_groups, group_tiles: int,
                           num_groups: int, max_active_q_tile_tokens: int = 0):
        """The map with one workgroup per row group (prefill chunks); `row_groups` is the device copy
        of GQAMetadataBuffers.group_rows()."""
        cfg, layout, s = self.config.struct(), self.config.page_table_layout.struct(), self.shape
        L.check(self.device.lib.psi_hip_split_kv_tiled_q_map_grouped(
            self.device.ctx, ctypes.byref(cfg), ctypes.byref(layout), self.config.q_token_tile_size, _ptr(q),
            _ptr(kv_pages), _nbytes(kv_pages), _ptr(req_slots), _ptr(page_ids), _ptr(flat_token_indices),
            _ptr(q_token_tiles), _ptr(sdpa_map_task_templates), _ptr(scratch.buffer), scratch.bytes,
            page_table_index, s.num_total_tokens, s.num_total_q_token_tiles, s.num_total_sdpa_map_task_templates,
            num_active_tokens, num_active_q_token_tiles, num_active_kv_splits, max_active_q_tile_tokens,
            _ptr(row_groups), group_tiles, num_groups))

    def invoke_reduce(self, scratch, q_token_tiles, cu_sdpa_partial_outputs, output):
        self.invoke_reduce_bucketed(scratch, q_token_tiles, cu_sdpa_partial_outputs, output,
                                    self.shape.num_total_q_token_tiles)

    def invoke_reduce_bucketed(self, scratch, q_token_tiles, cu_sdpa_partial_outputs, output,
                               num_active_q_token_tiles: int, partial_row_index=None,
                               gate: Optional["OutputGate"] = None):
        cfg, s = self.config.struct(), self.shape
        L.check(self.device.lib.psi_hip_split_kv_tiled_q_reduce(
            self.device.ctx, ctypes.byref(cfg), self.config.q_token_tile_size, _ptr(scratch.buffer), scratch.bytes,
            _ptr(q_token_tiles), _ptr(cu_sdpa_partial_outputs), _ptr(output), s.num_total_tokens,
            s.num_total_q_token_tiles, s.num_total_sdpa_map_task_templates, num_active_q_token_tiles,
            _ptr(partial_row_index), _gate_ref(gate)))
