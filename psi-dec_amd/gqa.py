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
    return t.numel() * t.element_size() if t is not None else 0


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

    def mute_loaders(self, on: bool):
        """For harnesses: the loading waves of the multi-query and prefill-chunk maps never say that a tile has
        landed, so that the other waves' bounded waits run out and the device error path runs, while every kernel
        still ends normally."""
        L.check(self.lib.psi_hip_ctx_set_flag(self.ctx, L.FLAG_MUTE_LOADERS, int(on)))

    def take_device_error(self) -> int:
        """Synchronises, then returns and clears the errors that kernels reported (`L.DEVICE_ERR_*` bits);
        `sync()` raises while one is set."""
        bits = ctypes.c_uint32()
        L.check(self.lib.psi_hip_ctx_take_device_error(self.ctx, ctypes.byref(bits)))
        return bits.value

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


def chunk_partition_tokens(config, q_token_tile_size: int, token_indices: Sequence[int], cu_tokens: Sequence[int],
                           num_compute_units: int = 0) -> int:
    """Partition length (tokens) for a FIXED_PARTITION plan of a batch of prefill chunks that the row-group map and its
    combine finish soonest with, by the library's model of that launch (psi_hip_split_kv_chunk_partition_tokens);
    `config` is any of the kernels' configs (it gives the heads, head_dim and page size), token_indices[r] the position
    of request r's first new token, cu_tokens the prefix sums of the new tokens.  0: the geometry has no row-group
    kernel.  Depends on the lengths only; cache it per shape class."""
    out, cfg = ctypes.c_uint32(), config.struct()
    L.check(L.load().psi_hip_split_kv_chunk_partition_tokens(
        ctypes.byref(cfg), q_token_tile_size, L.u32_array(token_indices), L.u32_array(cu_tokens), len(token_indices),
        num_compute_units, ctypes.byref(out)))
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
    """Capacity-sized metadata refreshed per microbatch (`GQAMetadataBuffers`, batch_metadata.rs:71-126).

    With a device, the host arrays are views into one pinned staging buffer and the device arrays views into one
    device buffer of the same layout: both keep their addresses for the object's lifetime (a recorded program
    holds them), and `upload()` is one or two asynchronous copies on the device's stream.  Without a device
    (`None`) only the host arrays exist.  `max_workers`: room for the rows a balanced worker plan may add."""

    def __init__(self, device: Optional[Device], max_tokens: int, max_kv_splits: Optional[int] = None,
                 max_workers: int = 256):
        assert max_tokens > 0, "GQA batch metadata requires tokens"
        self.device, self._max_tokens = device, max_tokens
        self._max_kv_splits = max_kv_splits if max_kv_splits is not None else max_tokens
        self._max_workers = max_workers
        rows = self._max_kv_splits + max_workers
        # replay_counts: the four words a recorded program reads its active counts from; they travel with the arrays
        sizes = (("replay_counts", 4), ("req_slots", max_tokens), ("flat_token_indices", max_tokens),
                 ("q_token_tiles", 2 * max_tokens),
                 ("cu_kv_splits", max_tokens + 1), ("worker_cu", max_workers + 1), ("kv_splits", 3 * rows),
                 ("partial_row_index", rows))
        self._offsets, total = {}, 0
        for name, n in sizes:
            self._offsets[name] = (total, n)
            total += n
        self._words = total
        if device is not None:
            import torch

            self._h_all_t = torch.zeros(total, dtype=torch.int32, pin_memory=True)
            h_all = self._h_all_t.numpy().view(np.uint32)
            self._d_all = torch.zeros(total, dtype=torch.int32, device=device.torch_device)
        else:
            h_all = np.zeros(total, np.uint32)
            self._d_all = None

        def host(name, used=None):
            off, n = self._offsets[name]
            return h_all[off:off + (n if used is None else used)]

        def dev(name):
            if self._d_all is None:
                return None
            off, n = self._offsets[name]
            return self._d_all[off:off + n]

        self.h_replay_counts, self.d_replay_counts = host("replay_counts"), dev("replay_counts")
        self.h_req_slots, self.d_req_slots = host("req_slots"), dev("req_slots")
        self.h_flat_token_indices, self.d_flat_token_indices = host("flat_token_indices"), dev("flat_token_indices")
        self.h_q_token_tiles, self.d_q_token_tiles = host("q_token_tiles"), dev("q_token_tiles")
        self.h_cu_kv_splits, self.d_cu_kv_splits = host("cu_kv_splits"), dev("cu_kv_splits")
        self._h_worker_cu_all, self._d_worker_cu_all = host("worker_cu"), dev("worker_cu")
        self._h_kv_splits_all = host("kv_splits")
        self.h_kv_splits = self._h_kv_splits_all[:3 * self._max_kv_splits]  # what the planner may fill
        self.d_kv_splits = dev("kv_splits")
        self._h_row_index_all, self._d_row_index_all = host("partial_row_index"), dev("partial_row_index")
        self._shape, self._variant = None, None
        self.h_partial_row_index = self.d_partial_row_index = None
        self.h_worker_cu = self.d_worker_cu = None
        self.num_workers = 0
        self.h_row_groups = self.d_row_groups = None
        self._h_row_groups_t = self._d_row_groups_all = self._h_row_groups_all = None
        self._host_struct = None
        self.group_tiles = self.num_row_groups = 0
        self.max_active_q_tile_tokens = 0
        self._uploaded = None  # event after the last upload: the staging buffer is free again once it has passed

    def max_tokens(self) -> int:
        return self._max_tokens

    def _staging_free(self):
        if self._uploaded is not None:
            self._uploaded.synchronize()
            self._uploaded = None

    def _update(self, req_slots, token_indices, cu_tokens, variant, mode, caller_tokens=0, boundaries=(),
                partition_tokens=0):
        assert len(req_slots) == len(token_indices) and len(cu_tokens) == len(req_slots) + 1
        shape = L.ReplayShapeStruct()
        v = variant.struct()

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        self._staging_free()
        self.h_kv_splits = self._h_kv_splits_all[:3 * self._max_kv_splits]
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
        self.h_worker_cu = self.d_worker_cu = None
        self.num_workers = 0
        self.h_row_groups = self.d_row_groups = None
        self.group_tiles = self.num_row_groups = 0
        q_lens = np.diff(np.asarray(cu_tokens, dtype=np.int64))
        self.max_active_q_tile_tokens = (int(min(q_lens.max(), variant.q_token_tile_size)) if variant.is_tiled()
                                         else 0)
        if self.device is not None:
            self.upload()
        return self._shape

    def upload(self):
        """Host arrays -> their device copies, asynchronously on the device's stream (pinned staging, fixed
        device addresses).  Everything up to the last planned row of kv_splits goes in one copy."""
        if self.device is None:
            return
        import torch

        rows = self._shape.num_total_sdpa_map_task_templates if self._shape is not None else 0
        if self._shape is not None:  # the layer word stays 0: programs that read these counts hold their layer
            self.h_replay_counts[:] = (self._shape.num_tokens, self._shape.num_q_token_tiles,
                                       self._shape.num_sdpa_map_task_templates, 0)
        off, _ = self._offsets["kv_splits"]
        end = off + 3 * rows
        with torch.cuda.stream(self.device.stream):
            self._d_all[:end].copy_(self._h_all_t[:end], non_blocking=True)
            if self.h_partial_row_index is not None:
                o, _ = self._offsets["partial_row_index"]
                self._d_all[o:o + rows].copy_(self._h_all_t[o:o + rows], non_blocking=True)
            self._uploaded = torch.cuda.Event()
            self._uploaded.record(self.device.stream)

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
        self._staging_free()
        self.h_partial_row_index = self._h_row_index_all
        self.h_partial_row_index[:] = np.arange(len(self.h_partial_row_index), dtype=np.uint32)

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        L.check(L.load().psi_hip_split_kv_order_longest_first(p(self.h_kv_splits), n, p(self.h_partial_row_index)))
        if self.device is not None:
            self.d_partial_row_index = self._d_row_index_all
            self.upload()
        return self.h_partial_row_index

    def group_rows(self, config) -> int:
        """Row groups of the current TiledQ plan for the prefill-chunk map
        (psi_hip_split_kv_tiled_q_group_rows); `config` is the kernels' GQASplitKVTiledQConfig.
        Returns the number of groups, 0 when the geometry has no grouped kernel.  Call after any
        re-ordering of the rows: the table holds row positions."""
        s = self._shape
        assert s is not None and self._variant.is_tiled()
        n = s.num_sdpa_map_task_templates
        words = max(n, 1) * 32
        if self._row_groups_words() < words:
            self._alloc_row_groups(words)
        table = self._h_row_groups_all[:words]
        table[:] = L.SENTINEL
        tiles, groups = ctypes.c_uint32(), ctypes.c_uint32()
        cfg = config.struct()

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        L.check(L.load().psi_hip_split_kv_tiled_q_group_rows(
            ctypes.byref(cfg), config.q_token_tile_size, p(self.h_kv_splits), n, p(self.h_q_token_tiles),
            s.num_q_token_tiles, p(self.h_req_slots), p(table), len(table), ctypes.byref(tiles), ctypes.byref(groups)))
        self.group_tiles, self.num_row_groups = tiles.value, groups.value
        used = max(tiles.value * groups.value, 1)
        self.h_row_groups = table[:used]
        if self.device is not None and groups.value:
            import torch

            with torch.cuda.stream(self.device.stream):
                self._d_row_groups_all[:used].copy_(self._h_row_groups_t[:used], non_blocking=True)
            self.d_row_groups = self._d_row_groups_all
        return groups.value

    def balance(self, num_workers: int):
        """Re-cuts the current plan into rows grouped for `num_workers` equal-work map workgroups per KV head
        (psi_hip_split_kv_balance_plan); adjacent pieces of one token inside a group become one row.  Returns the
        new replay shape."""
        s = self._shape
        assert s is not None
        assert num_workers <= self._max_workers, "more workers than the metadata buffers reserve rows for"
        groups = s.num_q_token_tiles if self._variant.is_tiled() else s.num_tokens  # what cu_kv_splits counts
        rows_in = s.num_sdpa_map_task_templates
        cap = self._max_kv_splits + self._max_workers
        assert rows_in + num_workers <= cap
        out_splits = np.full(cap * 3, L.SENTINEL, np.uint32)
        out_cu = np.zeros(self._max_tokens + 1, np.uint32)
        worker_cu = np.zeros(num_workers + 1, np.uint32)
        n_out = ctypes.c_uint32()

        def p(a):
            return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32))

        L.check(L.load().psi_hip_split_kv_balance_plan(p(self.h_kv_splits), rows_in, p(self.h_cu_kv_splits),
                                                       groups, num_workers, p(out_splits), cap, p(out_cu),
                                                       p(worker_cu), ctypes.byref(n_out)))
        self._staging_free()
        self.h_kv_splits = self._h_kv_splits_all
        self.h_kv_splits[:] = out_splits
        self.h_cu_kv_splits[:] = out_cu
        self.h_worker_cu = self._h_worker_cu_all[:num_workers + 1]
        self.h_worker_cu[:] = worker_cu
        self.num_workers = num_workers
        self._shape = GQAReplayShape(s.num_tokens, s.num_total_tokens, s.num_q_token_tiles,
                                     s.num_total_q_token_tiles, n_out.value, n_out.value, True)
        if self.device is not None:
            self.d_worker_cu = self._d_worker_cu_all
            self.upload()
        return self._shape

    def prepare(self, layer_struct, req_slots, token_indices, cu_tokens, capacity_mode=L.CAPACITY_EXACT,
                partition_tokens: int = 0, dispatch: int = L.DISPATCH_PLAN_ORDER, num_workers: int = 0,
                variant: Optional[GQASplitKVVariant] = None, policy: Optional[GQAReplayBucketPolicy] = None,
                caller_num_total_tokens: int = 0, bucket_capacities: bool = False) -> GQAReplayShape:
        """One host call for the whole of a step's planning (psi_hip_gqa_layer_prepare): variant selection when
        `variant` is None, metadata update, dispatch plan; then one upload.  `layer_struct`: `GQA.struct()`."""
        self._staging_free()
        rs = np.ascontiguousarray(req_slots, dtype=np.uint32)
        ti = np.ascontiguousarray(token_indices, dtype=np.uint32)
        cu = np.ascontiguousarray(cu_tokens, dtype=np.uint32)
        assert len(rs) == len(ti) and len(cu) == len(rs) + 1
        boundaries = L.u32_array(policy.token_topology_boundaries) if policy is not None else None
        options = L.PlanOptionsStruct(capacity_mode, partition_tokens, caller_num_total_tokens, dispatch, num_workers,
                                      policy.max_tokens() if policy is not None else 0, boundaries,
                                      len(policy.token_topology_boundaries) if policy is not None else 0,
                                      int(bucket_capacities))
        host = self._host_metadata(dispatch)
        plan, uses = L.BatchMetadataStruct(), ctypes.c_uint32()
        v = variant.struct() if variant is not None else None
        self._last_prepare = (options, plan, uses, boundaries)  # what advance_decode() continues from
        L.check(L.load().psi_hip_gqa_layer_prepare(
            ctypes.byref(layer_struct), ctypes.byref(options), rs.ctypes.data, ti.ctypes.data, cu.ctypes.data, len(rs),
            ctypes.byref(v) if v is not None else None, ctypes.byref(host), ctypes.byref(plan),
            ctypes.byref(uses)))
        return self._adopt(plan, uses.value)

    def _host_metadata(self, dispatch: int):
        """The host arrays as psi_hip_gqa_layer_prepare takes them (`psi_hip_gqa_host_metadata`); waits until the last
        upload has left the staging block."""
        self._staging_free()
        if dispatch in (L.DISPATCH_ROW_GROUPS, L.DISPATCH_AUTO) and self._row_groups_words() == 0:
            self._alloc_row_groups((self._max_kv_splits + self._max_workers) * 32)
        if self._host_struct is None or self._host_struct.row_groups_capacity != self._row_groups_words():
            def addr(a):
                return ctypes.c_void_p(a.ctypes.data) if a is not None else None

            self._host_struct = L.HostMetadataStruct(
                self._max_tokens, self._max_kv_splits + self._max_workers, self._max_workers, self._row_groups_words(),
                addr(self.h_req_slots), addr(self.h_flat_token_indices), addr(self.h_q_token_tiles),
                addr(self._h_kv_splits_all), addr(self.h_cu_kv_splits), addr(self._h_row_index_all),
                addr(self._h_worker_cu_all), addr(self._h_row_groups_all))
        return self._host_struct

    def _adopt(self, plan, uses: int) -> GQAReplayShape:
        """Takes over what a preparation wrote into the host arrays (`plan`: the psi_hip_gqa_batch_metadata it
        filled, `uses`: which dispatch tables are in use) and uploads it."""
        sh = plan.shape
        self._shape = GQAReplayShape(sh.num_tokens, sh.num_total_tokens, sh.num_q_token_tiles, sh.num_total_q_token_tiles,
                                     sh.num_kv_splits, sh.num_total_kv_splits, bool(sh.reduce_sdpa_partial_outputs))
        self._variant = GQASplitKVVariant.from_struct(plan.variant)
        self.h_kv_splits = self._h_kv_splits_all
        use_index, use_workers, use_groups = bool(uses & 1), bool(uses & 2), bool(uses & 4)
        self.h_partial_row_index = self._h_row_index_all if use_index else None
        self.d_partial_row_index = self._d_row_index_all if use_index else None
        self.num_workers = plan.num_workers
        self.h_worker_cu = self._h_worker_cu_all[:plan.num_workers + 1] if use_workers else None
        self.d_worker_cu = self._d_worker_cu_all if use_workers else None
        self.group_tiles, self.num_row_groups = plan.group_tiles, plan.num_row_groups
        self.h_row_groups = (self._h_row_groups_all[:max(plan.group_tiles * plan.num_row_groups, 1)]
                             if use_groups else None)
        self.d_row_groups = self._d_row_groups_all if use_groups else None
        self.max_active_q_tile_tokens = plan.max_active_q_tile_tokens
        if self.device is not None:
            if use_groups:
                import torch

                used = plan.group_tiles * plan.num_row_groups
                with torch.cuda.stream(self.device.stream):
                    self._d_row_groups_all[:used].copy_(self._h_row_groups_t[:used], non_blocking=True)
            self.upload()
        return self._shape

    def advance_decode(self) -> bool:
        """The next decode step of the batch `prepare` planned last (same requests, one more token each) without
        planning again (psi_hip_gqa_layer_advance_decode): True if the arrays were advanced in place and uploaded,
        False if a sequence starts a new 16-token tile or the plan is of another kind: prepare again."""
        assert getattr(self, "_last_prepare", None) is not None, "advance_decode() continues a prepare()"
        options, plan, uses, _keep = self._last_prepare
        self._staging_free()
        advanced = ctypes.c_int()
        L.check(L.load().psi_hip_gqa_layer_advance_decode(ctypes.byref(options), ctypes.byref(self._host_struct),
                                                          ctypes.byref(plan), uses.value, ctypes.byref(advanced)))
        if advanced.value and self.device is not None:
            self.upload()
        return bool(advanced.value)

    def _row_groups_words(self) -> int:
        return 0 if self._h_row_groups_all is None else len(self._h_row_groups_all)

    def _alloc_row_groups(self, words: int):
        if self.device is not None:
            import torch

            self._h_row_groups_t = torch.zeros(words, dtype=torch.int32, pin_memory=True)
            self._d_row_groups_all = torch.zeros(words, dtype=torch.int32, device=self.device.torch_device)
            self._h_row_groups_all = self._h_row_groups_t.numpy().view(np.uint32)
        else:
            self._h_row_groups_all = np.zeros(words, np.uint32)

    def replay_shape(self) -> GQAReplayShape:
        assert self._shape is not None, "GQA batch metadata must be updated before recording"
        return self._shape

    def split_kv_variant(self) -> GQASplitKVVariant:
        assert self._variant is not None, "GQA batch metadata must be updated before recording"
        return self._variant

    def struct(self, shape: Optional[GQAReplayShape] = None, counts_uploaded: bool = False):
        """The batch as the layer entry points take it (psi_hip_gqa_batch_metadata): device addresses of the
        arrays, the shape (`shape` overrides the capacities, e.g. a replay bucket) and the launch plans.
        `counts_uploaded`: name the count words that `upload()` brought along, so that a replay cache launches its
        program without a launch of its own ahead of it (the layer is then the input's, not a parameter)."""
        assert self.device is not None and self._shape is not None
        s = shape or self._shape
        return L.BatchMetadataStruct(
            L.ReplayShapeStruct(s.num_tokens, s.num_total_tokens, s.num_q_token_tiles, s.num_total_q_token_tiles,
                                s.num_sdpa_map_task_templates, s.num_total_sdpa_map_task_templates,
                                int(s.reduce_sdpa_partial_outputs)),
            self._variant.struct(), _ptr(self.d_req_slots), _ptr(self.d_flat_token_indices),
            _ptr(self.d_q_token_tiles), _ptr(self.d_kv_splits), _ptr(self.d_cu_kv_splits),
            _ptr(self.d_partial_row_index), _ptr(self.d_worker_cu), self.num_workers, _ptr(self.d_row_groups),
            self.group_tiles, self.num_row_groups, self.max_active_q_tile_tokens,
            _ptr(self.d_replay_counts) if counts_uploaded else None)


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


# ------------------------------------------------------------------ the attention layer


@dataclass(frozen=True)
class GQACore:
    """`GQACore` (crates/inference-executor-core/src/attn/gqa/core.rs:3-91)."""
    model_layer_index: int
    hidden_dim: int
    head_dim: int
    num_q_heads: int
    num_kv_heads: int
    scale: float

    def validate(self):
        assert self.hidden_dim > 0 and self.head_dim > 0 and self.num_q_heads > 0 and self.num_kv_heads > 0
        assert self.num_q_heads % self.num_kv_heads == 0 and self.scale > 0.0

    def q_dim(self) -> int:
        return self.num_q_heads * self.head_dim

    def k_dim(self) -> int:
        return self.num_kv_heads * self.head_dim

    def qgkv_dim(self) -> int:
        return 2 * self.q_dim() + 2 * self.k_dim()

    def qkv_dim(self) -> int:
        return self.q_dim() + 2 * self.k_dim()


@dataclass(frozen=True)
class GQAMetalConfig:
    """`GQAMetalConfig` (attn/gqa/backend.rs:114-146) without the matmul quantisation fields; the name is the
    reference's, the device is not."""
    page_bytes: int
    rope_dim: int
    norm_eps: float
    rope_theta: float
    rope_scaling: RopeScaling = RopeScaling()
    io_dtype: Dtype = Dtype.Bfloat16


class GQAReplayMode(IntEnum):
    Exact = L.REPLAY_EXACT
    Bucketed = L.REPLAY_BUCKETED


@dataclass
class GQAKVCacheBindings:
    kv_pages: object
    page_ids: object


@dataclass
class GQAWeights:
    """The norm weights of `GQAWeights` (backend.rs:156-166); the projection weights stay with the caller."""
    q_norm_weight: object
    k_norm_weight: object


class GQAScratch:
    """`GQAScratch` (attn/gqa/scratch.rs:17-92) as far as this path uses it: the projection output, the
    normalised queries, the partial states (one buffer, sized by the library) and the layer's output."""

    def __init__(self, device: Device, gqa: "GQA", max_tokens: int, max_kv_splits: Optional[int] = None):
        import torch

        core, dt = gqa.core, gqa.config.io_dtype.torch()
        dev = device.torch_device
        self.max_tokens = max_tokens
        self.max_kv_splits = max_kv_splits if max_kv_splits is not None else max_tokens
        width = core.qgkv_dim() if gqa.gated else core.qkv_dim()
        self.qgkv = torch.zeros(max_tokens * width, dtype=dt, device=dev)
        self.q_norm_rope = torch.zeros(max_tokens * core.q_dim(), dtype=dt, device=dev)
        # the wider of the two variants' layouts for the split capacity
        nbytes = 0
        for variant in (GQASplitKVVariant.SingleQ(256, 256, 1), GQASplitKVVariant.TiledQ(8, 16, 1)):
            nbytes = max(nbytes, gqa.scratch_bytes(variant, self.max_kv_splits))
        self.sdpa_partial = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        self.attention_output = torch.zeros(max_tokens * core.q_dim(), dtype=dt, device=dev)


@dataclass
class GQAInput:
    """`GQAInput` (backend.rs:169-182).  `qgkv`: the projection output (defaults to `scratch.qgkv`); or pass
    rows already split, normalised and rotated as `q`, `k`, `v` (and optionally gates `g`).  `output`: defaults
    to `scratch.attention_output`."""
    page_table_layout: GQAPageTableLayout
    gqa_layer_index: int
    batch_metadata: GQAMetadataBuffers
    kv_cache: GQAKVCacheBindings
    scratch: GQAScratch
    weights: Optional[GQAWeights] = None
    replay_mode: GQAReplayMode = GQAReplayMode.Bucketed
    qgkv: object = None
    q: object = None
    k: object = None
    v: object = None
    g: object = None
    output: object = None
    shape: Optional[GQAReplayShape] = None  # overrides batch_metadata.replay_shape() (e.g. wider capacities)
    counts_uploaded: bool = False  # a replay cache reads the count words the metadata upload brought along


@dataclass
class GQAMixedPlan:
    """What `GQA.prepare_mixed` planned: the batch's first `num_chunk_reqs` requests (`num_chunk_tokens` tokens) are
    prefill chunks, the others decode requests; each part's arrays live in its own `GQAMetadataBuffers`."""
    num_chunk_reqs: int
    num_chunk_tokens: int
    chunk_metadata: GQAMetadataBuffers
    decode_metadata: GQAMetadataBuffers
    has_chunk: bool
    has_decode: bool

    def struct(self):
        empty = L.BatchMetadataStruct()
        return L.MixedPlanStruct(self.num_chunk_reqs, self.num_chunk_tokens, 0, 0,
                                 self.chunk_metadata.struct() if self.has_chunk else empty,
                                 self.decode_metadata.struct() if self.has_decode else empty)


class GQA:
    """`GQA` / `UngatedGQA` (attn/gqa/backend.rs:214-392, ungated_backend.rs:104-180): the attention part of a
    layer behind `record`.  `gated`: projection rows [q_0|g_0|...|k|v] and a sigmoid gate on the output."""

    def __init__(self, device: Device, core: GQACore, config: GQAMetalConfig, gated: bool = True):
        core.validate()
        self.device, self.core, self.config, self.gated = device, core, config, gated
        self.split_kv = GQASplitKV.new(GQASplitKVConfig(config.io_dtype, config.page_bytes, core.num_q_heads,
                                                        core.num_kv_heads, core.head_dim))

    @staticmethod
    def new(device, core, config, gated=True):
        return GQA(device, core, config, gated)

    def struct(self):
        c, k = self.core, self.config
        return L.LayerConfigStruct(_cfg_struct(c.num_q_heads, c.num_kv_heads, c.head_dim, c.scale, k.page_bytes,
                                               k.io_dtype),
                                   int(self.gated), k.rope_dim, k.norm_eps, k.rope_theta, k.rope_scaling.struct())

    def num_tokens_per_page(self) -> int:
        return self.split_kv.config.num_tokens_per_page()

    def scratch_bytes(self, variant: GQASplitKVVariant, num_total_kv_splits: int) -> int:
        out, cfg, v = ctypes.c_uint64(), self.struct(), variant.struct()
        L.check(L.load().psi_hip_gqa_layer_scratch_bytes(ctypes.byref(cfg), ctypes.byref(v), num_total_kv_splits,
                                                         ctypes.byref(out)))
        return out.value

    def new_scratch(self, max_tokens: int, max_kv_splits: Optional[int] = None) -> GQAScratch:
        return GQAScratch(self.device, self, max_tokens, max_kv_splits)

    def select_variant(self, batch_metadata, token_indices, cu_tokens, policy=None) -> GQASplitKVVariant:
        return select_split_kv_variant(self.split_kv, batch_metadata.max_tokens(), policy, token_indices, cu_tokens)

    def prepare(self, batch_metadata: GQAMetadataBuffers, req_slots, token_indices, cu_tokens) -> GQAReplayShape:
        """`GQA::prepare` (backend.rs:289-304): variant selection and metadata update, one host call."""
        return batch_metadata.prepare(self.struct(), req_slots, token_indices, cu_tokens)

    def prepare_bucketed(self, batch_metadata, req_slots, token_indices, cu_tokens,
                         policy: GQAReplayBucketPolicy) -> GQAReplayShape:
        """`GQA::prepare_bucketed` (backend.rs:306-323)."""
        assert policy.max_tokens() == batch_metadata.max_tokens(), \
            "GQA replay bucket policy must match metadata token capacity"
        return batch_metadata.prepare(self.struct(), req_slots, token_indices, cu_tokens,
                                      capacity_mode=L.CAPACITY_BUCKETED, policy=policy)

    def prepare_fixed_partition(self, batch_metadata, req_slots, token_indices, cu_tokens, partition_tokens: int,
                                balanced: bool = True, grouped: bool = False,
                                variant: Optional[GQASplitKVVariant] = None, num_workers: int = 0,
                                bucket_capacities: bool = False,
                                policy: Optional[GQAReplayBucketPolicy] = None, auto: bool = False) -> GQAReplayShape:
        """Not in the reference: partitions of fixed length instead of the greedy budget, then (by default) the
        balanced worker plan that gives every compute unit an equal share of the batch's tiles; `grouped`
        selects the row-group plan of the prefill-chunk map instead (`partition_tokens` 0: the planner's), and `auto`
        lets the library pick between the two per batch (PSI_HIP_DISPATCH_AUTO: row groups over the planner's
        partition when a request brings more than one Q-token tile or a tile more than 48 query columns).  One host
        call and one upload.  `bucket_capacities`: the recorded capacities (the re-cut row count included) are rounded
        up to `ReplayBucketPolicy` buckets, so that a `GQAReplayCache` keeps one program per bucket."""
        dispatch = (L.DISPATCH_AUTO if auto else L.DISPATCH_ROW_GROUPS if grouped else
                    L.DISPATCH_BALANCED if balanced else L.DISPATCH_PLAN_ORDER)
        return batch_metadata.prepare(self.struct(), req_slots, token_indices, cu_tokens,
                                      capacity_mode=L.CAPACITY_FIXED_PARTITION, partition_tokens=partition_tokens,
                                      dispatch=dispatch, num_workers=num_workers, variant=variant,
                                      bucket_capacities=bucket_capacities, policy=policy)

    def prepare_mixed(self, chunk_metadata: GQAMetadataBuffers, decode_metadata: GQAMetadataBuffers, req_slots,
                      token_indices, cu_tokens, chunk_min_tokens: int = 8, chunk_partition: int = 4096,
                      decode_partition: int = 512, num_workers: int = 0) -> "GQAMixedPlan":
        """The host side of a step whose batch holds prefill chunks (more than `chunk_min_tokens` new tokens; they must
        come first) and decode requests: one call (psi_hip_gqa_layer_prepare_mixed) plans the chunk part for the
        row-group map and the decode part for the balanced decode map, each with fixed partitions, and uploads
        both.  The reference plans such a batch for one variant (backend.rs:289-364)."""
        rs = np.ascontiguousarray(req_slots, dtype=np.uint32)
        ti = np.ascontiguousarray(token_indices, dtype=np.uint32)
        cu = np.ascontiguousarray(cu_tokens, dtype=np.uint32)
        assert len(rs) == len(ti) and len(cu) == len(rs) + 1
        chunk_options = L.PlanOptionsStruct(L.CAPACITY_FIXED_PARTITION, chunk_partition, 0, L.DISPATCH_ROW_GROUPS, 0, 0,
                                            None, 0, 0)
        decode_options = L.PlanOptionsStruct(L.CAPACITY_FIXED_PARTITION, decode_partition, 0, L.DISPATCH_BALANCED,
                                             num_workers, 0, None, 0, 0)
        plan = L.MixedPlanStruct()
        cfg = self.struct()
        L.check(L.load().psi_hip_gqa_layer_prepare_mixed(
            ctypes.byref(cfg), ctypes.byref(chunk_options), ctypes.byref(decode_options), chunk_min_tokens,
            rs.ctypes.data, ti.ctypes.data, cu.ctypes.data, len(rs),
            ctypes.byref(chunk_metadata._host_metadata(L.DISPATCH_ROW_GROUPS)),
            ctypes.byref(decode_metadata._host_metadata(L.DISPATCH_BALANCED)), ctypes.byref(plan)))
        if plan.chunk.shape.num_tokens:
            chunk_metadata._adopt(plan.chunk, plan.chunk_uses)
        if plan.decode.shape.num_tokens:
            decode_metadata._adopt(plan.decode, plan.decode_uses)
            decode_metadata._last_prepare = (decode_options, plan.decode, ctypes.c_uint32(plan.decode_uses), plan)
        return GQAMixedPlan(plan.num_chunk_reqs, plan.num_chunk_tokens, chunk_metadata, decode_metadata,
                            bool(plan.chunk.shape.num_tokens), bool(plan.decode.shape.num_tokens))

    def mixed_scratch_bytes(self, plan: "GQAMixedPlan") -> int:
        cfg, n = self.struct(), ctypes.c_uint64()
        s = plan.struct()
        L.check(L.load().psi_hip_gqa_layer_mixed_scratch_bytes(ctypes.byref(cfg), ctypes.byref(s), ctypes.byref(n)))
        return n.value

    def record_mixed(self, inp: GQAInput, plan: "GQAMixedPlan"):
        """`GQA::record` for a mixed batch (psi_hip_gqa_layer_record_mixed): `inp` names the whole batch's rows and a
        scratch of `mixed_scratch_bytes(plan)`; its `batch_metadata` is not used."""
        cfg = self.struct()
        inp.batch_metadata = plan.chunk_metadata if plan.has_chunk else plan.decode_metadata  # any prepared one
        s, keep = self.input_struct(inp)
        p = plan.struct()
        L.check(self.device.lib.psi_hip_gqa_layer_record_mixed(self.device.ctx, ctypes.byref(cfg), ctypes.byref(s),
                                                               ctypes.byref(p)))
        return keep[1]

    def input_struct(self, inp: GQAInput):
        """(psi_hip_gqa_layer_input, keep-alive objects) for an input."""
        md = inp.batch_metadata.struct(inp.shape, counts_uploaded=inp.counts_uploaded)
        sc = inp.scratch
        qgkv = inp.qgkv if (inp.qgkv is not None or inp.q is not None) else sc.qgkv
        out = inp.output if inp.output is not None else sc.attention_output
        w = inp.weights
        s = L.LayerInputStruct(
            inp.page_table_layout.struct(), inp.gqa_layer_index, int(inp.replay_mode), ctypes.pointer(md),
            _ptr(qgkv if inp.q is None else None), _ptr(inp.q), _ptr(inp.k), _ptr(inp.v), _ptr(inp.g),
            _ptr(inp.kv_cache.kv_pages), _nbytes(inp.kv_cache.kv_pages), _ptr(inp.kv_cache.page_ids),
            _ptr(w.q_norm_weight if w else None), _ptr(w.k_norm_weight if w else None), _ptr(sc.q_norm_rope),
            _ptr(sc.sdpa_partial), _nbytes(sc.sdpa_partial), _ptr(out))
        return s, (md, out)

    def record(self, inp: GQAInput):
        """`GQA::record` (backend.rs:394-658): issues the layer's launches on the device's stream and returns
        the output buffer (the reference returns the caller-owned buffer it was given, too)."""
        cfg = self.struct()
        s, keep = self.input_struct(inp)
        L.check(self.device.lib.psi_hip_gqa_layer_record(self.device.ctx, ctypes.byref(cfg), ctypes.byref(s)))
        return keep[1]


def _record_static_scratch(self, inp: GQAInput):
    """`record` with the partial states in the library's built-in buffer (psi_hip_gqa_layer_record_static_scratch):
    for callers that cannot allocate.  `inp.scratch.sdpa_partial` is not used; batches whose partial states exceed
    `STATIC_SCRATCH_BYTES` are rejected."""
    cfg = self.struct()
    s, keep = self.input_struct(inp)
    s.partial_scratch, s.partial_scratch_bytes = None, 0
    L.check(self.device.lib.psi_hip_gqa_layer_record_static_scratch(self.device.ctx, ctypes.byref(cfg), ctypes.byref(s)))
    return keep[1]


GQA.record_static_scratch = _record_static_scratch
STATIC_SCRATCH_BYTES = L.STATIC_SCRATCH_BYTES


class GQAReplayCache:
    """One recorded program (HIP graph) per capacity bucket of a layer: the reference's replay-program store keyed
    by `(variant, total tokens, total Q-token tiles, total KV splits)` with the active counts bound at submission
    (crates/inference-executor-core/src/replay.rs:4-87, backend.rs:55-57).  The device must launch on a created
    stream (not the null stream)."""

    def __init__(self, device: Device, gqa: GQA, max_programs: int = 32):
        import torch

        self.device, self.gqa = device, gqa
        self.counts = torch.zeros(4, dtype=torch.int32, device=device.torch_device)
        handle, cfg = ctypes.c_void_p(), gqa.struct()
        L.check(device.lib.psi_hip_gqa_replay_cache_create(device.ctx, ctypes.byref(cfg), _ptr(self.counts),
                                                           max_programs, ctypes.byref(handle)))
        self.handle = handle

    def submit(self, inp: GQAInput, gqa_layer_parameter: int = 0) -> bool:
        """Replays the program of the input's bucket (recording it first when there is none); True if this call
        recorded.  `gqa_layer_parameter` n > 0 binds page-table layer n - 1 at submission."""
        s, _keep = self.gqa.input_struct(inp)
        recorded = ctypes.c_int()
        L.check(self.device.lib.psi_hip_gqa_replay_cache_submit(self.handle, ctypes.byref(s), gqa_layer_parameter,
                                                                ctypes.byref(recorded)))
        return bool(recorded.value)

    def stats(self):
        """(programs held, recordings, replays)."""
        p, r, n = ctypes.c_uint32(), ctypes.c_uint64(), ctypes.c_uint64()
        L.check(self.device.lib.psi_hip_gqa_replay_cache_stats(self.handle, ctypes.byref(p), ctypes.byref(r),
                                                               ctypes.byref(n)))
        return p.value, r.value, n.value

    def close(self):
        if self.handle:
            self.device.sync()
            self.device.lib.psi_hip_gqa_replay_cache_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
