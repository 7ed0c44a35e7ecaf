"""ctypes binding of libpsi_hip.so (the C ABI declared in include/psi_hip.h).

The library is loaded from psi-dec_amd/lib/; there is no CPU fallback: if the shared object is
missing, `load()` raises with the build command.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_size_t, c_uint32, c_uint64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpsi_hip.so")

OK = 0
ERR_INVALID_ARGUMENT = -1
ERR_RESOURCE_EXHAUSTED = -2
ERR_RUNTIME = -3
ERR_UNSUPPORTED = -4

F32, BF16, F16 = 0, 1, 2
SENTINEL = 0xFFFFFFFF
VARIANT_SINGLE_Q, VARIANT_TILED_Q = 0, 1
CAPACITY_EXACT, CAPACITY_BUCKETED, CAPACITY_CALLER_TOKENS, CAPACITY_FIXED_PARTITION = 0, 1, 2, 3
FLAG_FORCE_GENERIC = 1
FLAG_F32_OUTPUT = 2
FLAG_MUTE_LOADERS = 3
DEVICE_ERR_WAIT_GAVE_UP = 1
DEVICE_ERR_V_RANGE = 2
REPLAY_EXACT, REPLAY_BUCKETED = 0, 1
DISPATCH_PLAN_ORDER, DISPATCH_LONGEST_FIRST, DISPATCH_BALANCED, DISPATCH_ROW_GROUPS, DISPATCH_AUTO = 0, 1, 2, 3, 4
STATIC_SCRATCH_BYTES = 16 << 20


class PsiHipError(RuntimeError):
    """A non-zero status from the C ABI; `.code` is the status, the text is psi_hip_last_error()."""

    def __init__(self, code, message):
        super().__init__(f"psi_hip error {code}: {message}")
        self.code = code
        self.message = message


class GQAConfigStruct(ctypes.Structure):
    _fields_ = [
        ("num_q_heads", c_uint32),
        ("num_kv_heads", c_uint32),
        ("head_dim", c_uint32),
        ("scale", c_float),
        ("page_bytes", c_uint32),
        ("dtype", c_uint32),
    ]


class PageTableLayoutStruct(ctypes.Structure):
    _fields_ = [
        ("num_req_slots", c_uint32),
        ("num_gqa_layers", c_uint32),
        ("num_blocks", c_uint32),
        ("num_page_ids_per_block", c_uint32),
    ]


class VariantStruct(ctypes.Structure):
    _fields_ = [
        ("kind", c_uint32),
        ("q_token_tile_size", c_uint32),
        ("kv_token_tile_size", c_uint32),
        ("num_threads_per_threadblock", c_uint32),
        ("q_head_tile_size", c_uint32),
    ]


class RopeScalingStruct(ctypes.Structure):
    _fields_ = [
        ("kind", c_uint32),
        ("factor", c_float),
        ("attention_factor", c_float),
        ("beta_fast", c_float),
        ("beta_slow", c_float),
        ("original_max_position_embeddings", c_uint32),
        ("truncate", c_uint32),
    ]


class RMSNormRopeConfigStruct(ctypes.Structure):
    _fields_ = [
        ("num_heads", c_uint32),
        ("head_dim", c_uint32),
        ("rope_dim", c_uint32),
        ("eps", c_float),
        ("rope_theta", c_float),
        ("scaling", RopeScalingStruct),
        ("dtype", c_uint32),
    ]


class OutputGateStruct(ctypes.Structure):
    _fields_ = [("gates", c_void_p), ("token_stride", c_uint64), ("head_stride", c_uint64)]


class ReplayShapeStruct(ctypes.Structure):
    _fields_ = [
        ("num_tokens", c_uint32),
        ("num_total_tokens", c_uint32),
        ("num_q_token_tiles", c_uint32),
        ("num_total_q_token_tiles", c_uint32),
        ("num_kv_splits", c_uint32),
        ("num_total_kv_splits", c_uint32),
        ("reduce_sdpa_partial_outputs", c_uint32),
    ]


class BatchMetadataStruct(ctypes.Structure):
    _fields_ = [
        ("shape", ReplayShapeStruct),
        ("variant", VariantStruct),
        ("req_slots", c_void_p),
        ("flat_token_indices", c_void_p),
        ("q_token_tiles", c_void_p),
        ("kv_splits", c_void_p),
        ("cu_kv_splits", c_void_p),
        ("partial_row_index", c_void_p),
        ("worker_cu", c_void_p),
        ("num_workers", c_uint32),
        ("row_groups", c_void_p),
        ("group_tiles", c_uint32),
        ("num_row_groups", c_uint32),
        ("max_active_q_tile_tokens", c_uint32),
        ("replay_counts", c_void_p),
    ]


class MixedPlanStruct(ctypes.Structure):
    _fields_ = [
        ("num_chunk_reqs", c_uint32),
        ("num_chunk_tokens", c_uint32),
        ("chunk_uses", c_uint32),
        ("decode_uses", c_uint32),
        ("chunk", BatchMetadataStruct),
        ("decode", BatchMetadataStruct),
    ]


class LayerConfigStruct(ctypes.Structure):
    _fields_ = [
        ("attention", GQAConfigStruct),
        ("gated", c_uint32),
        ("rope_dim", c_uint32),
        ("norm_eps", c_float),
        ("rope_theta", c_float),
        ("rope_scaling", RopeScalingStruct),
    ]


class PlanOptionsStruct(ctypes.Structure):
    _fields_ = [
        ("capacity_mode", c_uint32),
        ("partition_tokens", c_uint32),
        ("caller_num_total_tokens", c_uint32),
        ("dispatch", c_uint32),
        ("num_workers", c_uint32),
        ("bucket_max_tokens", c_uint32),
        ("topology_boundaries", POINTER(c_uint32)),
        ("num_boundaries", c_uint32),
        ("bucket_capacities", c_uint32),
    ]


class HostMetadataStruct(ctypes.Structure):
    _fields_ = [
        ("max_tokens", c_uint32),
        ("kv_splits_capacity", c_uint32),
        ("max_workers", c_uint32),
        ("row_groups_capacity", c_uint64),
        ("req_slots_by_token", c_void_p),
        ("flat_token_indices", c_void_p),
        ("q_token_tiles", c_void_p),
        ("kv_splits", c_void_p),
        ("cu_kv_splits", c_void_p),
        ("partial_row_index", c_void_p),
        ("worker_cu", c_void_p),
        ("row_groups", c_void_p),
    ]


class LayerInputStruct(ctypes.Structure):
    _fields_ = [
        ("page_table_layout", PageTableLayoutStruct),
        ("gqa_layer_index", c_uint32),
        ("replay_mode", c_uint32),
        ("batch_metadata", POINTER(BatchMetadataStruct)),
        ("qgkv", c_void_p),
        ("q", c_void_p),
        ("k", c_void_p),
        ("v", c_void_p),
        ("g", c_void_p),
        ("kv_pages", c_void_p),
        ("kv_pages_bytes", c_uint64),
        ("page_ids", c_void_p),
        ("q_norm_weight", c_void_p),
        ("k_norm_weight", c_void_p),
        ("q_norm_rope", c_void_p),
        ("partial_scratch", c_void_p),
        ("partial_scratch_bytes", c_uint64),
        ("output", c_void_p),
    ]


class DecoderBlocksConfigStruct(ctypes.Structure):
    _fields_ = [("tokens_per_block", c_uint32), ("num_cache_lanes", c_uint32), ("pages_per_kv_block", c_uint32)]


class QueryTokensStruct(ctypes.Structure):
    _fields_ = [
        ("kind", c_uint32),
        ("window", c_uint32),
        ("epoch", c_uint64),
        ("token_index", c_uint64),
        ("tokens", POINTER(c_uint32)),
        ("num_tokens", c_size_t),
        ("tokens_capacity", c_size_t),
        ("spec_tokens", POINTER(c_uint32)),
        ("num_spec_tokens", c_size_t),
        ("spec_tokens_capacity", c_size_t),
    ]


class SampledTokensStruct(ctypes.Structure):
    _fields_ = [
        ("kind", c_uint32),
        ("sampled_token", c_uint32),
        ("epoch", c_uint64),
        ("validated_tokens", POINTER(c_uint32)),
        ("num_validated_tokens", c_size_t),
        ("spec_tokens", POINTER(c_uint32)),
        ("num_spec_tokens", c_size_t),
    ]


_U32P = POINTER(c_uint32)
_U64P = POINTER(c_uint64)
_SZP = POINTER(c_size_t)
_CFG = POINTER(GQAConfigStruct)
_LAYOUT = POINTER(PageTableLayoutStruct)
_VARIANT = POINTER(VariantStruct)

# name -> (restype, argtypes); every symbol include/psi_hip.h declares.
PROTOTYPES = {
    "psi_hip_last_error": (c_char_p, []),
    "psi_hip_version": (c_char_p, []),
    "psi_hip_ctx_create": (c_int, [c_int, c_void_p, POINTER(c_void_p)]),
    "psi_hip_ctx_destroy": (c_int, [c_void_p]),
    "psi_hip_ctx_set_stream": (c_int, [c_void_p, c_void_p]),
    "psi_hip_sync": (c_int, [c_void_p]),
    "psi_hip_ctx_set_timing": (c_int, [c_void_p, c_int]),
    "psi_hip_ctx_kernel_time_ms": (c_int, [c_void_p, c_char_p, POINTER(c_double), POINTER(c_uint64)]),
    "psi_hip_ctx_reset_timing": (c_int, [c_void_p]),
    "psi_hip_ctx_bind_replay_counts": (c_int, [c_void_p, c_void_p]),
    "psi_hip_ctx_set_flag": (c_int, [c_void_p, c_uint32, c_uint32]),
    "psi_hip_ctx_take_device_error": (c_int, [c_void_p, POINTER(c_uint32)]),
    "psi_hip_gqa_tokens_per_page": (c_int, [_CFG, _U32P]),
    "psi_hip_split_kv_select": (c_int, [_CFG, c_int, c_uint32, c_uint32, _VARIANT]),
    "psi_hip_split_kv_max_q_tokens_per_partial_output": (c_int, [_CFG, c_int, _U32P]),
    "psi_hip_split_kv_select_batch": (c_int, [_CFG, c_uint32, c_uint32, _U32P, _U32P, c_uint32, _VARIANT]),
    "psi_hip_replay_buckets": (c_int, [c_uint32, _U32P, c_uint32, _U32P, c_uint32, _U32P]),
    "psi_hip_replay_bucket_capacity": (c_int, [c_uint32, _U32P, c_uint32, c_uint32, _U32P]),
    "psi_hip_gqa_metadata_update": (
        c_int,
        [c_uint32, _U32P, _U32P, _U32P, c_uint32, _VARIANT, c_uint32, c_uint32, _U32P, c_uint32, c_uint32, c_uint32,
         _U32P, _U32P, _U32P, _U32P, _U32P, POINTER(ReplayShapeStruct)],
    ),
    "psi_hip_split_kv_balance_plan": (
        c_int, [_U32P, c_uint32, _U32P, c_uint32, c_uint32, _U32P, c_uint32, _U32P, _U32P, _U32P]),
    "psi_hip_split_kv_balanced_workers": (c_int, [_CFG, _U32P]),
    "psi_hip_split_kv_single_q_map_balanced": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, c_void_p, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32,
         c_void_p, c_uint64, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32],
    ),
    "psi_hip_kv_page_write": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32,
         c_uint32, c_uint32],
    ),
    "psi_hip_split_kv_single_q_scratch_bytes": (c_int, [_CFG, c_uint32, POINTER(c_uint64)]),
    "psi_hip_split_kv_single_q_map": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, c_void_p, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_uint64,
         c_uint32, c_uint32, c_uint32, c_uint32, c_uint32],
    ),
    "psi_hip_split_kv_single_q_reduce": (
        c_int, [c_void_p, _CFG, c_void_p, c_uint64, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32, c_void_p,
                POINTER(OutputGateStruct)]),
    "psi_hip_kv_page_write_split_kv_single_q_map": (
        c_int, [c_void_p, _CFG, _LAYOUT, c_void_p, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                c_void_p, c_void_p, c_uint32, c_void_p, c_uint64, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32]),
    "psi_hip_split_kv_single_q_store_partials": (
        c_int, [c_void_p, _CFG, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32,
                c_uint32, c_void_p]),
    "psi_hip_selected_ranges_payload_bytes": (c_int, [POINTER(c_uint32), c_uint32, c_uint64, c_uint64,
                                                      POINTER(c_uint64)]),
    "psi_hip_buffer_pack_selected": (c_int, [c_void_p, c_void_p, c_uint64, POINTER(c_uint32), c_uint32, c_uint64,
                                             c_void_p, c_uint64]),
    "psi_hip_buffer_unpack_selected": (c_int, [c_void_p, c_void_p, c_uint64, POINTER(c_uint32), c_uint32, c_uint64,
                                               c_void_p, c_uint64]),
    "psi_hip_rope_parameters": (c_int, [POINTER(RMSNormRopeConfigStruct), POINTER(c_float), POINTER(c_float),
                                        POINTER(c_float)]),
    "psi_hip_rms_norm_rope": (
        c_int, [c_void_p, POINTER(RMSNormRopeConfigStruct), c_void_p, c_uint64, c_uint64, c_void_p, c_void_p, c_void_p,
                c_uint32, c_uint32]),
    "psi_hip_qgkv_split": (
        c_int, [c_void_p, c_uint32, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                c_uint32, c_uint32]),
    "psi_hip_activation_gate": (
        c_int, [c_void_p, c_uint32, c_uint32, c_uint32, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32]),
    "psi_hip_qk_norm_rope_kv_page_write": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, POINTER(RMSNormRopeConfigStruct), POINTER(RMSNormRopeConfigStruct), c_void_p,
         c_uint64, c_uint64, c_void_p, c_void_p, c_void_p, c_uint64, c_void_p, c_uint64, c_void_p, c_uint64, c_void_p,
         c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32],
    ),
    "psi_hip_kv_page_write_norm_rope": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, POINTER(RMSNormRopeConfigStruct), c_void_p, c_uint64, c_void_p, c_uint64, c_void_p,
         c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32],
    ),
    "psi_hip_split_kv_order_longest_first": (c_int, [_U32P, c_uint32, _U32P]),
    "psi_hip_split_kv_tiled_q_scratch_bytes": (c_int, [_CFG, c_uint32, c_uint32, POINTER(c_uint64)]),
    "psi_hip_split_kv_tiled_q_map": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, c_uint32, c_void_p, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p, c_uint64, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
         c_uint32],
    ),
    "psi_hip_split_kv_tiled_q_map_balanced": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, c_uint32, c_void_p, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p, c_uint32, c_void_p, c_uint64, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
         c_uint32, c_uint32],
    ),
    "psi_hip_split_kv_tiled_q_map_grouped": (
        c_int,
        [c_void_p, _CFG, _LAYOUT, c_uint32, c_void_p, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p, c_uint64, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32, c_uint32,
         c_uint32, c_void_p, c_uint32, c_uint32],
    ),
    "psi_hip_split_kv_tiled_q_group_rows": (
        c_int, [_CFG, c_uint32, _U32P, c_uint32, _U32P, c_uint32, _U32P, _U32P, c_uint64, _U32P, _U32P]),
    "psi_hip_split_kv_chunk_partition_tokens": (
        c_int, [_CFG, c_uint32, _U32P, _U32P, c_uint32, c_uint32, _U32P]),
    "psi_hip_split_kv_tiled_q_reduce": (
        c_int,
        [c_void_p, _CFG, c_uint32, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_uint32, c_uint32, c_uint32,
         c_uint32, c_void_p, POINTER(OutputGateStruct)],
    ),
    "psi_hip_gqa_layer_scratch_bytes": (c_int, [POINTER(LayerConfigStruct), _VARIANT, c_uint32, POINTER(c_uint64)]),
    "psi_hip_gqa_layer_prepare": (
        c_int, [POINTER(LayerConfigStruct), POINTER(PlanOptionsStruct), c_void_p, c_void_p, c_void_p, c_uint32,
                _VARIANT, POINTER(HostMetadataStruct), POINTER(BatchMetadataStruct), _U32P]),
    "psi_hip_gqa_layer_advance_decode": (
        c_int, [POINTER(PlanOptionsStruct), POINTER(HostMetadataStruct), POINTER(BatchMetadataStruct), c_uint32,
                POINTER(ctypes.c_int)]),
    "psi_hip_gqa_layer_record": (c_int, [c_void_p, POINTER(LayerConfigStruct), POINTER(LayerInputStruct)]),
    "psi_hip_gqa_layer_prepare_mixed": (
        c_int, [POINTER(LayerConfigStruct), POINTER(PlanOptionsStruct), POINTER(PlanOptionsStruct), c_uint32, c_void_p,
                c_void_p, c_void_p, c_uint32, POINTER(HostMetadataStruct), POINTER(HostMetadataStruct),
                POINTER(MixedPlanStruct)]),
    "psi_hip_gqa_layer_mixed_scratch_bytes": (
        c_int, [POINTER(LayerConfigStruct), POINTER(MixedPlanStruct), POINTER(c_uint64)]),
    "psi_hip_gqa_layer_record_mixed": (
        c_int, [c_void_p, POINTER(LayerConfigStruct), POINTER(LayerInputStruct), POINTER(MixedPlanStruct)]),
    "psi_hip_gqa_layer_record_static_scratch": (
        c_int, [c_void_p, POINTER(LayerConfigStruct), POINTER(LayerInputStruct)]),
    "psi_hip_gqa_replay_cache_create": (
        c_int, [c_void_p, POINTER(LayerConfigStruct), c_void_p, c_uint32, POINTER(c_void_p)]),
    "psi_hip_gqa_replay_cache_destroy": (c_int, [c_void_p]),
    "psi_hip_gqa_replay_cache_submit": (c_int, [c_void_p, POINTER(LayerInputStruct), c_uint32, POINTER(c_int)]),
    "psi_hip_gqa_replay_cache_stats": (c_int, [c_void_p, _U32P, _U64P, _U64P]),
    "psi_hip_page_table_write_page_ids": (
        c_int, [c_void_p, _LAYOUT, c_void_p, c_uint32, c_uint32, c_uint32, _U32P, c_uint32, c_uint32]),
    "psi_hip_page_table_reset_req_slot": (c_int, [c_void_p, _LAYOUT, c_void_p, c_uint32]),
    "psi_hip_page_table_start_index": (c_int, [_LAYOUT, c_uint32, c_uint32, c_uint32, POINTER(c_uint64)]),
    "psi_hip_page_ids_by_layer": (c_int, [_U32P, c_uint32, c_uint32, c_uint32, _U32P]),
    "psi_hip_id_allocator_create": (c_int, [c_uint64, POINTER(c_void_p)]),
    "psi_hip_id_allocator_destroy": (c_int, [c_void_p]),
    "psi_hip_id_allocator_alloc_one": (c_int, [c_void_p, _U32P]),
    "psi_hip_id_allocator_alloc_many": (c_int, [c_void_p, c_size_t, _U32P]),
    "psi_hip_id_allocator_free_one": (c_int, [c_void_p, c_uint32]),
    "psi_hip_id_allocator_free_many": (c_int, [c_void_p, _U32P, c_size_t]),
    "psi_hip_id_allocator_counts": (c_int, [c_void_p, _U64P, _U64P, _U64P]),
    "psi_hip_id_allocator_bitmap": (c_int, [c_void_p, _U64P, c_size_t]),
    "psi_hip_bitmap_allocated_ranges": (c_int, [_U64P, c_size_t, _U32P, c_size_t, _SZP]),
    "psi_hip_decoder_blocks_create": (
        c_int, [c_void_p, POINTER(DecoderBlocksConfigStruct), _U32P, c_size_t, POINTER(c_void_p)]),
    "psi_hip_decoder_blocks_destroy": (c_int, [c_void_p]),
    "psi_hip_decoder_blocks_ready_token_slots": (c_int, [c_void_p, _SZP]),
    "psi_hip_decoder_blocks_init_block_once": (c_int, [c_void_p, _SZP]),
    "psi_hip_decoder_blocks_uninit_block_once": (c_int, [c_void_p, _SZP]),
    "psi_hip_decoder_blocks_set_spec_tokens": (c_int, [c_void_p, _U32P, c_size_t]),
    "psi_hip_decoder_blocks_prepare": (c_int, [c_void_p, c_size_t, POINTER(QueryTokensStruct)]),
    "psi_hip_decoder_blocks_cancel": (c_int, [c_void_p, POINTER(QueryTokensStruct)]),
    "psi_hip_decoder_blocks_commit": (
        c_int, [c_void_p, POINTER(QueryTokensStruct), POINTER(SampledTokensStruct)]),
    "psi_hip_decoder_blocks_prepare_blocks": (c_int, [c_void_p, _SZP, _SZP, _U32P, c_size_t]),
    "psi_hip_decoder_blocks_cancel_blocks": (c_int, [c_void_p, c_size_t]),
    "psi_hip_decoder_blocks_counts": (c_int, [c_void_p, _SZP, _SZP, _SZP, _SZP]),
    "psi_hip_decoder_blocks_tokens": (c_int, [c_void_p, c_uint32, _U32P, c_size_t, _SZP]),
}

_lib = None


def load():
    """Loads libpsi_hip.so once and installs the prototypes.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {_HERE}` (or __graft_entry__.build()); "
            "there is no CPU fallback for the attention path"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status):
    if status != OK:
        raise PsiHipError(status, load().psi_hip_last_error().decode("utf-8", "replace"))


def u32_array(values):
    values = [int(v) for v in values]
    return (c_uint32 * max(len(values), 1))(*values)
