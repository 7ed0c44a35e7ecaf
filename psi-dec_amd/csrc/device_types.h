// Device-side element helpers: widening loads and round-to-nearest-even narrowing stores for the
// three element types of the path (f32, bf16, f16).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace psi {

struct F32Tag {
    using storage = float;
    static constexpr uint32_t id = 0;
};
struct BF16Tag {
    using storage = uint16_t;
    static constexpr uint32_t id = 1;
};
struct F16Tag {
    using storage = uint16_t;
    static constexpr uint32_t id = 2;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
    uint32_t b = __float_as_uint(v);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x0040u);
    return (uint16_t)((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float v) {
    return __builtin_bit_cast(uint16_t, (_Float16)v);  // v_cvt_f16_f32: round-to-nearest-even
}

template <typename Tag>
__device__ __forceinline__ float load_as_f32(const void* base, uint64_t index);
template <>
__device__ __forceinline__ float load_as_f32<F32Tag>(const void* base, uint64_t index) {
    return reinterpret_cast<const float*>(base)[index];
}
template <>
__device__ __forceinline__ float load_as_f32<BF16Tag>(const void* base, uint64_t index) {
    return bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(base)[index]);
}
template <>
__device__ __forceinline__ float load_as_f32<F16Tag>(const void* base, uint64_t index) {
    return f16_bits_to_f32(reinterpret_cast<const uint16_t*>(base)[index]);
}

template <typename Tag>
__device__ __forceinline__ void store_from_f32(void* base, uint64_t index, float v);
template <>
__device__ __forceinline__ void store_from_f32<F32Tag>(void* base, uint64_t index, float v) {
    reinterpret_cast<float*>(base)[index] = v;
}
template <>
__device__ __forceinline__ void store_from_f32<BF16Tag>(void* base, uint64_t index, float v) {
    reinterpret_cast<uint16_t*>(base)[index] = f32_to_bf16_bits(v);
}
template <>
__device__ __forceinline__ void store_from_f32<F16Tag>(void* base, uint64_t index, float v) {
    reinterpret_cast<uint16_t*>(base)[index] = f32_to_f16_bits(v);
}

// T(v): v rounded through the storage type.
template <typename Tag>
__device__ __forceinline__ float round_through(float v);
template <>
__device__ __forceinline__ float round_through<F32Tag>(float v) { return v; }
template <>
__device__ __forceinline__ float round_through<BF16Tag>(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
template <>
__device__ __forceinline__ float round_through<F16Tag>(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }

// 16 bytes of K or V.  Pages are read once per launch, so the load is non-temporal: the lines do not displace what
// is reused in L2 -- page IDs, Q, and above all the partial states on their way to the combine (C2's decode map runs
// 8 % faster for it and the combine 15 %).
typedef uint32_t stream_u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 stream_load_b128(const void* p) {
    const stream_u32x4 t = __builtin_nontemporal_load(static_cast<const stream_u32x4*>(p));
    return make_uint4(t.x, t.y, t.z, t.w);
}

// Element `index` of an array whose element type is only known at run time (0 f32, 1 bf16, 2 f16).
__device__ __forceinline__ float load_any_as_f32(const void* base, uint64_t index, uint32_t dtype) {
    if (dtype == F32Tag::id) return load_as_f32<F32Tag>(base, index);
    if (dtype == BF16Tag::id) return load_as_f32<BF16Tag>(base, index);
    return load_as_f32<F16Tag>(base, index);
}

// Gate of a gated GQA layer, crates/inference-backend-metal/src/components/metal/gqa_activation_gate.metal:13-27:
// sigmoid(x) = y or 1 - y with y = 1 / (1 + exp(-|x|)); in a 2-byte type every step is rounded to that type.
template <typename Tag>
__device__ __forceinline__ float gate_sigmoid(float x) {
    const float abs_x = round_through<Tag>(fabsf(x));
    const float exp_x = round_through<Tag>(expf(-abs_x));
    const float denom = round_through<Tag>(1.0f + exp_x);
    const float y = round_through<Tag>(1.0f / denom);
    return x < 0.0f ? round_through<Tag>(1.0f - y) : y;
}

// Active counts at kernel run time.  `replay_counts` (null or device u32[4] = {tokens, Q-token tiles, KV
// splits, reserved}) lets a captured launch serve any batch of its capacity bucket: the value passed
// with the launch is then only an upper bound.  Index constants below.
constexpr int kReplayTokens = 0, kReplayTiles = 1, kReplaySplits = 2, kReplayLayer = 3;
__device__ __forceinline__ uint32_t active_count(const uint32_t* replay_counts, int which, uint32_t by_value) {
    return replay_counts != nullptr ? min(replay_counts[which], by_value) : by_value;
}

// Word 3 of the block carries the page-table layer of the launch, plus one (`gqa_layer_index` bound as a
// parameter, crates/inference-executor-metal/src/model/qwen/v3_5/mtp/layer.rs:88); zero leaves the by-value layer
// in force.  Clamped to the table's layers, so that a stale block cannot index outside it.
__device__ __forceinline__ uint32_t active_layer(const uint32_t* replay_counts, uint32_t by_value, uint32_t num_layers) {
    if (replay_counts == nullptr) return by_value;
    const uint32_t bound = replay_counts[kReplayLayer];
    return bound == 0 ? by_value : min(bound - 1, num_layers - 1);
}

// Page-table walk shared by every attention kernel; the expressions of
// crates/inference-backend-metal/src/components/metal/gqa_split_kv_single_q_map.metal:96-111.
struct PageWalk {
    const uint32_t* page_ids;
    uint32_t num_layers, num_blocks, ids_per_block, tokens_per_page;
    uint32_t hkv, d;
    uint64_t page_elems;
};

__device__ __forceinline__ uint64_t page_id_for(const PageWalk& w, uint32_t req_slot, uint32_t layer, uint32_t token) {
    const uint32_t block = token / (w.tokens_per_page * w.ids_per_block);
    const uint32_t id_index = (token / w.tokens_per_page) % w.ids_per_block;
    const uint64_t table_index =
        (((uint64_t)req_slot * w.num_layers + layer) * w.num_blocks + block) * w.ids_per_block + id_index;
    return w.page_ids[table_index];
}

// Element offset of (kind, kv_head, token, dim 0); kind 0 = K, 1 = V.
__device__ __forceinline__ uint64_t kv_line_offset(const PageWalk& w, uint32_t req_slot, uint32_t layer,
                                                   uint32_t token, uint32_t kind, uint32_t kv_head) {
    const uint64_t page_id = page_id_for(w, req_slot, layer, token);
    const uint32_t page_token = token % w.tokens_per_page;
    return page_id * w.page_elems + (((uint64_t)kind * w.hkv + kv_head) * w.tokens_per_page + page_token) * w.d;
}

}  // namespace psi
