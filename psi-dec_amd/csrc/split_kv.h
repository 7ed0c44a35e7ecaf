// Shared declarations of the split-KV attention kernels: scratch layout and kernel arguments.
#pragma once
#include "common.h"
#include "device_types.h"

namespace psi {

// Partial state of one (kv_split, q_head [, q_token_in_tile]) row, private to this library:
//   max2 : reference value of the row's logits in the log2 domain (logit * scale * log2(e)), -inf if empty: their
//          maximum, or (multi-query and chunk maps) a value at most 8 below it - the combine only needs sum and acc
//          to be relative to the same value
//   sum  : sum of exp2(logit2 - max2) over the split's keys
//   acc  : un-normalised sum of exp2(logit2 - max2) * V, f32 [head_dim]
// Arrays are laid out [row][...] with row = (split * num_q_heads + q_head) * rows_per_split_head + r.
struct PartialLayout {
    uint64_t rows;
    uint64_t max_offset, sum_offset, acc_offset, total_bytes;
};

inline PartialLayout partial_layout(uint64_t num_total_kv_splits, uint32_t hq, uint32_t d,
                                    uint32_t rows_per_split_head) {
    PartialLayout l;
    l.rows = num_total_kv_splits * hq * rows_per_split_head;
    auto align = [](uint64_t v) { return (v + 255) & ~uint64_t(255); };
    l.max_offset = 0;
    l.sum_offset = align(l.rows * 4);
    l.acc_offset = l.sum_offset + align(l.rows * 4);
    l.total_bytes = l.acc_offset + align(l.rows * d * 4);
    return l;
}

struct MapArgs {
    const void* q;
    const void* kv_pages;
    const uint32_t* req_slots;
    const uint32_t* kv_splits;
    float* part_max;
    float* part_sum;
    float* part_acc;
    PageWalk walk;
    uint32_t layer;
    uint32_t hq, group;
    uint32_t num_total_kv_splits;
    uint32_t num_active_tokens, num_active_kv_splits;
    float scale_log2;  // scale * log2(e)
    // TiledQ only (null / 1 / 0 for SingleQ): kv_splits rows then name Q-token tiles.
    const uint32_t* q_token_tiles = nullptr;       // [tiles][2] = flat token begin, end
    const uint32_t* flat_token_indices = nullptr;  // request-absolute position of each flat token
    uint32_t rows_per_split_head = 1;              // q_token_tile_size
    uint32_t num_active_q_token_tiles = 0;
    uint32_t max_q_tile_tokens = 0;                // largest active tile (0: up to rows_per_split_head)
    // Balanced decode launch only: workgroup w of a KV head serves kv_splits rows
    // [worker_cu[w], worker_cu[w + 1]).
    const uint32_t* worker_cu = nullptr;
    uint32_t num_workers = 0;
    const uint32_t* replay_counts = nullptr;  // see active_count()
    // Decode map with the append folded in (null otherwise): the step's new K/V rows [token][Hkv][D].  The
    // workgroup whose row ends at a token's own position writes that token's lines into its page, and every
    // position appended in this step is read from these rows instead of the page.
    const void* flat_k = nullptr;
    const void* flat_v = nullptr;
    // Where a kernel reports a row that it could not compute (word i = bit i of PSI_HIP_DEVICE_ERR_*); and, for
    // harnesses, non-zero: the loading waves of the multi-query and prefill-chunk maps do not say that their tiles
    // have landed, so that the other waves' waits run out.
    uint32_t* status = nullptr;
    uint32_t mute_loaders = 0;
    // Prefill-chunk map: the context's two work-sharing words (psi_hip_ctx::work_claim).
    uint32_t* work_claim = nullptr;
};

// Fills the three fields above from the context.
inline void set_device_status(MapArgs* a, const psi_hip_ctx* ctx) {
    a->status = ctx->status_device;
    a->mute_loaders = ctx->mute_loaders ? 1u : 0u;
    a->work_claim = ctx->work_claim;
}

// First statement of every map kernel.
__device__ __forceinline__ void resolve_active(MapArgs& a) {
    a.num_active_tokens = active_count(a.replay_counts, kReplayTokens, a.num_active_tokens);
    a.num_active_q_token_tiles = active_count(a.replay_counts, kReplayTiles, a.num_active_q_token_tiles);
    a.num_active_kv_splits = active_count(a.replay_counts, kReplaySplits, a.num_active_kv_splits);
    a.layer = active_layer(a.replay_counts, a.layer, a.walk.num_layers);
}

struct ReduceArgs {
    const float* part_max;
    const float* part_sum;
    const float* part_acc;
    const uint32_t* cu_kv_splits;
    void* output;
    uint32_t hq, d;
    uint32_t num_active_tokens;
    uint32_t num_total_kv_splits = 0;  // capacity of the split list (sizes the combine's parallelism)
    uint32_t out_dtype = PSI_HIP_F32;  // element type of `output`
    // Optional: the partial rows of token / tile t are row_index[cu[t] .. cu[t + 1]) instead of
    // cu[t] .. cu[t + 1] themselves (plans whose rows were re-ordered for dispatch).
    const uint32_t* row_index = nullptr;
    // TiledQ only: cu_kv_splits is indexed by Q-token tile.
    const uint32_t* q_token_tiles = nullptr;
    uint32_t rows_per_split_head = 1;
    uint32_t num_active_q_token_tiles = 0;
    // Optional attention-output gate: element (token, q_head, d) at gates[token * gate_token_stride +
    // q_head * gate_head_stride + d], in gate_dtype (the IO dtype of the layer).
    const void* gates = nullptr;
    uint64_t gate_token_stride = 0, gate_head_stride = 0;
    uint32_t gate_dtype = PSI_HIP_F32;
    const uint32_t* replay_counts = nullptr;  // see active_count()
};

// First statement of every combine kernel.
__device__ __forceinline__ void resolve_active(ReduceArgs& a) {
    a.num_active_tokens = active_count(a.replay_counts, kReplayTokens, a.num_active_tokens);
    a.num_active_q_token_tiles = active_count(a.replay_counts, kReplayTiles, a.num_active_q_token_tiles);
}

// The combine's last step: the output element in f32 -> what is stored.  With a gate the element is
// first rounded to the output type, as the separate attention output would have been, then
// multiplied by sigmoid(gate) in that type (gqa_activation_gate.metal:29-38).
template <typename Tag>
__device__ __forceinline__ float finish_output(const ReduceArgs& a, float value, uint32_t token, uint32_t q_head,
                                               uint32_t d) {
    if (a.gates == nullptr) return value;
    const float gate = load_any_as_f32(a.gates, token * a.gate_token_stride + q_head * a.gate_head_stride + d, a.gate_dtype);
    return round_through<Tag>(value) * gate_sigmoid<Tag>(gate);
}

// Copies an optional psi_hip_output_gate into the kernel arguments; PSI_HIP_OK or an argument error.
inline int set_output_gate(ReduceArgs* a, const psi_hip_output_gate* gate, const Geometry& g) {
    if (gate == nullptr) return PSI_HIP_OK;
    PSI_REQUIRE(gate->gates != nullptr, "GQA output gate pointer must not be null");
    PSI_REQUIRE(gate->head_stride >= g.d && gate->token_stride >= (uint64_t)(g.hq - 1) * gate->head_stride + g.d,
                "GQA output gate strides overlap rows");
    a->gates = gate->gates;
    a->gate_token_stride = gate->token_stride;
    a->gate_head_stride = gate->head_stride;
    a->gate_dtype = g.dtype;
    return PSI_HIP_OK;
}

// Prefill-chunk map: a workgroup serves up to kChunkCols query columns (tokens of a row group x
// heads).  The heads of one KV head are dealt to chunk_head_subsets() workgroups, and a row group
// holds up to chunk_group_tiles() Q-token tiles (0: the shape does not fit the kernel).
constexpr int kChunkCols = 256;
// Six heads per KV head go to three workgroups of two (two heads x 128 tokens fill the 256 columns; three heads x 80
// tokens would leave sixteen of them empty).
// Keys of one KV tile of the prefill-chunk map (16 KiB of K and of V at either head_dim).
constexpr uint32_t chunk_tile_keys(uint32_t d) { return d == 128 ? 64u : 32u; }
inline uint32_t chunk_head_subsets(uint32_t group) { return group == 6 ? 3u : (group > 5 ? 2u : 1u); }
inline uint32_t chunk_group_tiles(uint32_t group, uint32_t q_token_tile_size) {
    const uint32_t subsets = chunk_head_subsets(group);
    const uint32_t heads = (group + subsets - 1) / subsets;
    const uint32_t tiles = (uint32_t)kChunkCols / (heads * q_token_tile_size);
    return tiles > 32 ? 32u : tiles;
}
// Q-token tiles of a row group whose tokens times all the heads of a KV head fit the columns of one workgroup.
inline uint32_t chunk_all_heads_tiles(uint32_t group, uint32_t q_token_tile_size) {
    return (uint32_t)kChunkCols / (group * q_token_tile_size);
}
// Head subsets of a launch over a row-group table `group_tiles` wide.  A table that narrow that a group's tokens
// times all the heads fit one workgroup (short chunks, verify steps) is walked without subsets: a work item then
// reads its KV range once for all the heads.  (The width of the table says it: psi_hip_split_kv_tiled_q_group_rows
// writes the narrow form when no group is wider.)
inline uint32_t chunk_launch_subsets(uint32_t group, uint32_t group_tiles, uint32_t q_token_tile_size) {
    return group_tiles <= chunk_all_heads_tiles(group, q_token_tile_size) ? 1u : chunk_head_subsets(group);
}
// True when the prefill-chunk map covers the geometry: 2-byte elements, head_dim 128 or 256, pages of 8 * 2^k tokens
// (the reference's TiledQ profiles (128, 8), (256, 8), (256, 16) among them,
// crates/inference-backend-metal/src/components/gqa_split_kv_tiled_q.rs:66-76).
inline bool chunk_map_supported(const Geometry& g, uint32_t q_token_tile_size) {
    const uint32_t p = g.tokens_per_page;
    return (g.dtype == PSI_HIP_BF16 || g.dtype == PSI_HIP_F16) && (g.d == 256 || g.d == 128) && p >= 8 &&
           (p & (p - 1)) == 0 && q_token_tile_size > 0 && chunk_group_tiles(g.group, q_token_tile_size) >= 1;
}

// Shape-generic kernels (any head_dim / page size / element type), SingleQ and TiledQ layouts.
void launch_map_generic(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);
void launch_reduce_generic(psi_hip_ctx* ctx, const Geometry& g, const ReduceArgs& a, uint32_t num_total_tokens);
void fill_walk(PageWalk* walk, const Geometry& g, const psi_hip_page_table_layout* layout, const uint32_t* page_ids);

// Fast decode map for head_dim 256 / 128, 2-byte elements, power-of-two pages; returns
// PSI_HIP_ERR_UNSUPPORTED when the shape is outside its domain (caller falls back).
int launch_decode_map_fast(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);
bool decode_map_takes_append(const psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);
int launch_reduce_fast(psi_hip_ctx* ctx, const Geometry& g, const ReduceArgs& a);
// MFMA TiledQ map for bf16 / f16, head_dim 256 / 128; PSI_HIP_ERR_UNSUPPORTED outside its domain.
int launch_tiled_map_fast(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);
// MFMA prefill-chunk map over row groups; PSI_HIP_ERR_UNSUPPORTED outside chunk_map_supported().
int launch_chunk_map(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                     uint32_t group_tiles, uint32_t num_groups);

}  // namespace psi
