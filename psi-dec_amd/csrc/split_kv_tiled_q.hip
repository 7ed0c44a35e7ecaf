// Split-KV multi-query attention (TiledQ): C-ABI entry points for speculative verify and prefill
// chunks.  A kv_split row names a request-local tile of up to q_token_tile_size Q tokens; keys
// after a query's own position are hidden (causal among the new tokens).  Semantics follow
// crates/inference-backend-metal/src/components/metal/gqa_split_kv_tiled_q.metal:49-378.
#include "split_kv.h"

namespace psi {

constexpr float kLog2eTiled = 1.4426950408889634f;

// gqa_split_kv_tiled_q.rs:171-186
static int check_tiled_shape(const Geometry& g, uint32_t q_token_tile_size, uint32_t num_total_tokens,
                             uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits) {
    PSI_REQUIRE(g.scale > 0.0f, "GQA attention scale must be positive");
    PSI_REQUIRE(q_token_tile_size > 0 && q_token_tile_size <= 64, "GQA Q-token tile size must be in 1..64");
    PSI_REQUIRE(num_total_tokens > 0, "GQA SplitKV TiledQ requires tokens");
    PSI_REQUIRE(num_total_q_token_tiles > 0 && num_total_q_token_tiles <= num_total_tokens,
                "GQA SplitKV TiledQ requires 0 < q_token_tiles <= tokens");
    PSI_REQUIRE(num_total_kv_splits >= num_total_q_token_tiles,
                "GQA SplitKV TiledQ requires at least one KV split per Q-token tile");
    PSI_REQUIRE((uint64_t)num_total_q_token_tiles * 2 - 1 <= UINT32_MAX,
                "GQA SplitKV TiledQ Q-token-tile metadata exceeds the shader u32 element-index domain");
    PSI_REQUIRE((uint64_t)num_total_kv_splits * 3 - 1 <= UINT32_MAX,
                "GQA SplitKV TiledQ map TaskTemplate metadata exceeds the shader u32 element-index domain");
    return PSI_HIP_OK;
}

}  // namespace psi

using namespace psi;

extern "C" int psi_hip_split_kv_tiled_q_scratch_bytes(const psi_hip_gqa_config* cfg, uint32_t q_token_tile_size,
                                                      uint32_t num_total_kv_splits, uint64_t* out_bytes) {
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_bytes != nullptr, "out pointer must not be null");
    PSI_REQUIRE(q_token_tile_size > 0 && q_token_tile_size <= 64, "GQA Q-token tile size must be in 1..64");
    PSI_REQUIRE(num_total_kv_splits > 0, "GQA SplitKV TiledQ requires KV splits");
    *out_bytes = partial_layout(num_total_kv_splits, g.hq, g.d, q_token_tile_size).total_bytes;
    return PSI_HIP_OK;
}

// Shared body of the two map entry points; row_groups == nullptr: one workgroup per (row, KV head).
static int tiled_q_map(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
                       uint32_t q_token_tile_size, const void* q, const void* kv_pages, uint64_t kv_pages_bytes,
                       const uint32_t* req_slots, const uint32_t* page_ids, const uint32_t* flat_token_indices,
                       const uint32_t* q_token_tiles, const uint32_t* kv_splits, void* scratch, uint64_t scratch_bytes,
                       uint32_t gqa_layer_index, uint32_t num_total_tokens, uint32_t num_total_q_token_tiles,
                       uint32_t num_total_kv_splits, uint32_t num_active_tokens, uint32_t num_active_q_token_tiles,
                       uint32_t num_active_kv_splits, uint32_t max_active_q_tile_tokens, const uint32_t* row_groups,
                       uint32_t group_tiles, uint32_t num_groups, const uint32_t* worker_cu = nullptr,
                       uint32_t num_workers = 0) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_layout(layout);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_tiled_shape(g, q_token_tile_size, num_total_tokens, num_total_q_token_tiles, num_total_kv_splits);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(q && kv_pages && req_slots && page_ids && flat_token_indices && q_token_tiles && kv_splits && scratch,
                "GQA SplitKV TiledQ map buffers must not be null");
    PSI_REQUIRE(gqa_layer_index < layout->num_gqa_layers, "GQA page-table index exceeds layer count");
    PSI_REQUIRE(num_active_tokens > 0 && num_active_tokens <= num_total_tokens,
                "GQA SplitKV TiledQ active token count must be in 1..capacity");
    PSI_REQUIRE(num_active_q_token_tiles > 0 && num_active_q_token_tiles <= num_total_q_token_tiles,
                "GQA SplitKV TiledQ active Q-token-tile count must be in 1..capacity");
    PSI_REQUIRE(num_active_kv_splits > 0 && num_active_kv_splits <= num_total_kv_splits,
                "GQA SplitKV TiledQ active KV split count must be in 1..capacity");
    PSI_REQUIRE(kv_pages_bytes == 0 || kv_pages_bytes >= cfg->page_bytes, "GQA page arena is smaller than one page");
    const PartialLayout pl = partial_layout(num_total_kv_splits, g.hq, g.d, q_token_tile_size);
    PSI_REQUIRE(scratch_bytes >= pl.total_bytes, "GQA SplitKV TiledQ scratch too small: %llu < %llu",
                (unsigned long long)scratch_bytes, (unsigned long long)pl.total_bytes);

    MapArgs a;
    a.q = q;
    a.kv_pages = kv_pages;
    a.req_slots = req_slots;
    a.kv_splits = kv_splits;
    a.part_max = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.max_offset);
    a.part_sum = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.sum_offset);
    a.part_acc = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.acc_offset);
    fill_walk(&a.walk, g, layout, page_ids);
    a.layer = gqa_layer_index;
    a.hq = g.hq;
    a.group = g.group;
    a.num_total_kv_splits = num_total_kv_splits;
    a.num_active_tokens = num_active_tokens;
    a.num_active_kv_splits = num_active_kv_splits;
    a.replay_counts = ctx->replay_counts;
    set_device_status(&a, ctx);
    a.scale_log2 = g.scale * kLog2eTiled;
    a.q_token_tiles = q_token_tiles;
    a.flat_token_indices = flat_token_indices;
    a.rows_per_split_head = q_token_tile_size;
    a.num_active_q_token_tiles = num_active_q_token_tiles;
    PSI_REQUIRE(max_active_q_tile_tokens <= q_token_tile_size,
                "GQA SplitKV TiledQ largest active tile exceeds the Q-token tile size");
    a.max_q_tile_tokens = max_active_q_tile_tokens;
    a.worker_cu = worker_cu;
    a.num_workers = num_workers;

    LaunchScope scope(ctx, "tiled_q_map");
    rc = PSI_HIP_ERR_UNSUPPORTED;
    if (row_groups != nullptr && num_groups != 0) rc = launch_chunk_map(ctx, g, a, row_groups, group_tiles, num_groups);
    if (rc == PSI_HIP_ERR_UNSUPPORTED) rc = launch_tiled_map_fast(ctx, g, a);
    if (rc == PSI_HIP_ERR_UNSUPPORTED) {
        a.worker_cu = nullptr;  // the generic kernel launches one workgroup per row
        a.num_workers = 0;
        const uint64_t grid = (uint64_t)num_total_kv_splits * g.hq * q_token_tile_size * ((g.d + 63) / 64);
        PSI_REQUIRE(grid <= 0x7fffffffull, "GQA SplitKV TiledQ map grid exceeds the launch domain");
        launch_map_generic(ctx, g, a);
        rc = PSI_HIP_OK;
    }
    if (rc != PSI_HIP_OK) return rc;
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_split_kv_tiled_q_map(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                            const psi_hip_page_table_layout* layout, uint32_t q_token_tile_size,
                                            const void* q, const void* kv_pages, uint64_t kv_pages_bytes,
                                            const uint32_t* req_slots, const uint32_t* page_ids,
                                            const uint32_t* flat_token_indices, const uint32_t* q_token_tiles,
                                            const uint32_t* kv_splits, void* scratch, uint64_t scratch_bytes,
                                            uint32_t gqa_layer_index, uint32_t num_total_tokens,
                                            uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits,
                                            uint32_t num_active_tokens, uint32_t num_active_q_token_tiles,
                                            uint32_t num_active_kv_splits, uint32_t max_active_q_tile_tokens) {
    return tiled_q_map(ctx, cfg, layout, q_token_tile_size, q, kv_pages, kv_pages_bytes, req_slots, page_ids,
                       flat_token_indices, q_token_tiles, kv_splits, scratch, scratch_bytes, gqa_layer_index,
                       num_total_tokens, num_total_q_token_tiles, num_total_kv_splits, num_active_tokens,
                       num_active_q_token_tiles, num_active_kv_splits, max_active_q_tile_tokens, nullptr, 0, 0);
}

extern "C" int psi_hip_split_kv_tiled_q_map_balanced(
    psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
    uint32_t q_token_tile_size, const void* q, const void* kv_pages, uint64_t kv_pages_bytes,
    const uint32_t* req_slots, const uint32_t* page_ids, const uint32_t* flat_token_indices,
    const uint32_t* q_token_tiles, const uint32_t* kv_splits, const uint32_t* worker_cu, uint32_t num_workers,
    void* scratch, uint64_t scratch_bytes, uint32_t gqa_layer_index, uint32_t num_total_tokens,
    uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits, uint32_t num_active_tokens,
    uint32_t num_active_q_token_tiles, uint32_t num_active_kv_splits, uint32_t max_active_q_tile_tokens) {
    PSI_REQUIRE(worker_cu != nullptr && num_workers > 0, "balanced map needs a worker table");
    return tiled_q_map(ctx, cfg, layout, q_token_tile_size, q, kv_pages, kv_pages_bytes, req_slots, page_ids,
                       flat_token_indices, q_token_tiles, kv_splits, scratch, scratch_bytes, gqa_layer_index,
                       num_total_tokens, num_total_q_token_tiles, num_total_kv_splits, num_active_tokens,
                       num_active_q_token_tiles, num_active_kv_splits, max_active_q_tile_tokens, nullptr, 0, 0,
                       worker_cu, num_workers);
}

extern "C" int psi_hip_split_kv_tiled_q_map_grouped(
    psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
    uint32_t q_token_tile_size, const void* q, const void* kv_pages, uint64_t kv_pages_bytes,
    const uint32_t* req_slots, const uint32_t* page_ids, const uint32_t* flat_token_indices,
    const uint32_t* q_token_tiles, const uint32_t* kv_splits, void* scratch, uint64_t scratch_bytes,
    uint32_t gqa_layer_index, uint32_t num_total_tokens, uint32_t num_total_q_token_tiles,
    uint32_t num_total_kv_splits, uint32_t num_active_tokens, uint32_t num_active_q_token_tiles,
    uint32_t num_active_kv_splits, uint32_t max_active_q_tile_tokens, const uint32_t* row_groups,
    uint32_t group_tiles, uint32_t num_groups) {
    PSI_REQUIRE(row_groups != nullptr && group_tiles > 0 && num_groups > 0,
                "GQA SplitKV TiledQ grouped map requires a row-group table");
    PSI_REQUIRE(group_tiles <= 32, "GQA SplitKV TiledQ row groups hold at most 32 tiles");
    return tiled_q_map(ctx, cfg, layout, q_token_tile_size, q, kv_pages, kv_pages_bytes, req_slots, page_ids,
                       flat_token_indices, q_token_tiles, kv_splits, scratch, scratch_bytes, gqa_layer_index,
                       num_total_tokens, num_total_q_token_tiles, num_total_kv_splits, num_active_tokens,
                       num_active_q_token_tiles, num_active_kv_splits, max_active_q_tile_tokens, row_groups,
                       group_tiles, num_groups);
}

extern "C" int psi_hip_split_kv_tiled_q_reduce(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                               uint32_t q_token_tile_size, const void* scratch,
                                               uint64_t scratch_bytes, const uint32_t* q_token_tiles,
                                               const uint32_t* cu_kv_splits, void* output, uint32_t num_total_tokens,
                                               uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits,
                                               uint32_t num_active_q_token_tiles,
                                               const uint32_t* partial_row_index, const psi_hip_output_gate* gate) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_tiled_shape(g, q_token_tile_size, num_total_tokens, num_total_q_token_tiles, num_total_kv_splits);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(scratch && q_token_tiles && cu_kv_splits && output,
                "GQA SplitKV TiledQ reduce buffers must not be null");
    PSI_REQUIRE(num_active_q_token_tiles > 0 && num_active_q_token_tiles <= num_total_q_token_tiles,
                "GQA SplitKV TiledQ active Q-token-tile count must be in 1..capacity");
    const PartialLayout pl = partial_layout(num_total_kv_splits, g.hq, g.d, q_token_tile_size);
    PSI_REQUIRE(scratch_bytes >= pl.total_bytes, "GQA SplitKV TiledQ scratch too small: %llu < %llu",
                (unsigned long long)scratch_bytes, (unsigned long long)pl.total_bytes);
    ReduceArgs a;
    a.part_max = reinterpret_cast<const float*>(static_cast<const char*>(scratch) + pl.max_offset);
    a.part_sum = reinterpret_cast<const float*>(static_cast<const char*>(scratch) + pl.sum_offset);
    a.part_acc = reinterpret_cast<const float*>(static_cast<const char*>(scratch) + pl.acc_offset);
    a.cu_kv_splits = cu_kv_splits;
    a.row_index = partial_row_index;
    a.replay_counts = ctx->replay_counts;
    a.output = output;
    a.hq = g.hq;
    a.d = g.d;
    a.out_dtype = ctx->f32_output ? PSI_HIP_F32 : g.dtype;
    a.num_active_tokens = num_total_tokens;
    a.q_token_tiles = q_token_tiles;
    a.rows_per_split_head = q_token_tile_size;
    a.num_active_q_token_tiles = num_active_q_token_tiles;
    rc = set_output_gate(&a, gate, g);
    if (rc != PSI_HIP_OK) return rc;

    LaunchScope scope(ctx, "tiled_q_reduce");
    if (launch_reduce_fast(ctx, g, a) == PSI_HIP_ERR_UNSUPPORTED) launch_reduce_generic(ctx, g, a, num_active_q_token_tiles);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}
