// Dispatch of the gfx950 multi-query (TiledQ) map, instantiated per element type and head_dim in
// the split_kv_tiled_*.hip files.
#include "split_kv.h"

namespace psi {

int launch_tiled_map_bf16_d256(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, uint32_t max_tile_tokens);
int launch_tiled_map_bf16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, uint32_t max_tile_tokens);
int launch_tiled_map_f16_d256(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, uint32_t max_tile_tokens);
int launch_tiled_map_f16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, uint32_t max_tile_tokens);

int launch_chunk_map_bf16_d256(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                               uint32_t group_tiles, uint32_t num_groups);
int launch_chunk_map_f16_d256(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                              uint32_t group_tiles, uint32_t num_groups);
int launch_chunk_map_bf16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                               uint32_t group_tiles, uint32_t num_groups);
int launch_chunk_map_f16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                              uint32_t group_tiles, uint32_t num_groups);

int launch_chunk_map(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                     uint32_t group_tiles, uint32_t num_groups) {
    if (ctx->force_generic || !chunk_map_supported(g, a.rows_per_split_head)) return PSI_HIP_ERR_UNSUPPORTED;
    const bool aligned = reinterpret_cast<uintptr_t>(a.q) % 16 == 0 && reinterpret_cast<uintptr_t>(a.kv_pages) % 16 == 0;
    if (!aligned || group_tiles == 0 || group_tiles > chunk_group_tiles(g.group, a.rows_per_split_head)) return PSI_HIP_ERR_UNSUPPORTED;
    if ((uint64_t)num_groups * g.hkv * chunk_head_subsets(g.group) > 0x7fffffffull) return PSI_HIP_ERR_UNSUPPORTED;
    if (g.d == 128)
        return g.dtype == PSI_HIP_BF16 ? launch_chunk_map_bf16_d128(ctx, g, a, row_groups, group_tiles, num_groups)
                                       : launch_chunk_map_f16_d128(ctx, g, a, row_groups, group_tiles, num_groups);
    return g.dtype == PSI_HIP_BF16 ? launch_chunk_map_bf16_d256(ctx, g, a, row_groups, group_tiles, num_groups)
                                   : launch_chunk_map_f16_d256(ctx, g, a, row_groups, group_tiles, num_groups);
}

int launch_tiled_map_fast(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    if (ctx->force_generic) return PSI_HIP_ERR_UNSUPPORTED;
    const bool two_byte = g.dtype == PSI_HIP_BF16 || g.dtype == PSI_HIP_F16;
    const uint32_t p = g.tokens_per_page;
    const bool page_ok = p >= 8 && (p & (p - 1)) == 0;
    const bool aligned = reinterpret_cast<uintptr_t>(a.q) % 16 == 0 && reinterpret_cast<uintptr_t>(a.kv_pages) % 16 == 0;
    // partial rows are laid out for 8-token tiles; the kernels hold at most 64 query columns
    if (!two_byte || !page_ok || !aligned || (g.d != 256 && g.d != 128) || a.rows_per_split_head > 8) return PSI_HIP_ERR_UNSUPPORTED;
    uint32_t max_tile_tokens = a.max_q_tile_tokens == 0 ? a.rows_per_split_head : a.max_q_tile_tokens;
    if (max_tile_tokens > a.rows_per_split_head) max_tile_tokens = a.rows_per_split_head;
    if (max_tile_tokens * g.group > 64) return PSI_HIP_ERR_UNSUPPORTED;
    if ((uint64_t)a.num_total_kv_splits * g.hkv > 0x7fffffffull) return PSI_HIP_ERR_UNSUPPORTED;
    // More columns than the paired pipeline holds (8 tokens x 7 or 8 heads per KV head): the row-group kernel with
    // every row a group of its own, which takes 256 columns and reads the row's K/V once.
    if (max_tile_tokens * g.group > 48) return launch_chunk_map(ctx, g, a, nullptr, 1, a.num_total_kv_splits);
    if (g.dtype == PSI_HIP_BF16)
        return g.d == 256 ? launch_tiled_map_bf16_d256(ctx, g, a, max_tile_tokens)
                          : launch_tiled_map_bf16_d128(ctx, g, a, max_tile_tokens);
    return g.d == 256 ? launch_tiled_map_f16_d256(ctx, g, a, max_tile_tokens)
                      : launch_tiled_map_f16_d128(ctx, g, a, max_tile_tokens);
}

}  // namespace psi
