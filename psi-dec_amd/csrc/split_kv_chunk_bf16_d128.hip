// Instantiates the gfx950 prefill-chunk map for bf16 K/V, head_dim 128.
#include "split_kv_chunk_kernel.h"

namespace psi {
int launch_chunk_map_bf16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, const uint32_t* row_groups,
                               uint32_t group_tiles, uint32_t num_groups) {
    return launch_chunk_map_typed<BF16Tag, 128>(ctx, g, a, row_groups, group_tiles, num_groups);
}
}  // namespace psi
