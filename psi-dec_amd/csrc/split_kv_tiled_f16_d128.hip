// Instantiates the gfx950 multi-query map for f16 K/V, head_dim 128 (1..4 column blocks).
#include "split_kv_tiled_kernel.h"

namespace psi {
int launch_tiled_map_f16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a, uint32_t max_tile_tokens) {
    return launch_tiled_map_typed<F16Tag, 128>(ctx, g, a, max_tile_tokens);
}
}  // namespace psi
