// Instantiates the gfx950 decode map for f16 K/V, head_dim 128 (all group sizes and workgroup widths).
#include "split_kv_decode_kernel.h"

namespace psi {
int launch_decode_map_f16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    return launch_decode_map_group<F16Tag, 128>(ctx, g, a);
}
}  // namespace psi
