// gfx950 MFMA path of the TiledQ map (speculative verify, prefill chunks).
#include "split_kv.h"

namespace psi {

int launch_tiled_map_fast(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    (void)ctx;
    (void)g;
    (void)a;
    return PSI_HIP_ERR_UNSUPPORTED;
}

}  // namespace psi
