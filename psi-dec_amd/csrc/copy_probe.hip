// A plain device-to-device copy of known size.  It exists for measurement only: the HBM traffic
// counters of this GPU are calibrated against it (bytes the counter reports for a copy of N bytes),
// and its rate is the practical read+write ceiling the attention kernels are compared with.
#include "common.h"

namespace {

__global__ void __launch_bounds__(256) psi_copy_probe(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                       uint64_t count) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride)
        dst[i] = src[i];
}

__global__ void __launch_bounds__(256) psi_read_probe(const uint4* __restrict__ src, uint4* __restrict__ sink,
                                                       uint64_t count) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    uint4 acc = make_uint4(0, 0, 0, 0);
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += stride) {
        const uint4 v = src[i];
        acc.x ^= v.x;
        acc.y ^= v.y;
        acc.z ^= v.z;
        acc.w ^= v.w;
    }
    // Never true for the probe's inputs, but keeps the loads alive.
    if ((acc.x & acc.y & acc.z & acc.w) == 0xFFFFFFFFu) sink[0] = acc;
}

}  // namespace

extern "C" int psi_hip_copy_probe(psi_hip_ctx* ctx, void* dst, const void* src, uint64_t bytes, int read_only) {
    PSI_REQUIRE(ctx != nullptr && dst != nullptr && src != nullptr, "ctx, dst and src must not be null");
    PSI_REQUIRE(bytes != 0 && bytes % 16 == 0, "probe size must be a positive multiple of 16 bytes");
    PSI_REQUIRE((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16 == 0,
                "probe buffers must be 16-byte aligned");
    const uint64_t count = bytes / 16;
    const uint64_t want = (count + 255) / 256;
    const unsigned grid = static_cast<unsigned>(want < 256ull * 16 ? want : 256ull * 16);
    psi::LaunchScope scope(ctx, read_only ? "read_probe" : "copy_probe");
    if (read_only)
        hipLaunchKernelGGL(psi_read_probe, dim3(grid), dim3(256), 0, ctx->stream, static_cast<const uint4*>(src),
                           static_cast<uint4*>(dst), count);
    else
        hipLaunchKernelGGL(psi_copy_probe, dim3(grid), dim3(256), 0, ctx->stream, static_cast<const uint4*>(src),
                           static_cast<uint4*>(dst), count);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}
