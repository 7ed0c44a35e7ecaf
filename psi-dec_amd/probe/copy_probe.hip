// A plain device-to-device copy and a pure read of known size.  Measurement only, built into its own
// library (lib/libpsi_hip_probe.so) so that the attention library ships nothing it does not need: the HBM
// traffic counters of this GPU are calibrated against the copy (bytes the counter reports for a copy of N
// bytes), and the rates are the practical ceilings the attention kernels are compared with.
#include <hip/hip_runtime.h>

#include <cstdint>

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

// stream: a hipStream_t.  Returns 0, -1 for a bad argument, or the positive hipError_t of the launch.
extern "C" int psi_probe_copy(void* stream, void* dst, const void* src, uint64_t bytes, int read_only) {
    if (dst == nullptr || src == nullptr || bytes == 0 || bytes % 16 != 0) return -1;
    if ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) % 16 != 0) return -1;
    const uint64_t count = bytes / 16;
    const uint64_t want = (count + 255) / 256;
    const unsigned grid = static_cast<unsigned>(want < 256ull * 16 ? want : 256ull * 16);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (read_only)
        hipLaunchKernelGGL(psi_read_probe, dim3(grid), dim3(256), 0, s, static_cast<const uint4*>(src),
                           static_cast<uint4*>(dst), count);
    else
        hipLaunchKernelGGL(psi_copy_probe, dim3(grid), dim3(256), 0, s, static_cast<const uint4*>(src),
                           static_cast<uint4*>(dst), count);
    return static_cast<int>(hipGetLastError());
}
