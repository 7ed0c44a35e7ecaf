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

// A bare stream in the attention kernels' page layout and load shape: a tile is 16 rows of 512 bytes of K and of V
// inside a 64 KiB page (K of head h at h * 8 KiB, V at 32 KiB + h * 8 KiB), the pages are visited in a scattered
// order, one load instruction fetches 8 rows x one 128-byte line straight into LDS, and a wave keeps at most
// kOutstanding + 1 of them in flight.  What this reads per second is the ceiling of the access pattern.
template <int kOutstanding>
__global__ __launch_bounds__(256) void psi_page_stream_probe(const unsigned char* __restrict__ src,
                                                             uint32_t tiles_per_wave, uint32_t num_pages) {
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * 16384];
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const uint32_t wave_global = blockIdx.x * (blockDim.x >> 6) + wave;
    const uint32_t base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char*)(lds) + wave * 16384;
    const uint32_t lane_offset = (lane & 7) * 512 + (lane >> 3) * 16;
    for (uint32_t t = 0; t < tiles_per_wave; ++t) {
        const uint32_t seq = wave_global * tiles_per_wave + t;
        const uint32_t page = (uint32_t)(((uint64_t)(seq >> 2) * 2654435761u) % num_pages);  // 4 heads share a page
        const unsigned char* tile = src + (uint64_t)page * 65536 + (seq & 3) * 8192 + lane_offset;
#pragma unroll
        for (int kv = 0; kv < 2; ++kv)
#pragma unroll
            for (int half = 0; half < 2; ++half)
#pragma unroll
                for (int line = 0; line < 4; ++line) {
                    const uint32_t dst = base + (kv * 8 + half * 4 + line) * 1024;
                    asm volatile(
                        "s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt\n\ts_waitcnt vmcnt(%2)" ::"s"(dst),
                        "v"(tile + kv * 32768 + half * 4096 + line * 128), "n"(kOutstanding)
                        : "memory", "m0");
                }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace

// Streams `bytes` (a multiple of 4 MiB: 256 workgroups x 4 waves x whole tiles) of `src` as described above.
// outstanding: 1, 2, 4, 8 or 32 loads in flight per wave.  Returns 0, -1 for a bad argument, or the hipError_t.
extern "C" int psi_probe_page_stream(void* stream, const void* src, uint64_t bytes, int outstanding) {
    if (src == nullptr || bytes == 0 || bytes % (1024ull * 16384) != 0 || bytes / 65536 > 0xffffffffull) return -1;
    const uint32_t tiles_per_wave = static_cast<uint32_t>(bytes / 16384 / 1024), pages = static_cast<uint32_t>(bytes / 65536);
    const unsigned char* p = static_cast<const unsigned char*>(src);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (outstanding) {
        case 1: hipLaunchKernelGGL(psi_page_stream_probe<0>, dim3(256), dim3(256), 0, s, p, tiles_per_wave, pages); break;
        case 2: hipLaunchKernelGGL(psi_page_stream_probe<1>, dim3(256), dim3(256), 0, s, p, tiles_per_wave, pages); break;
        case 4: hipLaunchKernelGGL(psi_page_stream_probe<3>, dim3(256), dim3(256), 0, s, p, tiles_per_wave, pages); break;
        case 8: hipLaunchKernelGGL(psi_page_stream_probe<7>, dim3(256), dim3(256), 0, s, p, tiles_per_wave, pages); break;
        case 32: hipLaunchKernelGGL(psi_page_stream_probe<31>, dim3(256), dim3(256), 0, s, p, tiles_per_wave, pages); break;
        default: return -1;
    }
    return static_cast<int>(hipGetLastError());
}

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
