// The rates that bound the prefill-chunk map, measured with nothing else in the way.  Measurement only, part of
// lib/libpsi_hip_probe.so:
//   psi_probe_mfma_rate      eight waves per compute unit (two per SIMD) issue independent v_mfma_f32_16x16x32_bf16
//                            back to back: what the matrix cores sustain at the clock the chip keeps under that load;
//   psi_probe_lds_read_rate  eight waves per compute unit read a K tile with 128-bit reads, or a V tile with the
//                            transposing 64-bit reads, in the chunk map's own layouts, conflict-free.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__global__ __launch_bounds__(512, 1) void psi_mfma_rate_probe(uint32_t iters, float* sink) {
    f32x4 acc[8];
    for (int i = 0; i < 8; ++i) acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    bf16x8 a, b;
    for (int i = 0; i < 8; ++i) {
        a[i] = (__bf16)(float)((threadIdx.x + i) & 7);
        b[i] = (__bf16)(float)((blockIdx.x + i) & 3);
    }
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[i], 0, 0, 0);
    }
    float s = 0.0f;
    for (int i = 0; i < 8; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (s == 12345.678f) sink[threadIdx.x] = s;  // (never: keeps the loop)
}

constexpr int kRowBytes = 512;  // head_dim 256, 2-byte elements

// pattern 0: the A operand of K * Q^T (16 x ds_read_b128 per wave and iteration, 16 KiB); 1: the transposed V
// operand (32 x ds_read_b64_tr_b16, 16 KiB)
__global__ __launch_bounds__(512, 1) void psi_lds_read_probe(int pattern, uint32_t iters, float* sink) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    for (uint32_t i = threadIdx.x; i < 32 * kRowBytes / 4; i += blockDim.x) reinterpret_cast<uint32_t*>(lds)[i] = i;
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t mt = lane & 15, mc = lane >> 4;
    uint32_t acc = 0;
    if (pattern == 0) {
        const uint32_t k_row0 = mt * kRowBytes;
        for (uint32_t it = 0; it < iters; ++it) {
            uint4 v[16];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) {
                const uint32_t off = k_row0 + (((4 * ks + mc) ^ mt) * 16);
                asm volatile("ds_read_b128 %0, %1" : "=v"(v[2 * ks]) : "v"(off));
                asm volatile("ds_read_b128 %0, %1 offset:8192" : "=v"(v[2 * ks + 1]) : "v"(off));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < 16; ++j) acc ^= v[j].x + v[j].y + v[j].z + v[j].w;
        }
    } else {
        const uint32_t v_key = 4 * mc + (mt >> 2);
        const uint32_t v_row0 = v_key * kRowBytes + (mt & 3) * 8;
        const uint32_t swizzle = (v_key & 7) * 32;
        for (uint32_t it = 0; it < iters; ++it) {
            uint2 v[32];
#pragma unroll
            for (int db = 0; db < 16; ++db) {
                const uint32_t off = v_row0 + ((db * 32) ^ swizzle);
                asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v[2 * db]) : "v"(off));
                asm volatile("ds_read_b64_tr_b16 %0, %1 offset:8192" : "=v"(v[2 * db + 1]) : "v"(off));
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int j = 0; j < 32; ++j) acc ^= v[j].x + v[j].y;
        }
    }
    if (acc == 0x12345678u) sink[threadIdx.x] = acc;  // (keeps the loop)
}

}  // namespace

// Launches 256 workgroups of eight waves, each wave issuing 8 * iters matrix instructions of 16 x 16 x 32 x 2 flops
// per lane group: 256 * 8 * 8 * iters * 16384 flops per launch.  stream: a hipStream_t; sink: 2 KiB of device memory
// that is never written.  Returns 0, -1 for a bad argument, or the positive hipError_t of the launch.
extern "C" int psi_probe_mfma_rate(void* stream, void* sink, uint32_t iters) {
    if (sink == nullptr || iters == 0) return -1;
    hipLaunchKernelGGL(psi_mfma_rate_probe, dim3(256), dim3(512), 0, static_cast<hipStream_t>(stream), iters,
                       static_cast<float*>(sink));
    return static_cast<int>(hipGetLastError());
}

// Launches 256 workgroups of eight waves, each wave reading 16 KiB of LDS per iteration: 256 * 8 * 16384 * iters
// bytes per launch.  pattern: 0 = 128-bit reads of a K tile, 1 = transposing 64-bit reads of a V tile.
extern "C" int psi_probe_lds_read_rate(void* stream, void* sink, int pattern, uint32_t iters) {
    if (sink == nullptr || iters == 0 || (pattern != 0 && pattern != 1)) return -1;
    hipLaunchKernelGGL(psi_lds_read_probe, dim3(256), dim3(512), 32 * kRowBytes, static_cast<hipStream_t>(stream),
                       pattern, iters, static_cast<float*>(sink));
    return static_cast<int>(hipGetLastError());
}
