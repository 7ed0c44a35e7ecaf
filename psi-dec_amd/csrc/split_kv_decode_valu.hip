// All-VALU variant of the gfx950 split-KV decode map (2-byte K/V, head_dim 128 or 256, pages of
// 16*k tokens): logits by packed dot2 on the vector ALU with the query group in LDS, no matrix
// cores.  Kept selectable (PSI_HIP_FLAG_DECODE_VALU_QK) as the comparison point for the default
// kernel, which moves the QK^T contraction to MFMA.
//
// Work decomposition
//   one workgroup (4 waves) = one (kv_split, kv_head); it serves all G query heads of that KV head
//   one wave = every 4th 16-token tile of the split, with its own online-softmax state; the four
//   wave states are merged through LDS once, at the end.
//
// Per 16-token tile and wave
//   K   lane = (token t = lane/4, dim quarter c = lane%4); D/32 128-bit loads per lane, each
//       instruction covering 64 contiguous bytes of 16 token lines.  Logits = packed dot2 against
//       the query group staged in LDS (unscaled, native type), reduced over the quad with DPP.
//   softmax  every lane of a quad holds its token's G logits; tile maximum over tokens by DPP row
//       rotates + two cross-row exchanges; probabilities go to LDS as P[token][head].
//   V   lane = (token parity, 8 dims); each 128-bit load instruction covers 1 KiB of contiguous V
//       lines; the output accumulators acc[G][8] stay in registers for the whole split.
//
// Algorithmic bytes per (kv token, kv head): 2 * head_dim * 2 (one K and one V line), read once.
#include "split_kv.h"

namespace psi {
namespace valu {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

template <typename Tag>
__device__ __forceinline__ float dot2_acc(uint32_t a, uint32_t b, float acc);
template <>
__device__ __forceinline__ float dot2_acc<BF16Tag>(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), acc, false);
}
template <>
__device__ __forceinline__ float dot2_acc<F16Tag>(uint32_t a, uint32_t b, float acc) {
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), acc, false);
}

template <typename Tag>
__device__ __forceinline__ void unpack2(uint32_t packed, float& lo, float& hi);
template <>
__device__ __forceinline__ void unpack2<BF16Tag>(uint32_t packed, float& lo, float& hi) {
    lo = __uint_as_float(packed << 16);
    hi = __uint_as_float(packed & 0xffff0000u);
}
template <>
__device__ __forceinline__ void unpack2<F16Tag>(uint32_t packed, float& lo, float& hi) {
    const f16x2_t h = __builtin_bit_cast(f16x2_t, packed);
    lo = (float)h.x;
    hi = (float)h.y;
}

__device__ __forceinline__ float dpp_quad_xor1(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_row_ror4(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_row_ror8(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, true));
}

// Orders this wave's LDS traffic: earlier LDS writes have landed and the compiler keeps later
// reads after this point.  A wave's LDS operations execute in issue order.
__device__ __forceinline__ void wave_lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

constexpr int kTileTokens = 16;
constexpr int kWaves = 4;

template <int D>
struct TileRegs {
    uint4 k[D / 32];               // lane (t, c): chunk i = dims [i*32 + c*8, +8) of token t
    uint4 v[kTileTokens * D / 512];  // lane (sub, dl): load j = token j*(512/D) + sub, dims [dl*8, +8)
};

template <typename Tag, int D, int G>
__global__ __launch_bounds__(256, 2) void split_kv_decode_map_valu(MapArgs a) {
    resolve_active(a);
    constexpr int kVLanesPerToken = D / 8;                  // 32 (D=256) or 16 (D=128)
    constexpr int kVTokensPerLoad = 64 / kVLanesPerToken;   // 2 or 4
    constexpr int kVLoads = kTileTokens / kVTokensPerLoad;  // 8 or 4
    constexpr int kKLoads = D / 32;                         // 8 or 4
    constexpr int kPStride = 8;                             // floats per token row of P in LDS

    const uint32_t kv_head = blockIdx.x % a.walk.hkv;
    const uint32_t split = blockIdx.x / a.walk.hkv;
    if (split >= a.num_active_kv_splits) return;
    const uint32_t q_token = a.kv_splits[split * 3];
    if (q_token >= a.num_active_tokens) return;  // sentinel padding or a slot owned by another producer
    const uint32_t kv_begin = a.kv_splits[split * 3 + 1];
    const uint32_t kv_end = a.kv_splits[split * 3 + 2];
    const uint32_t req_slot = a.req_slots[q_token];

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    __shared__ __attribute__((aligned(16))) uint16_t q_lds[G * D];
    __shared__ __attribute__((aligned(16))) float p_lds[kWaves][kTileTokens * kPStride];
    __shared__ __attribute__((aligned(16))) float merge_acc[kWaves][G * D];
    __shared__ float merge_max[kWaves][G];
    __shared__ float merge_sum[kWaves][G];

    // Stage the query group [G][D] of this KV head, unscaled, in its native 2-byte type.
    {
        const uint4* q_src = reinterpret_cast<const uint4*>(
            reinterpret_cast<const uint16_t*>(a.q) + ((uint64_t)q_token * a.hq + (uint64_t)kv_head * G) * D);
        for (uint32_t i = tid; i < (uint32_t)(G * D / 8); i += 256) reinterpret_cast<uint4*>(q_lds)[i] = q_src[i];
    }
    __syncthreads();

    const uint32_t log2p = 31 - __builtin_clz(a.walk.tokens_per_page);
    const uint32_t page_mask = a.walk.tokens_per_page - 1;
    const uint32_t* table_row = a.walk.page_ids + ((uint64_t)req_slot * a.walk.num_layers + a.layer) *
                                                      a.walk.num_blocks * a.walk.ids_per_block;
    const uint16_t* pages = reinterpret_cast<const uint16_t*>(a.kv_pages);
    const uint64_t v_region = (uint64_t)a.walk.hkv * a.walk.tokens_per_page * D;

    const uint32_t tile_begin = kv_begin / kTileTokens;
    const uint32_t tile_end = (kv_end + kTileTokens - 1) / kTileTokens;

    // K lane coordinates and V lane coordinates.
    const uint32_t kt = lane >> 2, kc = lane & 3;
    const uint32_t vsub = lane / kVLanesPerToken, vdl = lane % kVLanesPerToken;

    float run_max[G], lane_sum[G], acc[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
        run_max[h] = -INFINITY;
        lane_sum[h] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = 0.0f;
    }

    auto load_page_id = [&](uint32_t tile) -> uint32_t {
        return tile < tile_end ? table_row[(tile * kTileTokens) >> log2p] : 0u;
    };
    auto issue_loads = [&](uint32_t tile, uint32_t page_id, TileRegs<D>& r) {
        const uint32_t in_page = (tile * kTileTokens) & page_mask;
        const uint16_t* k_base =
            pages + (uint64_t)page_id * a.walk.page_elems + ((uint64_t)kv_head * a.walk.tokens_per_page + in_page) * D;
        const uint16_t* v_base = k_base + v_region;
        const uint16_t* k_lane = k_base + kt * D + kc * 8;
#pragma unroll
        for (int i = 0; i < kKLoads; ++i) r.k[i] = stream_load_b128(k_lane + i * 32);
        const uint16_t* v_lane = v_base + vsub * D + vdl * 8;
#pragma unroll
        for (int j = 0; j < kVLoads; ++j) r.v[j] = stream_load_b128(v_lane + j * kVTokensPerLoad * D);
    };

    uint32_t tile = tile_begin + wave;
    TileRegs<D> cur;
    uint32_t pid_next = 0;
    if (tile < tile_end) {
        issue_loads(tile, load_page_id(tile), cur);
        pid_next = load_page_id(tile + kWaves);
    }

    float* my_p = p_lds[wave];

    while (tile < tile_end) {
        const uint32_t next_tile = tile + kWaves;
        const bool has_next = next_tile < tile_end;
        const uint32_t pid_after = load_page_id(next_tile + kWaves);
        TileRegs<D> nxt;
        if (has_next) issue_loads(next_tile, pid_next, nxt);

        // ---- logits: s[h] = q_h . k_t over this lane's dim quarter, then quad reduction.
        float s[G];
#pragma unroll
        for (int h = 0; h < G; ++h) s[h] = 0.0f;
#pragma unroll
        for (int i = 0; i < kKLoads; ++i) {
            const uint4 kk = cur.k[i];
#pragma unroll
            for (int h = 0; h < G; ++h) {
                const uint4 qq = *reinterpret_cast<const uint4*>(&q_lds[h * D + i * 32 + kc * 8]);
                s[h] = dot2_acc<Tag>(kk.x, qq.x, s[h]);
                s[h] = dot2_acc<Tag>(kk.y, qq.y, s[h]);
                s[h] = dot2_acc<Tag>(kk.z, qq.z, s[h]);
                s[h] = dot2_acc<Tag>(kk.w, qq.w, s[h]);
            }
        }
        const uint32_t token = tile * kTileTokens + kt;
        const bool token_valid = token >= kv_begin && token < kv_end;
        const bool partial_tile = tile * kTileTokens < kv_begin || (tile + 1) * kTileTokens > kv_end;
        float alpha[G], p[G];
        bool rescale = false;
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float v = s[h];
            v += dpp_quad_xor1(v);
            v += dpp_quad_xor2(v);
            v = token_valid ? v * a.scale_log2 : -INFINITY;
            // tile maximum over the 16 tokens: within a row of 16 lanes, then across the 4 rows
            float m = fmaxf(v, dpp_row_ror4(v));
            m = fmaxf(m, dpp_row_ror8(m));
            m = fmaxf(m, __shfl_xor(m, 16, 64));
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            const float next_max = fmaxf(run_max[h], m);
            alpha[h] = __builtin_amdgcn_exp2f(run_max[h] - next_max);  // 0 on the first tile (run_max = -inf)
            rescale |= next_max != run_max[h];
            run_max[h] = next_max;
            p[h] = __builtin_amdgcn_exp2f(v - next_max);
            lane_sum[h] = lane_sum[h] * alpha[h] + p[h];
        }
        // ---- probabilities to LDS as P[token][head]; quad lane c writes heads 2c and 2c+1.
        wave_lds_fence();  // previous tile's P reads are complete
        {
            float lo = 0.0f, hi = 0.0f;
#pragma unroll
            for (int h = 0; h < G; ++h) {
                if ((uint32_t)(h >> 1) == kc) {
                    if (h & 1) hi = p[h];
                    else lo = p[h];
                }
            }
            if (kc * 2 < (uint32_t)G) *reinterpret_cast<float2*>(&my_p[kt * kPStride + kc * 2]) = make_float2(lo, hi);
        }
        wave_lds_fence();

        if (__builtin_amdgcn_readfirstlane((int)rescale)) {  // run_max is wave-uniform, so is `rescale`
#pragma unroll
            for (int h = 0; h < G; ++h)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] *= alpha[h];
        }

        // ---- acc[h][e] += P[token][h] * V[token][dl*8 + e]
#pragma unroll
        for (int j = 0; j < kVLoads; ++j) {
            const uint32_t tok_in_tile = j * kVTokensPerLoad + vsub;
            uint4 vv = cur.v[j];
            if (partial_tile) {
                const uint32_t vtoken = tile * kTileTokens + tok_in_tile;
                if (vtoken < kv_begin || vtoken >= kv_end) vv = make_uint4(0, 0, 0, 0);
            }
            float pv[8];
            {
                const float4 p0 = *reinterpret_cast<const float4*>(&my_p[tok_in_tile * kPStride]);
                pv[0] = p0.x; pv[1] = p0.y; pv[2] = p0.z; pv[3] = p0.w;
                if (G > 4) {
                    const float4 p1 = *reinterpret_cast<const float4*>(&my_p[tok_in_tile * kPStride + 4]);
                    pv[4] = p1.x; pv[5] = p1.y; pv[6] = p1.z; pv[7] = p1.w;
                }
            }
            float vf[8];
            unpack2<Tag>(vv.x, vf[0], vf[1]);
            unpack2<Tag>(vv.y, vf[2], vf[3]);
            unpack2<Tag>(vv.z, vf[4], vf[5]);
            unpack2<Tag>(vv.w, vf[6], vf[7]);
#pragma unroll
            for (int h = 0; h < G; ++h)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(pv[h], vf[e], acc[h][e]);
        }

        if (!has_next) break;
        cur = nxt;
        pid_next = pid_after;
        tile = next_tile;
    }

    // ---- wave epilogue: fold the V token sub-lanes together, reduce the per-lane sums.
#pragma unroll
    for (int h = 0; h < G; ++h) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float v = acc[h][e];
            v += __shfl_xor(v, 32, 64);
            if (kVTokensPerLoad == 4) v += __shfl_xor(v, 16, 64);
            acc[h][e] = v;
        }
        float l = lane_sum[h];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) l += __shfl_xor(l, off, 64);
        lane_sum[h] = l * 0.25f;  // every token's probability was held by the 4 lanes of its quad
    }
    if (lane < (uint32_t)kVLanesPerToken) {
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float4* dst = reinterpret_cast<float4*>(&merge_acc[wave][h * D + lane * 8]);
            dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int h = 0; h < G; ++h) {
            merge_max[wave][h] = run_max[h];
            merge_sum[wave][h] = lane_sum[h];
        }
    }
    __syncthreads();

    // ---- merge the four wave states and emit the partial of (split, q_head).
    for (uint32_t idx = tid; idx < (uint32_t)(G * D); idx += 256) {
        const uint32_t h = idx / D, dim = idx % D;
        float m = merge_max[0][h];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) m = fmaxf(m, merge_max[w][h]);
        float out = 0.0f, sum = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float mw = merge_max[w][h];
            const float f = mw > -INFINITY ? exp2f(mw - m) : 0.0f;
            out = fmaf(f, merge_acc[w][idx], out);
            sum = fmaf(f, merge_sum[w][h], sum);
        }
        const uint64_t row = (uint64_t)split * a.hq + (uint64_t)kv_head * G + h;
        a.part_acc[row * D + dim] = out;
        if (dim == 0) {
            a.part_max[row] = m;
            a.part_sum[row] = sum;
        }
    }
}

}  // namespace valu
using namespace valu;

template <typename Tag, int D>
static int launch_map_valu_g(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    const dim3 grid(a.num_total_kv_splits * g.hkv), block(256);
    switch (g.group) {
#define PSI_CASE(G)                                                                              \
    case G:                                                                                      \
        hipLaunchKernelGGL((split_kv_decode_map_valu<Tag, D, G>), grid, block, 0, ctx->stream, a);     \
        return PSI_HIP_OK;
        PSI_CASE(1)
        PSI_CASE(2)
        PSI_CASE(3)
        PSI_CASE(4)
        PSI_CASE(5)
        PSI_CASE(6)
        PSI_CASE(7)
        PSI_CASE(8)
#undef PSI_CASE
        default:
            return PSI_HIP_ERR_UNSUPPORTED;
    }
}

int launch_decode_map_valu(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    const bool two_byte = g.dtype == PSI_HIP_BF16 || g.dtype == PSI_HIP_F16;
    const uint32_t p = g.tokens_per_page;
    const bool page_ok = p >= 16 && (p & (p - 1)) == 0;
    const bool aligned = reinterpret_cast<uintptr_t>(a.q) % 16 == 0 && reinterpret_cast<uintptr_t>(a.kv_pages) % 16 == 0;
    if (!two_byte || !page_ok || !aligned || g.group > 8 || (g.d != 256 && g.d != 128)) return PSI_HIP_ERR_UNSUPPORTED;
    if ((uint64_t)a.num_total_kv_splits * g.hkv > 0x7fffffffull) return PSI_HIP_ERR_UNSUPPORTED;
    if (g.dtype == PSI_HIP_BF16)
        return g.d == 256 ? launch_map_valu_g<BF16Tag, 256>(ctx, g, a) : launch_map_valu_g<BF16Tag, 128>(ctx, g, a);
    return g.d == 256 ? launch_map_valu_g<F16Tag, 256>(ctx, g, a) : launch_map_valu_g<F16Tag, 128>(ctx, g, a);
}

}  // namespace psi
