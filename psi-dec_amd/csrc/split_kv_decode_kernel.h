// gfx950 split-KV grouped-query decode map for 2-byte K/V (bf16 / f16),
// head_dim 128 or 256, pages of 8 or 16*2^k tokens.
//
// Work decomposition
//   one workgroup (4 waves) = one (kv_split, kv_head); it serves all G query heads of that KV head.
//   One wave = every 4th 16-token tile of the split, with its own online-softmax state; the wave
//   states are merged through LDS once, at the end.  (1- and 2-wave workgroups measured no faster
//   at any grid size: they only add partial rows per byte read.)
//
// Per 16-token tile and wave
//   QK^T  one 16x16 MFMA tile: A = the K tile (16 tokens x head_dim, read straight from the page
//         with 128-bit loads, lane = (token lane%16, 8-dim chunk lane/16)), B = the query group
//         (G rows, zero-padded to 16) held in registers for the whole split.  The contraction runs
//         over head_dim, which is the contiguous axis of a K line, so no transpose is needed.
//   softmax  the MFMA result leaves each lane with 4 tokens of one query row; tile maximum by two
//         cross-row exchanges; probabilities go to LDS as P[token][head].
//   PV    vector ALU: lane = (token parity, 8 dims); each 128-bit load instruction covers 1 KiB of
//         contiguous V lines; acc[G][8] stays in registers for the whole split.  (PV contracts
//         over tokens, the strided axis of V, so it stays on the vector ALU with P broadcast
//         from LDS.)
//   Loads are software-pipelined one tile ahead: every K / V register is re-requested for the
//   next tile right after its last use in the current one.
//
// Algorithmic bytes per (kv token, kv head): 2 * head_dim * 2 (one K and one V line), read once.
#pragma once
#include <type_traits>

#include "split_kv.h"

namespace psi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

// D(16x16, f32) += A(16x32) * B(32x16).  Lane l holds A[row l%16][k 8*(l/16)..+8],
// B[k 8*(l/16)..+8][col l%16] and D[row 4*(l/16)+r][col l%16], r = 0..3.
template <typename Tag>
__device__ __forceinline__ f32x4_t mfma_16x16x32(uint4 a, uint4 b, f32x4_t c);
template <>
__device__ __forceinline__ f32x4_t mfma_16x16x32<BF16Tag>(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c,
                                                   0, 0, 0);
}
template <>
__device__ __forceinline__ f32x4_t mfma_16x16x32<F16Tag>(uint4 a, uint4 b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c,
                                                  0, 0, 0);
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

// Orders this wave's LDS traffic: earlier LDS operations have completed and the compiler keeps
// later ones after this point.  A wave's LDS operations execute in issue order.
// Maximum over the four lanes l % 16 == const of a wave, in every one of them, on the vector ALU: the two swaps
// exchange the odd 16-lane (32-lane) rows of one operand with the even rows of the other.
__device__ __forceinline__ float quarter_wave_max(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const uint32_t m = __float_as_uint(fmaxf(__uint_as_float(h[0]), __uint_as_float(h[1])));
    const auto q = __builtin_amdgcn_permlane16_swap(m, m, false, false);
    return fmaxf(__uint_as_float(q[0]), __uint_as_float(q[1]));
}

// The same for a sum: x + (the lane 32 on), and x + (the lanes 16, 32, 48 on).
__device__ __forceinline__ float half_wave_sum(float x) {
    const uint32_t u = __float_as_uint(x);
    const auto h = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(h[0]) + __uint_as_float(h[1]);
}
__device__ __forceinline__ float quarter_wave_sum(float x) {
    const uint32_t m = __float_as_uint(half_wave_sum(x));
    const auto q = __builtin_amdgcn_permlane16_swap(m, m, false, false);
    return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}

__device__ __forceinline__ void wave_lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

#ifndef PSI_DECODE_WAVES_PER_SIMD
#define PSI_DECODE_WAVES_PER_SIMD 3
#endif

// Workgroups per SIMD the register allocator is held to.  Three (168 registers) fits up to five query heads per
// KV head; six to eight need 172 to 198 registers and would spill, and a kernel with a private segment starts far
// slower than one resident wave less costs (two and three workgroups per SIMD stream equally fast), so those
// are held to two.
constexpr int decode_waves_per_simd(int group) { return group > 5 ? 2 : PSI_DECODE_WAVES_PER_SIMD; }

constexpr int kTileTokens = 16;

// Page IDs behind one 16-token tile: one page when a page holds at least 16 tokens, two when it
// holds 8 (tokens 0..7 of the tile in `a`, 8..15 in `b`).
struct TilePages {
    uint32_t a, b;
};

template <typename Tag, int D, int G, int kWaves, bool kHalfPage>
__global__ __launch_bounds__(64 * kWaves, decode_waves_per_simd(G)) void split_kv_decode_map(
    MapArgs a, const uint32_t* __restrict__ page_ids, const uint32_t* __restrict__ kv_splits,
    const uint32_t* __restrict__ req_slots, const uint16_t* __restrict__ q, const uint16_t* __restrict__ pages,
    const uint32_t* __restrict__ worker_cu) {
    resolve_active(a);
    constexpr int kVLanesPerToken = D / 8;                  // 32 (D=256) or 16 (D=128)
    constexpr int kVTokensPerLoad = 64 / kVLanesPerToken;   // 2 or 4
    constexpr int kVLoads = kTileTokens / kVTokensPerLoad;  // 8 or 4
    constexpr int kKSteps = D / 32;                         // 8 or 4 MFMA k-steps
    constexpr int kPStride = 8;                             // floats per token row of P in LDS

    // Workgroups go to the eight XCDs in turn (blockIdx % 8).  With an even number of KV heads, neighbouring heads
    // change places, so that an even XCD serves odd heads and the other way round: measured, not explained - the
    // workgroups of even heads on even XCDs ended 4 us later than the rest in a 93 us launch, and with the
    // exchange the map takes 1 % less on every decode configuration (C2 92.5 -> 91.6 us, C5 1267 -> 1252 us).
    const uint32_t kv_head = (blockIdx.x % a.walk.hkv) ^ ((a.walk.hkv & 1) ? 0u : 1u);
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    __shared__ __attribute__((aligned(16))) float p_lds[kWaves][kTileTokens * kPStride];
    __shared__ __attribute__((aligned(16))) float alpha_lds[kWaves][8];
    __shared__ __attribute__((aligned(16))) float merge_acc[kWaves][G * D];
    __shared__ float merge_max[kWaves][G];
    __shared__ float merge_sum[kWaves][G];
    __shared__ __attribute__((aligned(16))) uint4 qb_lds[D / 32][64];

    // MFMA lane coordinates: row of A (token) and column of B / D (query row); 8-dim chunk of A
    // and B, token quad of D.
    const uint32_t mt = lane & 15, mc = lane >> 4;
    // V lane coordinates.
    const uint32_t vsub = lane / kVLanesPerToken, vdl = lane % kVLanesPerToken;

    // Rows of kv_splits this workgroup serves: one row (blockIdx / Hkv) in the plain launch, or the
    // worker's row range when a balanced plan hands each workgroup an equal share of tiles.
    uint32_t row_begin = blockIdx.x / a.walk.hkv, row_end = row_begin + 1;
    if (worker_cu != nullptr) {
        row_begin = worker_cu[blockIdx.x / a.walk.hkv];
        row_end = worker_cu[blockIdx.x / a.walk.hkv + 1];
    }
    for (uint32_t split = row_begin; split < row_end; ++split) {
    if (split >= a.num_active_kv_splits) break;
    const uint32_t q_token = kv_splits[split * 3];
    if (q_token >= a.num_active_tokens) continue;  // sentinel padding or a slot owned by another producer
    const uint32_t kv_begin = kv_splits[split * 3 + 1];
    const uint32_t kv_end = kv_splits[split * 3 + 2];
    const uint32_t req_slot = req_slots[q_token];

    // Query group as the MFMA B operand, unscaled, in its native 2-byte type; rows >= G are zero.
    // Staged once per row in LDS in operand order [k-step][lane] and re-read per tile, which
    // costs 8 conflict-free LDS reads per tile and frees 32 registers per lane.
    if (wave == 0) {
        const uint16_t* q_row =
            q + ((uint64_t)q_token * a.hq + (uint64_t)kv_head * G + (mt < (uint32_t)G ? mt : 0)) * D + mc * 8;
#pragma unroll
        for (int i = 0; i < kKSteps; ++i) {
            const uint4 v = *reinterpret_cast<const uint4*>(q_row + i * 32);
            qb_lds[i][lane] = mt < (uint32_t)G ? v : make_uint4(0, 0, 0, 0);
        }
    }
    __syncthreads();

    const uint32_t log2p = 31 - __builtin_clz(a.walk.tokens_per_page);
    const uint32_t page_mask = a.walk.tokens_per_page - 1;
    const uint32_t* table_row = page_ids + ((uint64_t)req_slot * a.walk.num_layers + a.layer) *
                                                      a.walk.num_blocks * a.walk.ids_per_block;
    const uint64_t v_region = (uint64_t)a.walk.hkv * a.walk.tokens_per_page * D;

    // Append folded into the map (a.flat_k set): positions [new_begin, own] of this request are this step's
    // new tokens.  They are read from the flat rows after the paged tiles, never from the page, which another
    // workgroup may be writing right now; the paged part of the row ends at page_end.
    uint32_t page_end = kv_end, new_begin = kv_end;
    if (a.flat_k != nullptr) {
        const uint32_t own = a.flat_token_indices[q_token];  // this token's position
        if (kv_end + q_token > own) {  // the row can reach a token of this step (at most q_token of them precede)
            uint32_t before = 0;
            while (before < q_token && req_slots[q_token - before - 1] == req_slot &&
                   a.flat_token_indices[q_token - before - 1] + before + 1 == own)
                ++before;
            new_begin = max(own - before, kv_begin);
            page_end = min(kv_end, new_begin);
        }
        if (kv_end == own + 1 && wave == 0) {
            // this workgroup owns the token's append for its KV head: one 16-byte chunk per lane, K line then V line
            const uint32_t page_id = table_row[own >> log2p];
            constexpr uint32_t kChunks = D / 8;
            const uint16_t* flat_k = reinterpret_cast<const uint16_t*>(a.flat_k);
            const uint16_t* flat_v = reinterpret_cast<const uint16_t*>(a.flat_v);
            for (uint32_t c = lane; c < 2 * kChunks; c += 64) {
                const uint32_t kind = c / kChunks, chunk = c % kChunks;
                // a choice of two pointers, not an index into an array of them: the load stays a global one
                const uint16_t* src = (kind ? flat_v : flat_k) + ((uint64_t)q_token * a.walk.hkv + kv_head) * D + chunk * 8;
                uint16_t* dst = const_cast<uint16_t*>(pages) + (uint64_t)page_id * a.walk.page_elems + kind * v_region +
                                ((uint64_t)kv_head * a.walk.tokens_per_page + (own & page_mask)) * D + chunk * 8;
                *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(src);
            }
        }
    }

    const uint32_t tile_begin = kv_begin / kTileTokens;
    const uint32_t tile_end = page_end > kv_begin ? (page_end + kTileTokens - 1) / kTileTokens : tile_begin;

    float run_max = -INFINITY, lane_sum = 0.0f;  // of query row mt, over this lane's tokens
    float acc[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = 0.0f;

    const uint32_t last_page = (max(page_end, 1u) - 1) >> log2p;
    auto load_page_id = [&](uint32_t tile) -> TilePages {
        TilePages p{0u, 0u};
        if (tile < tile_end) {
            const uint32_t first = (tile * kTileTokens) >> log2p;
            p.a = table_row[first];
            if (kHalfPage) p.b = table_row[min(first + 1, last_page)];
        }
        return p;
    };
    // K line 0 of (page, kv_head); the V lines follow v_region elements later.
    auto head_base = [&](uint32_t page_id) -> const uint16_t* {
        return pages + (uint64_t)page_id * a.walk.page_elems + (uint64_t)kv_head * a.walk.tokens_per_page * D;
    };

    // One K and one V register buffer per wave.  A buffer entry is re-requested for the next tile
    // as soon as its last use in the current tile has issued, so each load has about a whole tile
    // period to land while the wave keeps only 16 KiB of tile data in registers.
    uint4 kreg[kKSteps];  // lane (t = lane%16, c = lane/16): step i = dims [i*32 + c*8, +8) of token t
    uint4 vreg[kVLoads];  // lane (sub, dl): load j = token j*kVTokensPerLoad + sub, dims [dl*8, +8)
    auto issue_k = [&](uint32_t tile, TilePages p) {
        const uint16_t* k_lane;
        if (kHalfPage)
            k_lane = head_base(mt < 8 ? p.a : p.b) + (mt & 7) * D + mc * 8;
        else
            k_lane = head_base(p.a) + (((tile * kTileTokens) & page_mask) + mt) * D + mc * 8;
#pragma unroll
        for (int i = 0; i < kKSteps; ++i) kreg[i] = stream_load_b128(k_lane + i * 32);
    };
    auto issue_v = [&](uint32_t tile, TilePages p) {
#pragma unroll
        for (int j = 0; j < kVLoads; ++j) {
            const uint16_t* v_lane;
            if (kHalfPage)  // load j covers tokens j*kVTokensPerLoad .. +kVTokensPerLoad-1: one half of the tile
                v_lane = head_base(j * kVTokensPerLoad < 8 ? p.a : p.b) + v_region +
                         ((j * kVTokensPerLoad + vsub) & 7) * D + vdl * 8;
            else
                v_lane = head_base(p.a) + v_region +
                         (((tile * kTileTokens) & page_mask) + j * kVTokensPerLoad + vsub) * D + vdl * 8;
            vreg[j] = stream_load_b128(v_lane);
        }
    };

    float* my_p = p_lds[wave];
    float* my_alpha = alpha_lds[wave];

    // One 16-token tile.  `partial`: the tile holds tokens outside [kv_begin, kv_end).
    // `has_next`: another tile of this wave follows; its K and V are requested on the way, each
    // into the registers the current tile has just finished with.  Both flags are wave-uniform.
    // `base`: position of the tile's first token; positions outside [lo, hi) are masked.
    auto process_tile = [&](uint32_t base, uint32_t lo, uint32_t hi, bool partial, auto has_next_tag, uint32_t next,
                            TilePages next_pid) __attribute__((always_inline)) {
        // compile-time flag: the steady-state copy issues its refill loads unconditionally, which
        // keeps the hardware load counter's order exact for the waits that follow
        constexpr bool has_next = decltype(has_next_tag)::value;
        // ---- logits of query rows x 16 tokens on the matrix cores
        f32x4_t s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < kKSteps; i += 2) {
            s0 = mfma_16x16x32<Tag>(kreg[i], qb_lds[i][lane], s0);
            s1 = mfma_16x16x32<Tag>(kreg[i + 1], qb_lds[i + 1][lane], s1);
        }
        __builtin_amdgcn_sched_barrier(0);
        if (has_next) issue_k(next, next_pid);
        __builtin_amdgcn_sched_barrier(0);
        // ---- online softmax of query row mt over this lane's tokens 4*mc + r
        float v[4];
        float m = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t token = base + mc * 4 + r;
            const bool valid = token >= lo && token < hi;
            v[r] = valid ? (s0[r] + s1[r]) * a.scale_log2 : -INFINITY;
            m = fmaxf(m, v[r]);
        }
        m = quarter_wave_max(m);
        const float next_max = fmaxf(run_max, m);
        const float alpha = __builtin_amdgcn_exp2f(run_max - next_max);  // 0 on the first tile
        const bool rescale = __any(mt < (uint32_t)G && next_max != run_max);
        run_max = next_max;
        float p[4], tile_sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            p[r] = __builtin_amdgcn_exp2f(v[r] - next_max);
            tile_sum += p[r];
        }
        lane_sum = lane_sum * alpha + tile_sum;
        wave_lds_fence();  // the previous tile's P reads are complete
        if (mt < 8) {
#pragma unroll
            for (int r = 0; r < 4; ++r) my_p[(mc * 4 + r) * kPStride + mt] = p[r];
            if (mc == 0) my_alpha[mt] = alpha;
        }
        wave_lds_fence();

        // ---- acc[h][e] += P[token][h] * V[token][dl*8 + e] on the vector ALU
        if (rescale) {
            float al[8];
            const float4 a0 = *reinterpret_cast<const float4*>(&my_alpha[0]);
            al[0] = a0.x; al[1] = a0.y; al[2] = a0.z; al[3] = a0.w;
            if (G > 4) {
                const float4 a1 = *reinterpret_cast<const float4*>(&my_alpha[4]);
                al[4] = a1.x; al[5] = a1.y; al[6] = a1.z; al[7] = a1.w;
            }
#pragma unroll
            for (int h = 0; h < G; ++h)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] *= al[h];
        }
        if (partial) {
            // tokens outside the split carry probability 0, but their V bytes may be NaN/Inf
#pragma unroll
            for (int j = 0; j < kVLoads; ++j) {
                const uint32_t vtoken = base + j * kVTokensPerLoad + vsub;
                if (vtoken < lo || vtoken >= hi) vreg[j] = make_uint4(0, 0, 0, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kVLoads; ++j) {
            const uint32_t tok_in_tile = j * kVTokensPerLoad + vsub;
            float pr[8];
            {
                const float4 p0 = *reinterpret_cast<const float4*>(&my_p[tok_in_tile * kPStride]);
                pr[0] = p0.x; pr[1] = p0.y; pr[2] = p0.z; pr[3] = p0.w;
                if (G > 4) {
                    const float4 p1 = *reinterpret_cast<const float4*>(&my_p[tok_in_tile * kPStride + 4]);
                    pr[4] = p1.x; pr[5] = p1.y; pr[6] = p1.z; pr[7] = p1.w;
                }
            }
            float vf[8];
            unpack2<Tag>(vreg[j].x, vf[0], vf[1]);
            unpack2<Tag>(vreg[j].y, vf[2], vf[3]);
            unpack2<Tag>(vreg[j].z, vf[4], vf[5]);
            unpack2<Tag>(vreg[j].w, vf[6], vf[7]);
#pragma unroll
            for (int h = 0; h < G; ++h)
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(pr[h], vf[e], acc[h][e]);
            // keeps later P reads and V unpacks from being hoisted above this point (register budget)
            __builtin_amdgcn_sched_barrier(0);
        }
        if (has_next) issue_v(next, next_pid);
        __builtin_amdgcn_sched_barrier(0);
    };

    uint32_t tile = tile_begin + wave;
    if (tile < tile_end) {
        {
            const TilePages pid = load_page_id(tile);
            issue_k(tile, pid);
            issue_v(tile, pid);
        }
        TilePages pid_next = load_page_id(tile + kWaves);
        auto is_partial = [&](uint32_t t) { return t * kTileTokens < kv_begin || (t + 1) * kTileTokens > page_end; };
        while (tile + kWaves < tile_end) {
            const uint32_t next = tile + kWaves;
            const TilePages pid_after = load_page_id(next + kWaves);
            process_tile(tile * kTileTokens, kv_begin, page_end, is_partial(tile), std::true_type(), next, pid_next);
            pid_next = pid_after;
            tile = next;
        }
        // the wave's last tile
        process_tile(tile * kTileTokens, kv_begin, page_end, is_partial(tile), std::false_type(), 0u, TilePages{0u, 0u});
    }
    if (new_begin < kv_end && wave == kWaves - 1) {
        // this step's tokens inside the row, sixteen at a time from the flat rows (one, in a decode batch)
        const uint16_t* flat_k = reinterpret_cast<const uint16_t*>(a.flat_k);
        const uint16_t* flat_v = reinterpret_cast<const uint16_t*>(a.flat_v);
        const uint32_t new_end = min(kv_end, a.flat_token_indices[q_token] + 1);
        const int64_t row0 = (int64_t)q_token - a.flat_token_indices[q_token];  // flat row of position p = row0 + p
        for (uint32_t base = new_begin; base < new_end; base += kTileTokens) {
            const uint32_t k_pos = min(base + mt, new_end - 1);
            const uint16_t* k_lane = flat_k + ((uint64_t)(row0 + k_pos) * a.walk.hkv + kv_head) * D + mc * 8;
#pragma unroll
            for (int i = 0; i < kKSteps; ++i) kreg[i] = *reinterpret_cast<const uint4*>(k_lane + i * 32);
#pragma unroll
            for (int j = 0; j < kVLoads; ++j) {
                const uint32_t v_pos = min(base + j * kVTokensPerLoad + vsub, new_end - 1);
                vreg[j] = *reinterpret_cast<const uint4*>(flat_v + ((uint64_t)(row0 + v_pos) * a.walk.hkv + kv_head) * D +
                                                          vdl * 8);
            }
            process_tile(base, base, new_end, true, std::false_type(), 0u, TilePages{0u, 0u});
        }
    }

    // ---- wave epilogue: fold the V token sub-lanes together, reduce the per-lane sums.
#pragma unroll
    for (int h = 0; h < G; ++h)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            acc[h][e] = kVTokensPerLoad == 4 ? quarter_wave_sum(acc[h][e]) : half_wave_sum(acc[h][e]);
        }
    lane_sum = quarter_wave_sum(lane_sum);
    if (lane < (uint32_t)kVLanesPerToken) {
#pragma unroll
        for (int h = 0; h < G; ++h) {
            float4* dst = reinterpret_cast<float4*>(&merge_acc[wave][h * D + lane * 8]);
            dst[0] = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            dst[1] = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
    }
    if (lane < (uint32_t)G) {  // mc == 0, mt = lane: one lane per query row
        merge_max[wave][lane] = run_max;
        merge_sum[wave][lane] = lane_sum;
    }
    __syncthreads();

    // ---- merge the wave states and emit the partial of (split, q_head): each thread owns 4
    // consecutive dims of one head, so a wave stores 1 KiB of contiguous f32 per instruction.
    for (uint32_t idx = tid * 4; idx < (uint32_t)(G * D); idx += 64 * kWaves * 4) {
        const uint32_t h = idx / D, dim = idx % D;
        float m = merge_max[0][h];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) m = fmaxf(m, merge_max[w][h]);
        float4 out = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const float mw = merge_max[w][h];
            const float f = mw > -INFINITY ? __builtin_amdgcn_exp2f(mw - m) : 0.0f;
            const float4 part = *reinterpret_cast<const float4*>(&merge_acc[w][idx]);
            out.x = fmaf(f, part.x, out.x);
            out.y = fmaf(f, part.y, out.y);
            out.z = fmaf(f, part.z, out.z);
            out.w = fmaf(f, part.w, out.w);
            sum = fmaf(f, merge_sum[w][h], sum);
        }
        const uint64_t row = (uint64_t)split * a.hq + (uint64_t)kv_head * G + h;
        *reinterpret_cast<float4*>(&a.part_acc[row * D + dim]) = out;
        if (dim == 0) {
            a.part_max[row] = m;
            a.part_sum[row] = sum;
        }
    }
    if (split + 1 < row_end) __syncthreads();  // the LDS staging areas are reused by the next row
    }  // rows of this workgroup
}


template <typename Tag, int D, int G>
inline void launch_decode_map_w(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    const dim3 grid((a.worker_cu ? a.num_workers : a.num_total_kv_splits) * g.hkv);
    const uint16_t* q = reinterpret_cast<const uint16_t*>(a.q);
    const uint16_t* pages = reinterpret_cast<const uint16_t*>(a.kv_pages);
    if (g.tokens_per_page == 8)  // a tile spans two pages
        hipLaunchKernelGGL((split_kv_decode_map<Tag, D, G, 4, true>), grid, dim3(256), 0, ctx->stream, a,
                           a.walk.page_ids, a.kv_splits, a.req_slots, q, pages, a.worker_cu);
    else
        hipLaunchKernelGGL((split_kv_decode_map<Tag, D, G, 4, false>), grid, dim3(256), 0, ctx->stream, a,
                           a.walk.page_ids, a.kv_splits, a.req_slots, q, pages, a.worker_cu);
}

// One translation unit per (element type, head_dim) instantiates every group size 1..8.
template <typename Tag, int D>
inline int launch_decode_map_group(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    switch (g.group) {
#define PSI_CASE(G)                                        \
    case G:                                                \
        launch_decode_map_w<Tag, D, G>(ctx, g, a);         \
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

}  // namespace psi
