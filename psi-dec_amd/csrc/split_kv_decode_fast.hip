// Dispatch of the gfx950 split-KV decode map (instantiated per element type and head_dim in the
// split_kv_decode_*.hip files) and the gfx950 log-sum-exp combine kernel.
#include "split_kv.h"

namespace psi {

int launch_decode_map_bf16_d256(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);
int launch_decode_map_bf16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);
int launch_decode_map_f16_d256(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);
int launch_decode_map_f16_d128(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a);

// Log-sum-exp combine: one wave per (token, q_head), lanes over head_dim.  The accumulator rows are
// read four at a time so that a wave keeps several 1 KiB reads in flight instead of one; the overall
// maximum comes from the first four rows' own values and a lane-parallel pass over the rest.
template <typename Tag, int D, bool kIndexed>
__global__ __launch_bounds__(256) void split_kv_reduce_fast(ReduceArgs a) {
    resolve_active(a);
    constexpr int kPerLane = D / 64;  // 4 or 2
    constexpr int kUnroll = 4;
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t row_out = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row_out >= (uint64_t)a.num_active_tokens * a.hq) return;
    const uint32_t token = (uint32_t)(row_out / a.hq), q_head = (uint32_t)(row_out % a.hq);
    const uint32_t begin = a.cu_kv_splits[token], end = a.cu_kv_splits[token + 1];
    const uint32_t* row_index = a.row_index;
    auto row_of = [&](uint32_t p) -> uint64_t { return (uint64_t)(kIndexed ? row_index[p] : p) * a.hq + q_head; };
    // The first four rows are asked for before anything waits: their maxima (the same in every lane) enter the
    // overall maximum from registers, and the lane-parallel pass over the maxima covers the rows behind them only,
    // so that a short list - the usual case - costs one round trip to memory instead of two.
    float m[kUnroll], sums[kUnroll], part[kUnroll][kPerLane];
    auto fetch = [&](uint32_t p0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool live = p0 + u < end;
            const uint64_t row = row_of(live ? p0 + u : begin);
            m[u] = a.part_max[row];
            if (!live) m[u] = -INFINITY;
            sums[u] = a.part_sum[row];
            const float* src = a.part_acc + row * D + lane * kPerLane;
#pragma unroll
            for (int e = 0; e < kPerLane; ++e) part[u][e] = src[e];
        }
    };
    if (begin < end) fetch(begin);
    float global_max = -INFINITY;
    for (uint32_t p = begin + kUnroll + lane; p < end; p += 64) global_max = fmaxf(global_max, a.part_max[row_of(p)]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) global_max = fmaxf(global_max, __shfl_xor(global_max, off, 64));
    if (begin < end) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) global_max = fmaxf(global_max, m[u]);
    }
    float weight_sum = 0.0f, value[kPerLane];
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) value[e] = 0.0f;
    for (uint32_t p0 = begin; p0 < end; p0 += kUnroll) {
        if (p0 != begin) fetch(p0);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const float w = m[u] > -INFINITY ? exp2f(m[u] - global_max) : 0.0f;
            weight_sum = fmaf(w, sums[u], weight_sum);
#pragma unroll
            for (int e = 0; e < kPerLane; ++e) value[e] = fmaf(w, part[u][e], value[e]);
        }
    }
    const float inv = weight_sum > 0.0f ? 1.0f / weight_sum : 0.0f;
    const uint64_t out_index = row_out * D + lane * kPerLane;
#pragma unroll
    for (int e = 0; e < kPerLane; ++e)
        store_from_f32<Tag>(a.output, out_index + e, finish_output<Tag>(a, value[e] * inv, token, q_head, lane * kPerLane + e));
}

// The combine for long split lists (long contexts, few tokens): one workgroup of eight waves per
// (token, q_head); wave w takes the rows begin + w, begin + w + 8, ... four at a time, and the wave
// results, all relative to the same maximum, are added through LDS.
constexpr int kWideWaves = 8;
template <typename Tag, int D, bool kIndexed>
__global__ __launch_bounds__(64 * kWideWaves) void split_kv_reduce_wide(ReduceArgs a) {
    resolve_active(a);
    constexpr int kPerLane = D / 64;
    constexpr int kUnroll = 4;
    __shared__ float wave_max[kWideWaves];
    __shared__ float wave_sum[kWideWaves];
    __shared__ float wave_val[kWideWaves][D];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint64_t row_out = blockIdx.x;
    const uint32_t token = (uint32_t)(row_out / a.hq), q_head = (uint32_t)(row_out % a.hq);
    // The grid is cut for the by-value count; with device-side counts bound that is the bucket's capacity, and a
    // workgroup beyond the active tokens must touch nothing (its cu_kv_splits entries are stale).  Uniform over
    // the workgroup and ahead of the first barrier.
    if (token >= a.num_active_tokens) return;
    const uint32_t begin = a.cu_kv_splits[token], end = a.cu_kv_splits[token + 1];
    const uint32_t* row_index = a.row_index;
    float global_max = -INFINITY;
    for (uint32_t p = begin + threadIdx.x; p < end; p += 64 * kWideWaves)
        global_max = fmaxf(global_max, a.part_max[(uint64_t)(kIndexed ? row_index[p] : p) * a.hq + q_head]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) global_max = fmaxf(global_max, __shfl_xor(global_max, off, 64));
    if (lane == 0) wave_max[wave] = global_max;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kWideWaves; ++w) global_max = fmaxf(global_max, wave_max[w]);
    float weight_sum = 0.0f, value[kPerLane];
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) value[e] = 0.0f;
    for (uint32_t p0 = begin + wave; p0 < end; p0 += kWideWaves * kUnroll) {
        float w[kUnroll], sums[kUnroll], part[kUnroll][kPerLane];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool live = p0 + u * kWideWaves < end;
            const uint32_t p = live ? p0 + u * kWideWaves : begin;
            const uint64_t row = (uint64_t)(kIndexed ? row_index[p] : p) * a.hq + q_head;
            const float m = a.part_max[row];
            sums[u] = a.part_sum[row];
            w[u] = live && m > -INFINITY ? exp2f(m - global_max) : 0.0f;
            const float* src = a.part_acc + row * D + lane * kPerLane;
#pragma unroll
            for (int e = 0; e < kPerLane; ++e) part[u][e] = src[e];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            weight_sum = fmaf(w[u], sums[u], weight_sum);
#pragma unroll
            for (int e = 0; e < kPerLane; ++e) value[e] = fmaf(w[u], part[u][e], value[e]);
        }
    }
    if (lane == 0) wave_sum[wave] = weight_sum;
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) wave_val[wave][lane * kPerLane + e] = value[e];
    __syncthreads();
    if (wave != 0) return;
    weight_sum = 0.0f;
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) value[e] = 0.0f;
#pragma unroll
    for (int w = 0; w < kWideWaves; ++w) {
        weight_sum += wave_sum[w];
#pragma unroll
        for (int e = 0; e < kPerLane; ++e) value[e] += wave_val[w][lane * kPerLane + e];
    }
    const float inv = weight_sum > 0.0f ? 1.0f / weight_sum : 0.0f;
    const uint64_t out_index = row_out * D + lane * kPerLane;
#pragma unroll
    for (int e = 0; e < kPerLane; ++e)
        store_from_f32<Tag>(a.output, out_index + e, finish_output<Tag>(a, value[e] * inv, token, q_head, lane * kPerLane + e));
}

// The same combine for Q-token tiles: one wave per (tile, token in tile, q_head); the tile's partial
// rows are cu_kv_splits[tile] .. cu_kv_splits[tile + 1].
template <typename Tag, int D, bool kIndexed>
__global__ __launch_bounds__(256) void split_kv_reduce_tiled_fast(ReduceArgs a) {
    resolve_active(a);
    constexpr int kPerLane = D / 64;
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t id = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const uint32_t rows = a.rows_per_split_head;
    const uint32_t q_head = (uint32_t)(id % a.hq);
    const uint32_t tile_row = (uint32_t)((id / a.hq) % rows);
    const uint64_t tile = id / ((uint64_t)a.hq * rows);
    if (tile >= a.num_active_q_token_tiles) return;
    const uint32_t flat_begin = a.q_token_tiles[tile * 2], flat_end = a.q_token_tiles[tile * 2 + 1];
    const uint32_t token = flat_begin + tile_row;
    if (token >= flat_end) return;
    const uint32_t begin = a.cu_kv_splits[tile], end = a.cu_kv_splits[tile + 1];
    constexpr int kUnroll = 4;
    const uint32_t* row_index = a.row_index;
    auto row_of = [&](uint32_t p) -> uint64_t {
        return ((uint64_t)(kIndexed ? row_index[p] : p) * a.hq + q_head) * rows + tile_row;
    };
    // (the first four rows ahead of the pass over the maxima, as in split_kv_reduce_fast)
    float m[kUnroll], sums[kUnroll], part[kUnroll][kPerLane];
    auto fetch = [&](uint32_t p0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool live = p0 + u < end;
            const uint64_t row = row_of(live ? p0 + u : begin);
            m[u] = a.part_max[row];
            if (!live) m[u] = -INFINITY;
            sums[u] = a.part_sum[row];
            const float* src = a.part_acc + row * D + lane * kPerLane;
#pragma unroll
            for (int e = 0; e < kPerLane; ++e) part[u][e] = src[e];
        }
    };
    if (begin < end) fetch(begin);
    float global_max = -INFINITY;
    for (uint32_t p = begin + kUnroll + lane; p < end; p += 64) global_max = fmaxf(global_max, a.part_max[row_of(p)]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) global_max = fmaxf(global_max, __shfl_xor(global_max, off, 64));
    if (begin < end) {
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) global_max = fmaxf(global_max, m[u]);
    }
    float weight_sum = 0.0f, value[kPerLane];
#pragma unroll
    for (int e = 0; e < kPerLane; ++e) value[e] = 0.0f;
    for (uint32_t p0 = begin; p0 < end; p0 += kUnroll) {
        if (p0 != begin) fetch(p0);
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const float w = m[u] > -INFINITY ? exp2f(m[u] - global_max) : 0.0f;
            weight_sum = fmaf(w, sums[u], weight_sum);
#pragma unroll
            for (int e = 0; e < kPerLane; ++e) value[e] = fmaf(w, part[u][e], value[e]);
        }
    }
    const float inv = weight_sum > 0.0f ? 1.0f / weight_sum : 0.0f;
    const uint64_t out_index = ((uint64_t)token * a.hq + q_head) * D + lane * kPerLane;
#pragma unroll
    for (int e = 0; e < kPerLane; ++e)
        store_from_f32<Tag>(a.output, out_index + e, finish_output<Tag>(a, value[e] * inv, token, q_head, lane * kPerLane + e));
}

// Shapes and pointers for which the MFMA decode map runs, i.e. for which the append can be folded into it.
bool decode_map_takes_append(const psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    if (ctx->force_generic) return false;
    const bool two_byte = g.dtype == PSI_HIP_BF16 || g.dtype == PSI_HIP_F16;
    const uint32_t p = g.tokens_per_page;
    const bool page_ok = p >= 8 && (p & (p - 1)) == 0;
    auto aligned = [](const void* ptr) { return reinterpret_cast<uintptr_t>(ptr) % 16 == 0; };
    return two_byte && page_ok && g.group <= 8 && (g.d == 256 || g.d == 128) && aligned(a.q) && aligned(a.kv_pages) &&
           aligned(a.flat_k) && aligned(a.flat_v) && (uint64_t)a.num_total_kv_splits * g.hkv <= 0x7fffffffull;
}

int launch_decode_map_fast(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    if (ctx->force_generic) return PSI_HIP_ERR_UNSUPPORTED;
    const bool two_byte = g.dtype == PSI_HIP_BF16 || g.dtype == PSI_HIP_F16;
    const uint32_t p = g.tokens_per_page;
    const bool page_ok = p >= 8 && (p & (p - 1)) == 0;
    const bool aligned = reinterpret_cast<uintptr_t>(a.q) % 16 == 0 && reinterpret_cast<uintptr_t>(a.kv_pages) % 16 == 0;
    if (!two_byte || !page_ok || !aligned || g.group > 8 || (g.d != 256 && g.d != 128)) return PSI_HIP_ERR_UNSUPPORTED;
    if ((uint64_t)a.num_total_kv_splits * g.hkv > 0x7fffffffull) return PSI_HIP_ERR_UNSUPPORTED;
    if (g.dtype == PSI_HIP_BF16)
        return g.d == 256 ? launch_decode_map_bf16_d256(ctx, g, a) : launch_decode_map_bf16_d128(ctx, g, a);
    return g.d == 256 ? launch_decode_map_f16_d256(ctx, g, a) : launch_decode_map_f16_d128(ctx, g, a);
}

int launch_reduce_fast(psi_hip_ctx* ctx, const Geometry& g, const ReduceArgs& a) {
    if (ctx->force_generic) return PSI_HIP_ERR_UNSUPPORTED;
    if (g.d != 256 && g.d != 128) return PSI_HIP_ERR_UNSUPPORTED;
    const bool tiled = a.q_token_tiles != nullptr;
    const uint64_t rows = tiled ? (uint64_t)a.num_active_q_token_tiles * a.rows_per_split_head * g.hq
                                : (uint64_t)a.num_active_tokens * g.hq;
    if ((rows + 3) / 4 > 0x7fffffffull) return PSI_HIP_ERR_UNSUPPORTED;
    const dim3 grid((uint32_t)((rows + 3) / 4)), block(256);
    // long split lists on few tokens: a workgroup per output row instead of a wave
    const bool wide = !tiled && a.num_active_tokens != 0 && a.num_total_kv_splits / a.num_active_tokens >= 32 &&
                      rows <= 0x7fffffffull;
#define PSI_REDUCE_D(TAG, DIM, INDEXED)                                                                          \
    do {                                                                                                         \
        if (tiled) hipLaunchKernelGGL((split_kv_reduce_tiled_fast<TAG, DIM, INDEXED>), grid, block, 0, ctx->stream, a); \
        else if (wide) hipLaunchKernelGGL((split_kv_reduce_wide<TAG, DIM, INDEXED>), dim3((uint32_t)rows), dim3(64 * kWideWaves), 0, ctx->stream, a); \
        else hipLaunchKernelGGL((split_kv_reduce_fast<TAG, DIM, INDEXED>), grid, block, 0, ctx->stream, a);     \
    } while (0)
#define PSI_REDUCE(TAG)                                                   \
    do {                                                                  \
        if (g.d == 256) {                                                 \
            if (a.row_index) PSI_REDUCE_D(TAG, 256, true);                \
            else PSI_REDUCE_D(TAG, 256, false);                           \
        } else {                                                          \
            if (a.row_index) PSI_REDUCE_D(TAG, 128, true);                \
            else PSI_REDUCE_D(TAG, 128, false);                           \
        }                                                                 \
    } while (0)
    if (a.out_dtype == PSI_HIP_F32) PSI_REDUCE(F32Tag);
    else if (a.out_dtype == PSI_HIP_BF16) PSI_REDUCE(BF16Tag);
    else PSI_REDUCE(F16Tag);
#undef PSI_REDUCE_D
#undef PSI_REDUCE
    return PSI_HIP_OK;
}

}  // namespace psi
