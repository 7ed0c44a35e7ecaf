// Shape-generic split-KV map and log-sum-exp combine: any head_dim, page size and element type,
// SingleQ (one Q token per split row) and TiledQ (a request-local tile of Q tokens per split row,
// causal among them).  Correctness-first kernels for shapes outside the gfx950 fast paths and the
// cross-check variant for them.  Semantics:
//   crates/inference-backend-metal/src/components/metal/gqa_split_kv_single_q_map.metal:31-253
//   crates/inference-backend-metal/src/components/metal/gqa_split_kv_single_q_reduce.metal:10-49
//   crates/inference-backend-metal/src/components/metal/gqa_split_kv_tiled_q.metal:49-378
// (exact softmax: no 1e-6 bias in the denominators).
#include "split_kv.h"

namespace psi {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// One wave per (kv_split, q_head, row-in-tile, 64-wide slice of head_dim).  Each slice recomputes
// the logits of its split so that no state is shared between waves.  Lane = key within a 64-key
// tile for QK, lane = dim for PV.
template <typename Tag>
__global__ __launch_bounds__(64) void split_kv_map_generic(MapArgs a) {
    resolve_active(a);
    const uint32_t d = a.walk.d;
    const uint32_t dim_slices = (d + 63) / 64;
    uint32_t b = blockIdx.x;
    const uint32_t slice = b % dim_slices;
    b /= dim_slices;
    const uint32_t tile_row = b % a.rows_per_split_head;
    b /= a.rows_per_split_head;
    const uint32_t split = b % a.num_total_kv_splits;
    const uint32_t q_head = b / a.num_total_kv_splits;
    if (split >= a.num_active_kv_splits) return;
    const uint32_t first = a.kv_splits[split * 3];
    uint32_t q_token, kv_end = a.kv_splits[split * 3 + 2];
    const uint32_t kv_begin = a.kv_splits[split * 3 + 1];
    if (a.q_token_tiles == nullptr) {
        q_token = first;
        if (q_token >= a.num_active_tokens) return;  // sentinel padding or a slot owned by another producer
    } else {
        if (first >= a.num_active_q_token_tiles) return;
        const uint32_t flat_begin = a.q_token_tiles[first * 2], flat_end = a.q_token_tiles[first * 2 + 1];
        if (flat_begin >= a.num_active_tokens || flat_end > a.num_active_tokens) return;
        q_token = flat_begin + tile_row;
        if (q_token >= flat_end) return;  // rows beyond the tile's tokens keep their bytes
        // causal: keys after the query's own position are hidden
        const uint32_t causal_end = a.flat_token_indices[q_token] + 1;
        kv_end = min(kv_end, causal_end);
    }
    const uint32_t req_slot = a.req_slots[q_token];
    const uint32_t kv_head = q_head / a.group;
    const uint32_t lane = threadIdx.x;
    const uint32_t my_dim = slice * 64 + lane;
    const uint64_t q_off = ((uint64_t)q_token * a.hq + q_head) * d;

    __shared__ float probs[64];
    __shared__ uint64_t v_offsets[64];

    float run_max = -INFINITY, run_sum = 0.0f, acc = 0.0f;
    for (uint32_t tile = kv_begin; tile < kv_end; tile += 64) {
        const uint32_t token = tile + lane;
        const bool valid = token < kv_end;
        float logit2 = -INFINITY;
        if (valid) {
            const uint64_t k_off = kv_line_offset(a.walk, req_slot, a.layer, token, 0, kv_head);
            float dot = 0.0f;
            for (uint32_t i = 0; i < d; ++i)
                dot += load_as_f32<Tag>(a.q, q_off + i) * load_as_f32<Tag>(a.kv_pages, k_off + i);
            logit2 = dot * a.scale_log2;
            v_offsets[lane] = kv_line_offset(a.walk, req_slot, a.layer, token, 1, kv_head);
        }
        const float tile_max = wave_max(logit2);
        const float next_max = fmaxf(run_max, tile_max);
        const float p = valid && next_max > -INFINITY ? exp2f(logit2 - next_max) : 0.0f;
        const float old_scale = run_max > -INFINITY ? exp2f(run_max - next_max) : 0.0f;
        run_sum = run_sum * old_scale + wave_sum(p);
        run_max = next_max;
        probs[lane] = p;
        __syncthreads();
        if (my_dim < d) {
            const uint32_t count = min(64u, kv_end - tile);
            float tile_acc = 0.0f;
            for (uint32_t t = 0; t < count; ++t)
                tile_acc += probs[t] * load_as_f32<Tag>(a.kv_pages, v_offsets[t] + my_dim);
            acc = acc * old_scale + tile_acc;
        }
        __syncthreads();
    }
    const uint64_t row = ((uint64_t)split * a.hq + q_head) * a.rows_per_split_head + tile_row;
    if (slice == 0 && lane == 0) {
        a.part_max[row] = run_max;
        a.part_sum[row] = run_sum;
    }
    if (my_dim < d) a.part_acc[row * d + my_dim] = acc;
}

// Log-sum-exp combine, one work-item per output element.  SingleQ: cu_kv_splits is indexed by
// token.  TiledQ: the token's tile is found from q_token_tiles and the partial row carries the
// token's offset inside the tile.
template <typename Tag>
__global__ __launch_bounds__(256) void split_kv_reduce_generic(ReduceArgs a, uint32_t num_tile_slots) {
    resolve_active(a);
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint32_t token, q_head, dim, begin, end, tile_row = 0;
    if (a.q_token_tiles == nullptr) {
        if (gid >= (uint64_t)a.num_active_tokens * a.hq * a.d) return;
        dim = (uint32_t)(gid % a.d);
        q_head = (uint32_t)((gid / a.d) % a.hq);
        token = (uint32_t)(gid / ((uint64_t)a.d * a.hq));
        begin = a.cu_kv_splits[token];
        end = a.cu_kv_splits[token + 1];
    } else {
        // gid enumerates (tile slot, row in tile, q_head, dim)
        if (gid >= (uint64_t)num_tile_slots * a.rows_per_split_head * a.hq * a.d) return;
        dim = (uint32_t)(gid % a.d);
        q_head = (uint32_t)((gid / a.d) % a.hq);
        tile_row = (uint32_t)((gid / ((uint64_t)a.d * a.hq)) % a.rows_per_split_head);
        const uint32_t tile = (uint32_t)(gid / ((uint64_t)a.d * a.hq * a.rows_per_split_head));
        if (tile >= a.num_active_q_token_tiles) return;
        const uint32_t flat_begin = a.q_token_tiles[tile * 2], flat_end = a.q_token_tiles[tile * 2 + 1];
        token = flat_begin + tile_row;
        if (token >= flat_end) return;
        begin = a.cu_kv_splits[tile];
        end = a.cu_kv_splits[tile + 1];
    }
    float global_max = -INFINITY;
    for (uint32_t p = begin; p < end; ++p) {
        const uint32_t phys = a.row_index ? a.row_index[p] : p;
        global_max = fmaxf(global_max, a.part_max[((uint64_t)phys * a.hq + q_head) * a.rows_per_split_head + tile_row]);
    }
    float weight_sum = 0.0f, value = 0.0f;
    for (uint32_t p = begin; p < end; ++p) {
        const uint32_t phys = a.row_index ? a.row_index[p] : p;
        const uint64_t row = ((uint64_t)phys * a.hq + q_head) * a.rows_per_split_head + tile_row;
        const float m = a.part_max[row];
        const float w = m > -INFINITY ? exp2f(m - global_max) : 0.0f;
        weight_sum += w * a.part_sum[row];
        value += w * a.part_acc[row * a.d + dim];
    }
    store_from_f32<Tag>(a.output, ((uint64_t)token * a.hq + q_head) * a.d + dim,
                        finish_output<Tag>(a, weight_sum > 0.0f ? value / weight_sum : 0.0f, token, q_head, dim));
}

void launch_map_generic(psi_hip_ctx* ctx, const Geometry& g, const MapArgs& a) {
    const uint64_t grid64 = (uint64_t)a.num_total_kv_splits * g.hq * a.rows_per_split_head * ((g.d + 63) / 64);
    const dim3 grid((uint32_t)grid64), block(64);
    if (g.dtype == PSI_HIP_F32) hipLaunchKernelGGL(split_kv_map_generic<F32Tag>, grid, block, 0, ctx->stream, a);
    else if (g.dtype == PSI_HIP_BF16) hipLaunchKernelGGL(split_kv_map_generic<BF16Tag>, grid, block, 0, ctx->stream, a);
    else hipLaunchKernelGGL(split_kv_map_generic<F16Tag>, grid, block, 0, ctx->stream, a);
}

void launch_reduce_generic(psi_hip_ctx* ctx, const Geometry& g, const ReduceArgs& a, uint32_t num_tile_slots) {
    const uint64_t total = a.q_token_tiles == nullptr
                               ? (uint64_t)a.num_active_tokens * a.hq * a.d
                               : (uint64_t)num_tile_slots * a.rows_per_split_head * a.hq * a.d;
    const dim3 grid((uint32_t)((total + 255) / 256)), block(256);
    (void)g;
    if (a.out_dtype == PSI_HIP_F32)
        hipLaunchKernelGGL(split_kv_reduce_generic<F32Tag>, grid, block, 0, ctx->stream, a, num_tile_slots);
    else if (a.out_dtype == PSI_HIP_BF16)
        hipLaunchKernelGGL(split_kv_reduce_generic<BF16Tag>, grid, block, 0, ctx->stream, a, num_tile_slots);
    else
        hipLaunchKernelGGL(split_kv_reduce_generic<F16Tag>, grid, block, 0, ctx->stream, a, num_tile_slots);
}

void fill_walk(PageWalk* walk, const Geometry& g, const psi_hip_page_table_layout* layout, const uint32_t* page_ids) {
    walk->page_ids = page_ids;
    walk->num_layers = layout->num_gqa_layers;
    walk->num_blocks = layout->num_blocks;
    walk->ids_per_block = layout->num_page_ids_per_block;
    walk->tokens_per_page = g.tokens_per_page;
    walk->hkv = g.hkv;
    walk->d = g.d;
    walk->page_elems = g.page_elems;
}

}  // namespace psi
