// Split-KV decode attention (SingleQ): C-ABI entry points and dispatch between the gfx950 fast
// kernels and the shape-generic ones.  Semantics follow
// crates/inference-backend-metal/src/components/metal/gqa_split_kv_single_q_map.metal:31-253 and
// gqa_split_kv_single_q_reduce.metal:10-49: one partial state per (kv_split, q_head), online
// softmax over the split's keys, log-sum-exp combine over the splits of each token.
#include <cmath>

#include "split_kv.h"

namespace psi {

constexpr float kLog2e = 1.4426950408889634f;

// Reference shape checks: gqa_split_kv_single_q.rs:197-209.
static int check_single_q_shape(const Geometry& g, uint32_t num_total_tokens, uint32_t num_total_kv_splits) {
    PSI_REQUIRE(g.scale > 0.0f, "GQA attention scale must be positive");
    PSI_REQUIRE(num_total_tokens > 0, "GQA SDPA requires tokens");
    PSI_REQUIRE(num_total_kv_splits > 0, "GQA SDPA requires KV splits");
    const uint64_t out_values = (uint64_t)num_total_tokens * g.hq * g.d;
    PSI_REQUIRE(out_values <= UINT32_MAX, "GQA SDPA query/output exceeds the shader u32 count domain: count=%llu",
                (unsigned long long)out_values);
    const uint64_t stats = (uint64_t)num_total_kv_splits * g.hq;
    PSI_REQUIRE(stats - 1 <= UINT32_MAX, "GQA SDPA partial-output stats exceeds the shader u32 element-index domain");
    PSI_REQUIRE(stats * g.d - 1 <= UINT32_MAX,
                "GQA SDPA partial output exceeds the shader u32 element-index domain");
    return PSI_HIP_OK;
}

struct StorePartialsArgs {
    const uint32_t* slot_rows;
    const uint32_t* row_index;
    const uint32_t* replay_counts;
    const float* exp_sums;
    const float* max_logits;
    const void* partial_output;
    float* part_max;
    float* part_sum;
    float* part_acc;
    uint32_t hq, d, dtype, num_active_tokens, num_total_kv_splits;
};

// One wave per (token, query head): the partial result another attention task produced for the token, in the
// form crates/inference-backend-metal/src/components/metal/gqa_block_sdpa.metal:47-76 writes it (maximum of
// the scaled natural-log logits, sum of exponentials, output already divided by that sum), entered into the
// split row reserved for it in the form the combine merges (base-2 maximum, sum, undivided output).
__global__ __launch_bounds__(256) void store_partials_kernel(StorePartialsArgs a) {
    const uint32_t active = active_count(a.replay_counts, kReplayTokens, a.num_active_tokens);
    const uint32_t item = (blockIdx.x * 256 + threadIdx.x) / 64, lane = threadIdx.x % 64;
    if (item >= active * a.hq) return;
    const uint32_t token = item / a.hq, head = item % a.hq;
    uint32_t row = a.slot_rows[token];
    if (row >= a.num_total_kv_splits) return;  // a token without a reserved row
    if (a.row_index != nullptr) row = a.row_index[row];
    const uint64_t src = (uint64_t)token * a.hq + head, dst = (uint64_t)row * a.hq + head;
    const float max_logit = a.max_logits[src], exp_sum = a.exp_sums[src];
    const bool live = isfinite(max_logit) && exp_sum > 0.0f;
    for (uint32_t dim = lane; dim < a.d; dim += 64)
        a.part_acc[dst * a.d + dim] = live ? load_any_as_f32(a.partial_output, src * a.d + dim, a.dtype) * exp_sum : 0.0f;
    if (lane == 0) {
        a.part_max[dst] = live ? max_logit * kLog2e : -INFINITY;
        a.part_sum[dst] = live ? exp_sum : 0.0f;
    }
}

}  // namespace psi

using namespace psi;

extern "C" int psi_hip_split_kv_single_q_scratch_bytes(const psi_hip_gqa_config* cfg, uint32_t num_total_kv_splits,
                                                       uint64_t* out_bytes) {
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_bytes != nullptr, "out pointer must not be null");
    PSI_REQUIRE(num_total_kv_splits > 0, "GQA SDPA requires KV splits");
    *out_bytes = partial_layout(num_total_kv_splits, g.hq, g.d, 1).total_bytes;
    return PSI_HIP_OK;
}

static int single_q_map_impl(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
                             const void* q, const void* kv_pages, uint64_t kv_pages_bytes, const uint32_t* req_slots,
                             const uint32_t* page_ids, const uint32_t* kv_splits, const uint32_t* worker_cu,
                             uint32_t num_workers, void* scratch, uint64_t scratch_bytes, uint32_t gqa_layer_index,
                             uint32_t num_total_tokens, uint32_t num_total_kv_splits, uint32_t num_active_tokens,
                             uint32_t num_active_kv_splits, const void* flat_k = nullptr, const void* flat_v = nullptr,
                             const uint32_t* flat_token_indices = nullptr) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_layout(layout);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_single_q_shape(g, num_total_tokens, num_total_kv_splits);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(q && kv_pages && req_slots && page_ids && kv_splits && scratch,
                "GQA SplitKV SingleQ map buffers must not be null");
    PSI_REQUIRE(gqa_layer_index < layout->num_gqa_layers, "GQA page-table index exceeds layer count");
    PSI_REQUIRE(num_active_tokens > 0, "GQA SplitKV SingleQ active token count must be positive");
    PSI_REQUIRE(num_active_tokens <= num_total_tokens,
                "GQA SplitKV SingleQ active token count exceeds recorded capacity");
    PSI_REQUIRE(num_active_kv_splits > 0, "GQA SplitKV SingleQ active KV split count must be positive");
    PSI_REQUIRE(num_active_kv_splits <= num_total_kv_splits,
                "GQA SplitKV SingleQ active KV split count exceeds recorded capacity");
    PSI_REQUIRE(kv_pages_bytes == 0 || kv_pages_bytes >= cfg->page_bytes, "GQA page arena is smaller than one page");
    const PartialLayout pl = partial_layout(num_total_kv_splits, g.hq, g.d, 1);
    PSI_REQUIRE(scratch_bytes >= pl.total_bytes, "GQA SplitKV SingleQ scratch too small: %llu < %llu",
                (unsigned long long)scratch_bytes, (unsigned long long)pl.total_bytes);

    MapArgs a;
    a.q = q;
    a.kv_pages = kv_pages;
    a.req_slots = req_slots;
    a.kv_splits = kv_splits;
    a.part_max = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.max_offset);
    a.part_sum = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.sum_offset);
    a.part_acc = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.acc_offset);
    fill_walk(&a.walk, g, layout, page_ids);
    a.layer = gqa_layer_index;
    a.hq = g.hq;
    a.group = g.group;
    a.num_total_kv_splits = num_total_kv_splits;
    a.num_active_tokens = num_active_tokens;
    a.num_active_kv_splits = num_active_kv_splits;
    a.replay_counts = ctx->replay_counts;
    a.scale_log2 = g.scale * kLog2e;
    a.worker_cu = worker_cu;
    a.num_workers = num_workers;
    if (flat_k != nullptr) {
        // the append travels with the map when the MFMA kernel serves the shape, else it is a launch of its own
        a.flat_k = flat_k;
        a.flat_v = flat_v;
        a.flat_token_indices = flat_token_indices;
        if (!decode_map_takes_append(ctx, g, a)) {
            rc = psi_hip_kv_page_write(ctx, cfg, layout, const_cast<void*>(kv_pages), kv_pages_bytes, flat_k, flat_v,
                                       req_slots, flat_token_indices, page_ids, num_total_tokens, num_active_tokens,
                                       gqa_layer_index);
            if (rc != PSI_HIP_OK) return rc;
            a.flat_k = a.flat_v = nullptr;
            a.flat_token_indices = nullptr;
        }
    }

    LaunchScope scope(ctx, "split_kv_map");
    rc = launch_decode_map_fast(ctx, g, a);
    if (rc == PSI_HIP_ERR_UNSUPPORTED) {
        const uint64_t grid = (uint64_t)num_total_kv_splits * g.hq * ((g.d + 63) / 64);
        PSI_REQUIRE(grid <= 0x7fffffffull, "GQA SDPA map threads exceeds the shader u32 count domain");
        a.worker_cu = nullptr;  // the generic kernel launches one workgroup per row
        launch_map_generic(ctx, g, a);
        rc = PSI_HIP_OK;
    }
    if (rc != PSI_HIP_OK) return rc;
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_split_kv_single_q_map(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                             const psi_hip_page_table_layout* layout, const void* q,
                                             const void* kv_pages, uint64_t kv_pages_bytes,
                                             const uint32_t* req_slots, const uint32_t* page_ids,
                                             const uint32_t* kv_splits, void* scratch, uint64_t scratch_bytes,
                                             uint32_t gqa_layer_index, uint32_t num_total_tokens,
                                             uint32_t num_total_kv_splits, uint32_t num_active_tokens,
                                             uint32_t num_active_kv_splits) {
    return single_q_map_impl(ctx, cfg, layout, q, kv_pages, kv_pages_bytes, req_slots, page_ids, kv_splits, nullptr, 0,
                             scratch, scratch_bytes, gqa_layer_index, num_total_tokens, num_total_kv_splits,
                             num_active_tokens, num_active_kv_splits);
}

extern "C" int psi_hip_split_kv_single_q_map_balanced(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                                      const psi_hip_page_table_layout* layout, const void* q,
                                                      const void* kv_pages, uint64_t kv_pages_bytes,
                                                      const uint32_t* req_slots, const uint32_t* page_ids,
                                                      const uint32_t* kv_splits, const uint32_t* worker_cu,
                                                      uint32_t num_workers, void* scratch, uint64_t scratch_bytes,
                                                      uint32_t gqa_layer_index, uint32_t num_total_tokens,
                                                      uint32_t num_total_kv_splits, uint32_t num_active_tokens,
                                                      uint32_t num_active_kv_splits) {
    PSI_REQUIRE(worker_cu != nullptr && num_workers > 0, "balanced map needs a worker table");
    return single_q_map_impl(ctx, cfg, layout, q, kv_pages, kv_pages_bytes, req_slots, page_ids, kv_splits, worker_cu,
                             num_workers, scratch, scratch_bytes, gqa_layer_index, num_total_tokens,
                             num_total_kv_splits, num_active_tokens, num_active_kv_splits);
}

extern "C" int psi_hip_split_kv_single_q_reduce(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const void* scratch,
                                                uint64_t scratch_bytes, const uint32_t* cu_kv_splits, void* output,
                                                uint32_t num_total_tokens, uint32_t num_total_kv_splits,
                                                uint32_t num_active_tokens, const uint32_t* partial_row_index,
                                                const psi_hip_output_gate* gate) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_single_q_shape(g, num_total_tokens, num_total_kv_splits);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(scratch && cu_kv_splits && output, "GQA SplitKV SingleQ reduce buffers must not be null");
    PSI_REQUIRE(num_active_tokens > 0, "GQA SplitKV SingleQ active token count must be positive");
    PSI_REQUIRE(num_active_tokens <= num_total_tokens,
                "GQA SplitKV SingleQ active token count exceeds recorded capacity");
    const PartialLayout pl = partial_layout(num_total_kv_splits, g.hq, g.d, 1);
    PSI_REQUIRE(scratch_bytes >= pl.total_bytes, "GQA SplitKV SingleQ scratch too small: %llu < %llu",
                (unsigned long long)scratch_bytes, (unsigned long long)pl.total_bytes);
    ReduceArgs a;
    a.part_max = reinterpret_cast<const float*>(static_cast<const char*>(scratch) + pl.max_offset);
    a.part_sum = reinterpret_cast<const float*>(static_cast<const char*>(scratch) + pl.sum_offset);
    a.part_acc = reinterpret_cast<const float*>(static_cast<const char*>(scratch) + pl.acc_offset);
    a.cu_kv_splits = cu_kv_splits;
    a.row_index = partial_row_index;
    a.replay_counts = ctx->replay_counts;
    a.output = output;
    a.hq = g.hq;
    a.d = g.d;
    a.out_dtype = ctx->f32_output ? PSI_HIP_F32 : g.dtype;
    a.num_active_tokens = num_active_tokens;
    a.num_total_kv_splits = num_total_kv_splits;
    rc = set_output_gate(&a, gate, g);
    if (rc != PSI_HIP_OK) return rc;

    LaunchScope scope(ctx, "split_kv_reduce");
    rc = launch_reduce_fast(ctx, g, a);
    if (rc == PSI_HIP_ERR_UNSUPPORTED) {
        launch_reduce_generic(ctx, g, a, 0);
        rc = PSI_HIP_OK;
    }
    if (rc != PSI_HIP_OK) return rc;
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_split_kv_single_q_store_partials(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, void* scratch,
                                                        uint64_t scratch_bytes, const uint32_t* slot_rows,
                                                        const float* partial_exp_sums, const float* partial_max_logits,
                                                        const void* partial_output, uint32_t num_total_tokens,
                                                        uint32_t num_total_kv_splits, uint32_t num_active_tokens,
                                                        const uint32_t* partial_row_index) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_single_q_shape(g, num_total_tokens, num_total_kv_splits);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(scratch && slot_rows && partial_exp_sums && partial_max_logits && partial_output,
                "GQA SplitKV SingleQ partial-output buffers must not be null");
    PSI_REQUIRE(num_active_tokens > 0, "GQA SplitKV SingleQ active token count must be positive");
    PSI_REQUIRE(num_active_tokens <= num_total_tokens,
                "GQA SplitKV SingleQ active token count exceeds recorded capacity");
    const PartialLayout pl = partial_layout(num_total_kv_splits, g.hq, g.d, 1);
    PSI_REQUIRE(scratch_bytes >= pl.total_bytes, "GQA SplitKV SingleQ scratch too small: %llu < %llu",
                (unsigned long long)scratch_bytes, (unsigned long long)pl.total_bytes);
    StorePartialsArgs a;
    a.slot_rows = slot_rows;
    a.row_index = partial_row_index;
    a.replay_counts = ctx->replay_counts;
    a.exp_sums = partial_exp_sums;
    a.max_logits = partial_max_logits;
    a.partial_output = partial_output;
    a.part_max = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.max_offset);
    a.part_sum = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.sum_offset);
    a.part_acc = reinterpret_cast<float*>(static_cast<char*>(scratch) + pl.acc_offset);
    a.hq = g.hq;
    a.d = g.d;
    a.dtype = g.dtype;
    a.num_active_tokens = num_active_tokens;
    a.num_total_kv_splits = num_total_kv_splits;

    LaunchScope scope(ctx, "split_kv_store_partials");
    const uint64_t waves = (uint64_t)num_active_tokens * g.hq;
    hipLaunchKernelGGL(store_partials_kernel, dim3((uint32_t)((waves + 3) / 4)), dim3(256), 0, ctx->stream, a);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_kv_page_write_split_kv_single_q_map(
    psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout, const void* q,
    void* kv_pages, uint64_t kv_pages_bytes, const void* flat_k, const void* flat_v, const uint32_t* req_slots,
    const uint32_t* flat_token_indices, const uint32_t* page_ids, const uint32_t* kv_splits,
    const uint32_t* worker_cu, uint32_t num_workers, void* scratch, uint64_t scratch_bytes, uint32_t gqa_layer_index,
    uint32_t num_total_tokens, uint32_t num_total_kv_splits, uint32_t num_active_tokens,
    uint32_t num_active_kv_splits) {
    PSI_REQUIRE(flat_k && flat_v && flat_token_indices, "GQA KV page write buffers must not be null");
    PSI_REQUIRE((worker_cu == nullptr) == (num_workers == 0), "a worker table needs its worker count and vice versa");
    return single_q_map_impl(ctx, cfg, layout, q, kv_pages, kv_pages_bytes, req_slots, page_ids, kv_splits, worker_cu,
                             num_workers, scratch, scratch_bytes, gqa_layer_index, num_total_tokens,
                             num_total_kv_splits, num_active_tokens, num_active_kv_splits, flat_k, flat_v,
                             flat_token_indices);
}
