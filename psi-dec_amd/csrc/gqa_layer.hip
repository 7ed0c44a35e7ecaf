// The attention layer as one call, and one recorded program per capacity bucket.
//
// psi_hip_gqa_layer_record mirrors `GQA::record` / `UngatedGQA::record`
// (crates/inference-executor-metal/src/attn/gqa/backend.rs:394-658, ungated_backend.rs:182-380) between the two
// matmuls: QGKV split -> Q / K RMSNorm + RoPE -> KV page write -> SplitKV map of the batch's variant -> combine ->
// gate, issued in this library's fused form (prepare launch, map, combine with gate).  It only sequences the
// component entry points of include/psi_hip.h; every check and kernel lives with them.
//
// psi_hip_gqa_replay_cache_* keeps one HIP graph per `(variant, total tokens, total Q-token tiles, total KV
// splits)` key, captured from that call with the device-side count block bound, as the reference keeps one
// recorded program per key and binds `gqa.num_active_*` at submission
// (crates/inference-executor-core/src/replay.rs:4-87, backend.rs:55-57).
#include <algorithm>
#include <cstring>
#include <list>
#include <vector>

#include "common.h"
#include "device_types.h"

// Partial-state storage for callers that cannot allocate: one array per GPU, inside the library's code object,
// held from the moment the library is loaded on that GPU until the process ends.  In host code `scratch` is only
// a stand-in for the symbol: the device address comes from hipGetSymbolAddress, once per device, and that address
// is what kernels and checks use.
constexpr uint64_t kStaticScratchBytes = PSI_HIP_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace psi {

constexpr int kMaxStaticScratchDevices = 64;
static void* g_static_scratch[kMaxStaticScratchDevices] = {};  // device address of `scratch` on each GPU

// Looks up this GPU's copy of the array.  `device` must be the current device of the calling thread.
int resolve_static_scratch(int device) {
    PSI_REQUIRE(device >= 0 && device < kMaxStaticScratchDevices, "device %d has no static scratch slot", device);
    if (g_static_scratch[device] != nullptr) return PSI_HIP_OK;
    void* ptr = nullptr;
    PSI_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    PSI_REQUIRE(ptr != nullptr && reinterpret_cast<uintptr_t>(ptr) % 256 == 0, "static scratch address is not usable");
    g_static_scratch[device] = ptr;
    return PSI_HIP_OK;
}

namespace {

struct LayerPlan {
    Geometry g;
    psi_hip_rms_norm_rope_config q_norm, k_norm;
    uint64_t token_width = 0;   // elements per projection row
    uint64_t q_head_stride = 0; // elements between the q rows of neighbouring heads
    uint64_t k_offset = 0, v_offset = 0;
};

int make_layer_plan(const psi_hip_gqa_layer_config* cfg, LayerPlan* plan) {
    PSI_REQUIRE(cfg != nullptr, "GQA layer config must not be null");
    int rc = make_geometry(&cfg->attention, &plan->g);
    if (rc != PSI_HIP_OK) return rc;
    const Geometry& g = plan->g;
    PSI_REQUIRE(cfg->gated <= 1, "GQA layer `gated` must be 0 or 1");
    psi_hip_rms_norm_rope_config n;
    n.num_heads = g.hq;
    n.head_dim = g.d;
    n.rope_dim = cfg->rope_dim;
    n.eps = cfg->norm_eps;
    n.rope_theta = cfg->rope_theta;
    n.scaling = cfg->rope_scaling;
    n.dtype = g.dtype;
    plan->q_norm = n;
    n.num_heads = g.hkv;
    plan->k_norm = n;
    if (cfg->gated) {  // [q_0|g_0|q_1|g_1|...|k|v], metal/gqa_qgkv_split.metal:5-43
        plan->token_width = 2ull * ((uint64_t)g.hq + g.hkv) * g.d;
        plan->q_head_stride = 2ull * g.d;
        plan->k_offset = 2ull * g.hq * g.d;
    } else {  // [q|k|v], metal/gqa_qkv_split.metal
        plan->token_width = ((uint64_t)g.hq + 2ull * g.hkv) * g.d;
        plan->q_head_stride = g.d;
        plan->k_offset = (uint64_t)g.hq * g.d;
    }
    plan->v_offset = plan->k_offset + (uint64_t)g.hkv * g.d;
    return PSI_HIP_OK;
}

const void* offset_elems(const void* base, uint64_t elems, uint32_t elem_bytes) {
    return static_cast<const char*>(base) + elems * elem_bytes;
}

// `GQAReplayShape::validate` (crates/inference-executor-core/src/attn/gqa/core.rs:135-142) and
// `GQA::validate_input` (backend.rs:231-252).
int check_input(const psi_hip_gqa_layer_input* in) {
    PSI_REQUIRE(in != nullptr, "GQA layer input must not be null");
    PSI_REQUIRE(in->batch_metadata != nullptr, "GQA batch metadata must be updated before recording");
    const psi_hip_gqa_replay_shape& s = in->batch_metadata->shape;
    PSI_REQUIRE(s.num_tokens > 0 && s.num_tokens <= s.num_total_tokens, "GQA replay shape: 0 < tokens <= capacity");
    PSI_REQUIRE(s.num_q_token_tiles > 0 && s.num_q_token_tiles <= s.num_tokens &&
                    s.num_q_token_tiles <= s.num_total_q_token_tiles,
                "GQA replay shape: 0 < Q-token tiles <= tokens, capacity");
    PSI_REQUIRE(s.num_kv_splits >= s.num_q_token_tiles && s.num_kv_splits <= s.num_total_kv_splits,
                "GQA replay shape: Q-token tiles <= KV splits <= capacity");
    PSI_REQUIRE(in->replay_mode == PSI_HIP_REPLAY_EXACT || in->replay_mode == PSI_HIP_REPLAY_BUCKETED,
                "unknown GQA replay mode %u", in->replay_mode);
    if (in->replay_mode == PSI_HIP_REPLAY_EXACT)
        PSI_REQUIRE(s.num_tokens == s.num_total_tokens && s.num_q_token_tiles == s.num_total_q_token_tiles,
                    "GQA exact replay requires active counts equal to the recorded capacities");
    int rc = check_layout(&in->page_table_layout);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(in->gqa_layer_index < in->page_table_layout.num_gqa_layers, "GQA page-table index exceeds layer count");
    const uint32_t kind = in->batch_metadata->variant.kind;
    PSI_REQUIRE(kind == PSI_HIP_VARIANT_SINGLE_Q || kind == PSI_HIP_VARIANT_TILED_Q, "unknown SplitKV variant %u", kind);
    PSI_REQUIRE(in->kv_pages && in->page_ids && in->partial_scratch && in->output,
                "GQA layer cache, scratch and output buffers must not be null");
    return PSI_HIP_OK;
}

int record_layer(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg, const psi_hip_gqa_layer_input* in) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    LayerPlan plan;
    int rc = make_layer_plan(cfg, &plan);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_input(in);
    if (rc != PSI_HIP_OK) return rc;
    const Geometry& g = plan.g;
    const psi_hip_gqa_batch_metadata& md = *in->batch_metadata;
    const psi_hip_gqa_replay_shape& s = md.shape;
    const psi_hip_gqa_config* acfg = &cfg->attention;
    const psi_hip_page_table_layout* layout = &in->page_table_layout;
    const bool tiled = md.variant.kind == PSI_HIP_VARIANT_TILED_Q;
    const uint32_t layer = in->gqa_layer_index;

    const void* q = in->q;
    psi_hip_output_gate gate_storage;
    const psi_hip_output_gate* gate = nullptr;
    bool append_with_map = false;
    if (in->qgkv != nullptr) {
        // split + Q norm/rope + K norm/rope + page write: one launch over strided views of the projection output
        PSI_REQUIRE(in->q_norm_weight && in->k_norm_weight && in->q_norm_rope,
                    "GQA layer norm weights and the q_norm_rope scratch must not be null");
        rc = psi_hip_qk_norm_rope_kv_page_write(
            ctx, acfg, layout, &plan.q_norm, &plan.k_norm, in->qgkv, plan.token_width, plan.q_head_stride,
            in->q_norm_weight, in->q_norm_rope, in->kv_pages, in->kv_pages_bytes,
            offset_elems(in->qgkv, plan.k_offset, g.elem), plan.token_width,
            offset_elems(in->qgkv, plan.v_offset, g.elem), plan.token_width, in->k_norm_weight, md.req_slots,
            md.flat_token_indices, in->page_ids, s.num_total_tokens, s.num_tokens, layer);
        if (rc != PSI_HIP_OK) return rc;
        q = in->q_norm_rope;
        if (cfg->gated) {
            gate_storage = psi_hip_output_gate{offset_elems(in->qgkv, g.d, g.elem), plan.token_width, 2ull * g.d};
            gate = &gate_storage;
        }
    } else {
        PSI_REQUIRE(in->q && in->k && in->v, "GQA layer needs the projection output or split q / k / v rows");
        if (in->g != nullptr) {
            gate_storage = psi_hip_output_gate{in->g, (uint64_t)g.hq * g.d, g.d};
            gate = &gate_storage;
        }
        if (tiled) {
            rc = psi_hip_kv_page_write(ctx, acfg, layout, in->kv_pages, in->kv_pages_bytes, in->k, in->v, md.req_slots,
                                       md.flat_token_indices, in->page_ids, s.num_total_tokens, s.num_tokens, layer);
            if (rc != PSI_HIP_OK) return rc;
        } else {
            append_with_map = true;  // the decode map writes each token's lines itself
        }
    }

    if (tiled) {
        const uint32_t ts = md.variant.q_token_tile_size;
        PSI_REQUIRE(md.q_token_tiles != nullptr, "GQA SplitKV TiledQ needs the Q-token tile table");
        if (md.row_groups != nullptr && md.num_row_groups != 0)
            rc = psi_hip_split_kv_tiled_q_map_grouped(
                ctx, acfg, layout, ts, q, in->kv_pages, in->kv_pages_bytes, md.req_slots, in->page_ids,
                md.flat_token_indices, md.q_token_tiles, md.kv_splits, in->partial_scratch, in->partial_scratch_bytes,
                layer, s.num_total_tokens, s.num_total_q_token_tiles, s.num_total_kv_splits, s.num_tokens,
                s.num_q_token_tiles, s.num_kv_splits, md.max_active_q_tile_tokens, md.row_groups, md.group_tiles,
                md.num_row_groups);
        else if (md.worker_cu != nullptr)
            rc = psi_hip_split_kv_tiled_q_map_balanced(
                ctx, acfg, layout, ts, q, in->kv_pages, in->kv_pages_bytes, md.req_slots, in->page_ids,
                md.flat_token_indices, md.q_token_tiles, md.kv_splits, md.worker_cu, md.num_workers,
                in->partial_scratch, in->partial_scratch_bytes, layer, s.num_total_tokens, s.num_total_q_token_tiles,
                s.num_total_kv_splits, s.num_tokens, s.num_q_token_tiles, s.num_kv_splits, md.max_active_q_tile_tokens);
        else
            rc = psi_hip_split_kv_tiled_q_map(
                ctx, acfg, layout, ts, q, in->kv_pages, in->kv_pages_bytes, md.req_slots, in->page_ids,
                md.flat_token_indices, md.q_token_tiles, md.kv_splits, in->partial_scratch, in->partial_scratch_bytes,
                layer, s.num_total_tokens, s.num_total_q_token_tiles, s.num_total_kv_splits, s.num_tokens,
                s.num_q_token_tiles, s.num_kv_splits, md.max_active_q_tile_tokens);
        if (rc != PSI_HIP_OK) return rc;
        return psi_hip_split_kv_tiled_q_reduce(ctx, acfg, ts, in->partial_scratch, in->partial_scratch_bytes,
                                               md.q_token_tiles, md.cu_kv_splits, in->output, s.num_total_tokens,
                                               s.num_total_q_token_tiles, s.num_total_kv_splits, s.num_q_token_tiles,
                                               md.partial_row_index, gate);
    }
    if (append_with_map)
        rc = psi_hip_kv_page_write_split_kv_single_q_map(
            ctx, acfg, layout, q, in->kv_pages, in->kv_pages_bytes, in->k, in->v, md.req_slots, md.flat_token_indices,
            in->page_ids, md.kv_splits, md.worker_cu, md.worker_cu ? md.num_workers : 0, in->partial_scratch,
            in->partial_scratch_bytes, layer, s.num_total_tokens, s.num_total_kv_splits, s.num_tokens, s.num_kv_splits);
    else if (md.worker_cu != nullptr)
        rc = psi_hip_split_kv_single_q_map_balanced(
            ctx, acfg, layout, q, in->kv_pages, in->kv_pages_bytes, md.req_slots, in->page_ids, md.kv_splits,
            md.worker_cu, md.num_workers, in->partial_scratch, in->partial_scratch_bytes, layer, s.num_total_tokens,
            s.num_total_kv_splits, s.num_tokens, s.num_kv_splits);
    else
        rc = psi_hip_split_kv_single_q_map(ctx, acfg, layout, q, in->kv_pages, in->kv_pages_bytes, md.req_slots,
                                           in->page_ids, md.kv_splits, in->partial_scratch, in->partial_scratch_bytes,
                                           layer, s.num_total_tokens, s.num_total_kv_splits, s.num_tokens,
                                           s.num_kv_splits);
    if (rc != PSI_HIP_OK) return rc;
    return psi_hip_split_kv_single_q_reduce(ctx, acfg, in->partial_scratch, in->partial_scratch_bytes, md.cu_kv_splits,
                                            in->output, s.num_total_tokens, s.num_total_kv_splits, s.num_tokens,
                                            md.partial_row_index, gate);
}

// Writes the four words of the count block from kernel arguments: stream-ordered ahead of the program that reads
// them, no host memory involved (a plain store; the block is ordinary device memory).
__global__ void set_replay_counts_kernel(uint32_t* block, uint32_t tokens, uint32_t tiles, uint32_t splits,
                                         uint32_t layer_plus_one) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        block[kReplayTokens] = tokens;
        block[kReplayTiles] = tiles;
        block[kReplaySplits] = splits;
        block[kReplayLayer] = layer_plus_one;
    }
}

// What a recorded program depends on: everything that becomes a kernel argument or a grid size.
struct ProgramKey {
    psi_hip_split_kv_variant variant;
    uint32_t totals[3];
    psi_hip_page_table_layout layout;
    uint32_t layer, replay_mode, layer_is_parameter;
    uint32_t num_workers, group_tiles, num_row_groups, max_active_q_tile_tokens;
    // context state that ends up in kernel arguments or decides which kernel runs
    uint32_t f32_output, force_generic, mute_loaders;
    uint64_t kv_pages_bytes, partial_scratch_bytes;
    const void* pointers[21];
};

ProgramKey make_key(const psi_hip_ctx& ctx, const psi_hip_gqa_layer_input& in, bool layer_is_parameter) {
    ProgramKey k;
    std::memset(&k, 0, sizeof(k));  // padding bytes take part in the comparison
    const psi_hip_gqa_batch_metadata& md = *in.batch_metadata;
    k.variant = md.variant;
    k.totals[0] = md.shape.num_total_tokens;
    k.totals[1] = md.shape.num_total_q_token_tiles;
    k.totals[2] = md.shape.num_total_kv_splits;
    k.layout = in.page_table_layout;
    k.layer = layer_is_parameter ? 0u : in.gqa_layer_index;
    k.layer_is_parameter = layer_is_parameter;
    k.replay_mode = in.replay_mode;
    k.num_workers = md.worker_cu ? md.num_workers : 0;
    k.group_tiles = md.row_groups ? md.group_tiles : 0;
    k.num_row_groups = md.row_groups ? md.num_row_groups : 0;
    k.max_active_q_tile_tokens = md.max_active_q_tile_tokens;
    k.f32_output = ctx.f32_output;
    k.force_generic = ctx.force_generic;
    k.mute_loaders = ctx.mute_loaders;
    k.kv_pages_bytes = in.kv_pages_bytes;
    k.partial_scratch_bytes = in.partial_scratch_bytes;
    const void* p[21] = {in.qgkv, in.q, in.k, in.v, in.g, in.kv_pages, in.page_ids, in.q_norm_weight,
                         in.k_norm_weight, in.q_norm_rope, in.partial_scratch, in.output, md.req_slots,
                         md.flat_token_indices, md.q_token_tiles, md.kv_splits, md.cu_kv_splits,
                         md.partial_row_index, md.worker_cu, md.row_groups, md.replay_counts};
    std::memcpy(k.pointers, p, sizeof(p));
    return k;
}

struct Program {
    ProgramKey key;
    hipGraphExec_t exec = nullptr;
};

}  // namespace
}  // namespace psi

struct psi_hip_gqa_replay_cache {
    psi_hip_ctx* ctx = nullptr;
    psi_hip_gqa_layer_config cfg;
    uint32_t* device_counts = nullptr;
    uint32_t max_programs = 0;
    std::list<psi::Program> programs;  // most recently used first
    uint64_t recordings = 0, replays = 0;
};

using namespace psi;

extern "C" int psi_hip_gqa_layer_scratch_bytes(const psi_hip_gqa_layer_config* cfg,
                                               const psi_hip_split_kv_variant* variant, uint32_t num_total_kv_splits,
                                               uint64_t* out_bytes) {
    PSI_REQUIRE(cfg != nullptr && variant != nullptr, "GQA layer config and variant must not be null");
    if (variant->kind == PSI_HIP_VARIANT_TILED_Q)
        return psi_hip_split_kv_tiled_q_scratch_bytes(&cfg->attention, variant->q_token_tile_size, num_total_kv_splits,
                                                      out_bytes);
    PSI_REQUIRE(variant->kind == PSI_HIP_VARIANT_SINGLE_Q, "unknown SplitKV variant %u", variant->kind);
    return psi_hip_split_kv_single_q_scratch_bytes(&cfg->attention, num_total_kv_splits, out_bytes);
}

extern "C" int psi_hip_gqa_layer_prepare(const psi_hip_gqa_layer_config* cfg, const psi_hip_gqa_plan_options* options,
                                         const uint32_t* req_slots, const uint32_t* token_indices,
                                         const uint32_t* cu_tokens, uint32_t num_reqs,
                                         const psi_hip_split_kv_variant* variant,
                                         const psi_hip_gqa_host_metadata* host, psi_hip_gqa_batch_metadata* out_plan,
                                         uint32_t* out_uses) {
    PSI_REQUIRE(cfg && options && host && out_plan, "GQA prepare: config, options, host arrays and out_plan must not be null");
    PSI_REQUIRE(req_slots && token_indices && cu_tokens && num_reqs > 0, "GQA prepare needs a batch");
    PSI_REQUIRE(host->req_slots_by_token && host->flat_token_indices && host->q_token_tiles && host->kv_splits &&
                    host->cu_kv_splits,
                "GQA prepare: the metadata arrays must not be null");
    PSI_REQUIRE(options->dispatch <= PSI_HIP_DISPATCH_AUTO, "unknown dispatch plan %u", options->dispatch);
    psi_hip_split_kv_variant chosen;
    int rc;
    if (variant != nullptr) {
        chosen = *variant;
    } else {
        rc = psi_hip_split_kv_select_batch(&cfg->attention, host->max_tokens, options->bucket_max_tokens, token_indices,
                                           cu_tokens, num_reqs, &chosen);
        if (rc != PSI_HIP_OK) return rc;
    }
    const bool tiled = chosen.kind == PSI_HIP_VARIANT_TILED_Q;
    uint32_t dispatch = options->dispatch;
    uint32_t partition_tokens = options->partition_tokens;
    if (dispatch == PSI_HIP_DISPATCH_AUTO) {
        // Row groups where they are the faster launch: a request brings more than one Q-token tile (the plain map
        // walks its KV range once per tile), or a tile more query columns than the multi-query pipeline holds.
        dispatch = PSI_HIP_DISPATCH_BALANCED;
        if (tiled && host->row_groups != nullptr && options->capacity_mode == PSI_HIP_CAPACITY_FIXED_PARTITION &&
            cfg->attention.num_kv_heads != 0) {
            uint32_t most = 0;
            for (uint32_t r = 0; r < num_reqs; ++r)
                if (cu_tokens[r + 1] > cu_tokens[r]) most = std::max(most, cu_tokens[r + 1] - cu_tokens[r]);
            const uint32_t heads = cfg->attention.num_q_heads / cfg->attention.num_kv_heads;
            uint32_t planned = 0;
            if (most > chosen.q_token_tile_size || most * heads > 48) {
                rc = psi_hip_split_kv_chunk_partition_tokens(&cfg->attention, chosen.q_token_tile_size, token_indices,
                                                             cu_tokens, num_reqs, 0, &planned);
                if (rc != PSI_HIP_OK) return rc;
            }
            if (planned != 0) {  // (0: no row-group kernel for the geometry)
                dispatch = PSI_HIP_DISPATCH_ROW_GROUPS;
                partition_tokens = planned;
            }
        }
    }
    if (dispatch == PSI_HIP_DISPATCH_ROW_GROUPS && !tiled) dispatch = PSI_HIP_DISPATCH_BALANCED;
    if (dispatch == PSI_HIP_DISPATCH_ROW_GROUPS && partition_tokens == 0 &&
        options->capacity_mode == PSI_HIP_CAPACITY_FIXED_PARTITION) {
        rc = psi_hip_split_kv_chunk_partition_tokens(&cfg->attention, chosen.q_token_tile_size, token_indices, cu_tokens,
                                                     num_reqs, 0, &partition_tokens);
        if (rc != PSI_HIP_OK) return rc;
        PSI_REQUIRE(partition_tokens != 0,
                    "GQA prepare: no row-group kernel for this geometry, so no partition length to plan; pass one");
    }
    uint32_t workers = 0;
    if (dispatch == PSI_HIP_DISPATCH_BALANCED || dispatch == PSI_HIP_DISPATCH_ROW_GROUPS) {
        workers = options->num_workers;
        if (workers == 0) {
            rc = psi_hip_split_kv_balanced_workers(&cfg->attention, &workers);
            if (rc != PSI_HIP_OK) return rc;
        }
    }
    // With a worker plan the planner's rows are an intermediate: they go to a side buffer and the re-cut rows to
    // the caller's array.
    thread_local std::vector<uint32_t> planned, planned_cu;
    const bool recut = dispatch == PSI_HIP_DISPATCH_BALANCED;
    uint32_t* plan_rows = host->kv_splits;
    uint32_t* plan_cu = host->cu_kv_splits;
    uint32_t plan_capacity = host->kv_splits_capacity;
    if (recut) {
        PSI_REQUIRE(host->worker_cu != nullptr && workers <= host->max_workers,
                    "GQA prepare: the worker table holds %u workers, the plan needs %u", host->max_workers, workers);
        PSI_REQUIRE(host->kv_splits_capacity > workers, "GQA prepare: kv_splits has no room for a worker plan");
        plan_capacity = host->kv_splits_capacity - workers;
        planned.resize((size_t)plan_capacity * 3);
        planned_cu.resize((size_t)host->max_tokens + 1);
        plan_rows = planned.data();
        plan_cu = planned_cu.data();
    }
    psi_hip_gqa_replay_shape shape;
    rc = psi_hip_gqa_metadata_update(host->max_tokens, req_slots, token_indices, cu_tokens, num_reqs, &chosen,
                                     options->capacity_mode, options->caller_num_total_tokens,
                                     options->topology_boundaries, options->num_boundaries, partition_tokens,
                                     plan_capacity, host->req_slots_by_token, host->flat_token_indices,
                                     host->q_token_tiles, plan_rows, plan_cu, &shape);
    if (rc != PSI_HIP_OK) return rc;
    uint32_t uses = 0, group_tiles = 0, num_groups = 0;
    if (dispatch == PSI_HIP_DISPATCH_ROW_GROUPS) {
        PSI_REQUIRE(host->row_groups != nullptr, "GQA prepare: row groups need their table");
        rc = psi_hip_split_kv_tiled_q_group_rows(&cfg->attention, chosen.q_token_tile_size, host->kv_splits,
                                                 shape.num_kv_splits, host->q_token_tiles, shape.num_q_token_tiles,
                                                 host->req_slots_by_token, host->row_groups, host->row_groups_capacity,
                                                 &group_tiles, &num_groups);
        if (rc != PSI_HIP_OK) return rc;
        if (num_groups != 0) uses |= 4u;
        // a geometry without the grouped kernel keeps the plain plan (one workgroup per row)
    } else if (recut) {
        uint32_t rows_out = 0;
        const uint32_t groups = tiled ? shape.num_q_token_tiles : shape.num_tokens;
        rc = psi_hip_split_kv_balance_plan(plan_rows, shape.num_kv_splits, plan_cu, groups, workers, host->kv_splits,
                                           host->kv_splits_capacity, host->cu_kv_splits, host->worker_cu, &rows_out);
        if (rc != PSI_HIP_OK) return rc;
        for (uint64_t i = (uint64_t)rows_out * 3; i < (uint64_t)host->kv_splits_capacity * 3; ++i)
            host->kv_splits[i] = PSI_HIP_SENTINEL;
        shape.num_kv_splits = shape.num_total_kv_splits = rows_out;
        shape.reduce_sdpa_partial_outputs = 1;
        uses |= 2u;
    } else if (dispatch == PSI_HIP_DISPATCH_LONGEST_FIRST) {
        PSI_REQUIRE(host->partial_row_index != nullptr, "GQA prepare: the dispatch order needs partial_row_index");
        for (uint32_t i = 0; i < host->kv_splits_capacity; ++i) host->partial_row_index[i] = i;
        rc = psi_hip_split_kv_order_longest_first(host->kv_splits, shape.num_kv_splits, host->partial_row_index);
        if (rc != PSI_HIP_OK) return rc;
        uses |= 1u;
    }
    if (options->bucket_capacities != 0 && options->capacity_mode == PSI_HIP_CAPACITY_FIXED_PARTITION) {
        // `ReplayBucketPolicy` capacities for the shape a replay cache keys its programs by (replay.rs:4-87): the
        // reference buckets its greedy plan the same way (batch_metadata.rs:277-294); here the row count being
        // bucketed is the dispatch plan's.
        uint32_t cap = 0;
        rc = psi_hip_replay_bucket_capacity(host->max_tokens, options->topology_boundaries, options->num_boundaries,
                                            shape.num_tokens, &cap);
        if (rc != PSI_HIP_OK) return rc;
        shape.num_total_tokens = cap;
        rc = psi_hip_replay_bucket_capacity(host->max_tokens, nullptr, 0, shape.num_q_token_tiles, &cap);
        if (rc != PSI_HIP_OK) return rc;
        shape.num_total_q_token_tiles = cap;
        rc = psi_hip_replay_bucket_capacity(host->kv_splits_capacity, nullptr, 0, shape.num_kv_splits, &cap);
        if (rc != PSI_HIP_OK) return rc;
        for (uint64_t i = (uint64_t)shape.num_kv_splits * 3; i < (uint64_t)cap * 3; ++i)
            host->kv_splits[i] = PSI_HIP_SENTINEL;
        shape.num_total_kv_splits = cap;
        if (num_groups != 0) {
            const uint64_t max_groups = host->row_groups_capacity / group_tiles;
            rc = psi_hip_replay_bucket_capacity((uint32_t)std::min<uint64_t>(max_groups, 0x7fffffffu), nullptr, 0,
                                                num_groups, &cap);
            if (rc != PSI_HIP_OK) return rc;
            for (uint64_t i = (uint64_t)num_groups * group_tiles; i < (uint64_t)cap * group_tiles; ++i)
                host->row_groups[i] = PSI_HIP_SENTINEL;  // a group without rows: its workgroups return at once
            num_groups = cap;
        }
    }
    uint32_t max_tile_tokens = 0;
    if (tiled) {
        for (uint32_t r = 0; r < num_reqs; ++r) {
            const uint32_t n = cu_tokens[r + 1] - cu_tokens[r];
            max_tile_tokens = n > max_tile_tokens ? n : max_tile_tokens;
        }
        if (max_tile_tokens > chosen.q_token_tile_size) max_tile_tokens = chosen.q_token_tile_size;
    }
    out_plan->shape = shape;
    out_plan->variant = chosen;
    out_plan->num_workers = (uses & 2u) ? workers : 0;
    out_plan->group_tiles = group_tiles;
    out_plan->num_row_groups = num_groups;
    out_plan->max_active_q_tile_tokens = max_tile_tokens;
    if (out_uses) *out_uses = uses;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_gqa_layer_advance_decode(const psi_hip_gqa_plan_options* options,
                                                const psi_hip_gqa_host_metadata* host,
                                                const psi_hip_gqa_batch_metadata* plan, uint32_t plan_uses,
                                                int* out_advanced) {
    PSI_REQUIRE(options && host && plan && out_advanced, "GQA advance: options, host arrays, plan and out_advanced must not be null");
    PSI_REQUIRE(host->req_slots_by_token && host->flat_token_indices && host->kv_splits && host->cu_kv_splits,
                "GQA advance: the metadata arrays must not be null");
    *out_advanced = 0;
    const uint32_t tokens = plan->shape.num_tokens;
    PSI_REQUIRE(tokens > 0 && tokens <= host->max_tokens, "GQA advance: the plan's token count does not fit the arrays");
    constexpr uint32_t kTile = 16;
    // Only plans whose rows follow from the tile counts alone, in an order that does not depend on the lengths.
    if (plan->variant.kind != PSI_HIP_VARIANT_SINGLE_Q || options->capacity_mode != PSI_HIP_CAPACITY_FIXED_PARTITION ||
        options->partition_tokens % kTile != 0 || (plan_uses & (1u | 4u)) != 0)
        return PSI_HIP_OK;
    const uint32_t* slots = host->req_slots_by_token;
    uint32_t* positions = host->flat_token_indices;
    uint32_t* rows = host->kv_splits;
    const uint32_t* cu = host->cu_kv_splits;
    for (uint32_t t = 0; t < tokens; ++t) {
        if (t > 0 && slots[t] == slots[t - 1]) return PSI_HIP_OK;  // several tokens of one request: not a decode batch
        const uint64_t context = (uint64_t)positions[t] + 1;
        if (context % kTile == 0 || context + 1 > 0xffffffffull) return PSI_HIP_OK;  // the next token starts a tile
        if (cu[t + 1] <= cu[t] || cu[t + 1] > host->kv_splits_capacity) return PSI_HIP_OK;
        const uint32_t* last = rows + (size_t)(cu[t + 1] - 1) * 3;
        if (last[0] != t || last[2] != context) return PSI_HIP_OK;  // not the table a preparation left here
    }
    for (uint32_t t = 0; t < tokens; ++t) {
        positions[t] += 1;
        rows[(size_t)(cu[t + 1] - 1) * 3 + 2] += 1;
    }
    *out_advanced = 1;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_gqa_layer_record(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg,
                                        const psi_hip_gqa_layer_input* input) {
    return record_layer(ctx, cfg, input);
}

extern "C" int psi_hip_gqa_layer_prepare_mixed(const psi_hip_gqa_layer_config* cfg,
                                               const psi_hip_gqa_plan_options* chunk_options,
                                               const psi_hip_gqa_plan_options* decode_options, uint32_t chunk_min_tokens,
                                               const uint32_t* req_slots, const uint32_t* token_indices,
                                               const uint32_t* cu_tokens, uint32_t num_reqs,
                                               const psi_hip_gqa_host_metadata* chunk_host,
                                               const psi_hip_gqa_host_metadata* decode_host,
                                               psi_hip_gqa_mixed_plan* out_plan) {
    PSI_REQUIRE(cfg && chunk_options && decode_options && out_plan, "GQA mixed prepare: config, options and out_plan must not be null");
    PSI_REQUIRE(req_slots && token_indices && cu_tokens && num_reqs > 0, "GQA prepare needs a batch");
    PSI_REQUIRE(cu_tokens[0] == 0, "GQA cu_tokens must start at zero");
    uint32_t n_chunk = 0;
    while (n_chunk < num_reqs && cu_tokens[n_chunk + 1] - cu_tokens[n_chunk] > chunk_min_tokens) ++n_chunk;
    for (uint32_t r = n_chunk; r < num_reqs; ++r)
        PSI_REQUIRE(cu_tokens[r + 1] >= cu_tokens[r] && cu_tokens[r + 1] - cu_tokens[r] <= chunk_min_tokens,
                    "GQA mixed batch: the requests with more than %u new tokens must come first (request %u)",
                    chunk_min_tokens, r);
    std::memset(out_plan, 0, sizeof(*out_plan));
    out_plan->num_chunk_reqs = n_chunk;
    out_plan->num_chunk_tokens = cu_tokens[n_chunk];
    int rc = PSI_HIP_OK;
    if (n_chunk > 0) {
        PSI_REQUIRE(chunk_host != nullptr, "GQA mixed prepare: the chunk part needs its host arrays");
        Geometry g;
        rc = make_geometry(&cfg->attention, &g);
        if (rc != PSI_HIP_OK) return rc;
        psi_hip_gqa_plan_options options = *chunk_options;
        options.dispatch = PSI_HIP_DISPATCH_ROW_GROUPS;
        const psi_hip_split_kv_variant tiled{PSI_HIP_VARIANT_TILED_Q, 8u, 16u, 0u, g.group < 8u ? g.group : 8u};
        rc = psi_hip_gqa_layer_prepare(cfg, &options, req_slots, token_indices, cu_tokens, n_chunk, &tiled, chunk_host,
                                       &out_plan->chunk, &out_plan->chunk_uses);
        if (rc != PSI_HIP_OK) return rc;
    }
    if (n_chunk < num_reqs) {
        PSI_REQUIRE(decode_host != nullptr, "GQA mixed prepare: the decode part needs its host arrays");
        thread_local std::vector<uint32_t> cu;
        cu.resize(num_reqs - n_chunk + 1);
        for (uint32_t r = n_chunk; r <= num_reqs; ++r) cu[r - n_chunk] = cu_tokens[r] - cu_tokens[n_chunk];
        rc = psi_hip_gqa_layer_prepare(cfg, decode_options, req_slots + n_chunk, token_indices + n_chunk, cu.data(),
                                       num_reqs - n_chunk, nullptr, decode_host, &out_plan->decode,
                                       &out_plan->decode_uses);
        if (rc != PSI_HIP_OK) return rc;
    }
    return PSI_HIP_OK;
}

// Bytes of one part's partial states, rounded up so that the next part starts on a 256-byte boundary.
static int mixed_part_bytes(const psi_hip_gqa_layer_config* cfg, const psi_hip_gqa_batch_metadata& md, uint64_t* out) {
    *out = 0;
    if (md.shape.num_tokens == 0) return PSI_HIP_OK;
    int rc = psi_hip_gqa_layer_scratch_bytes(cfg, &md.variant, md.shape.num_total_kv_splits, out);
    *out = (*out + 255) & ~uint64_t(255);
    return rc;
}

extern "C" int psi_hip_gqa_layer_mixed_scratch_bytes(const psi_hip_gqa_layer_config* cfg,
                                                     const psi_hip_gqa_mixed_plan* plan, uint64_t* out_bytes) {
    PSI_REQUIRE(cfg && plan && out_bytes, "GQA mixed scratch: config, plan and out pointer must not be null");
    uint64_t chunk = 0, decode = 0;
    int rc = mixed_part_bytes(cfg, plan->chunk, &chunk);
    if (rc != PSI_HIP_OK) return rc;
    rc = mixed_part_bytes(cfg, plan->decode, &decode);
    if (rc != PSI_HIP_OK) return rc;
    *out_bytes = chunk + decode;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_gqa_layer_record_mixed(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg,
                                              const psi_hip_gqa_layer_input* input, const psi_hip_gqa_mixed_plan* plan) {
    PSI_REQUIRE(ctx && cfg && input && plan, "ctx, config, input and plan must not be null");
    LayerPlan lp;
    int rc = make_layer_plan(cfg, &lp);
    if (rc != PSI_HIP_OK) return rc;
    const Geometry& g = lp.g;
    const bool has_chunk = plan->chunk.shape.num_tokens != 0, has_decode = plan->decode.shape.num_tokens != 0;
    PSI_REQUIRE(has_chunk || has_decode, "GQA mixed plan holds no tokens");
    PSI_REQUIRE(!has_chunk || plan->chunk.shape.num_tokens == plan->num_chunk_tokens,
                "GQA mixed plan: the chunk part's token count differs from num_chunk_tokens");
    uint64_t chunk_bytes = 0, decode_bytes = 0;
    rc = mixed_part_bytes(cfg, plan->chunk, &chunk_bytes);
    if (rc != PSI_HIP_OK) return rc;
    rc = mixed_part_bytes(cfg, plan->decode, &decode_bytes);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(input->partial_scratch != nullptr && input->partial_scratch_bytes >= chunk_bytes + decode_bytes,
                "GQA mixed scratch too small: %llu < %llu", (unsigned long long)input->partial_scratch_bytes,
                (unsigned long long)(chunk_bytes + decode_bytes));
    if (has_chunk) {
        psi_hip_gqa_layer_input part = *input;
        part.batch_metadata = &plan->chunk;
        part.partial_scratch_bytes = chunk_bytes;
        rc = record_layer(ctx, cfg, &part);
        if (rc != PSI_HIP_OK) return rc;
    }
    if (has_decode) {
        // the decode part's rows start behind the chunk part's: num_chunk_tokens rows of every per-token array
        const uint64_t skip = has_chunk ? plan->num_chunk_tokens : 0;
        const uint64_t q_row = (uint64_t)g.hq * g.d, kv_row = (uint64_t)g.hkv * g.d;
        const uint32_t out_elem = ctx->f32_output ? 4u : g.elem;
        auto rows_on = [&](const void* base, uint64_t row_elems, uint32_t elem) -> const void* {
            return base == nullptr ? nullptr : static_cast<const char*>(base) + skip * row_elems * elem;
        };
        psi_hip_gqa_layer_input part = *input;
        part.batch_metadata = &plan->decode;
        part.qgkv = rows_on(input->qgkv, lp.token_width, g.elem);
        part.q = rows_on(input->q, q_row, g.elem);
        part.k = rows_on(input->k, kv_row, g.elem);
        part.v = rows_on(input->v, kv_row, g.elem);
        part.g = rows_on(input->g, q_row, g.elem);
        part.q_norm_rope = const_cast<void*>(rows_on(input->q_norm_rope, q_row, g.elem));
        part.output = const_cast<void*>(rows_on(input->output, q_row, out_elem));
        part.partial_scratch = static_cast<char*>(input->partial_scratch) + chunk_bytes;
        part.partial_scratch_bytes = decode_bytes;
        rc = record_layer(ctx, cfg, &part);
        if (rc != PSI_HIP_OK) return rc;
    }
    return PSI_HIP_OK;
}

extern "C" int psi_hip_gqa_layer_record_static_scratch(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg,
                                                       const psi_hip_gqa_layer_input* input) {
    PSI_REQUIRE(ctx != nullptr && cfg != nullptr && input != nullptr && input->batch_metadata != nullptr,
                "ctx, config, input and batch metadata must not be null");
    PSI_REQUIRE(ctx->device >= 0 && ctx->device < kMaxStaticScratchDevices && g_static_scratch[ctx->device] != nullptr,
                "the static scratch of device %d was not resolved when the context was created", ctx->device);
    uint64_t need = 0;
    int rc = psi_hip_gqa_layer_scratch_bytes(cfg, &input->batch_metadata->variant,
                                             input->batch_metadata->shape.num_total_kv_splits, &need);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(need <= kStaticScratchBytes,
                "GQA partial states of %u KV splits need %llu bytes; the built-in scratch holds %llu (use "
                "psi_hip_gqa_layer_record with a buffer of your own)",
                input->batch_metadata->shape.num_total_kv_splits, (unsigned long long)need,
                (unsigned long long)kStaticScratchBytes);
    psi_hip_gqa_layer_input with_scratch = *input;
    with_scratch.partial_scratch = g_static_scratch[ctx->device];
    with_scratch.partial_scratch_bytes = kStaticScratchBytes;
    const bool timing_before = ctx->timing;
    ctx->timing = false;  // per-kernel timing creates events
    rc = record_layer(ctx, cfg, &with_scratch);
    ctx->timing = timing_before;
    return rc;
}

extern "C" int psi_hip_gqa_replay_cache_create(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg,
                                               uint32_t* device_counts, uint32_t max_programs,
                                               psi_hip_gqa_replay_cache** out_cache) {
    PSI_REQUIRE(ctx != nullptr && out_cache != nullptr, "ctx and out_cache must not be null");
    PSI_REQUIRE(device_counts != nullptr, "the replay cache needs a device count block (u32[4])");
    PSI_REQUIRE(max_programs > 0, "the replay cache must hold at least one program");
    LayerPlan plan;
    int rc = make_layer_plan(cfg, &plan);
    if (rc != PSI_HIP_OK) return rc;
    auto* cache = new psi_hip_gqa_replay_cache();
    cache->ctx = ctx;
    cache->cfg = *cfg;
    cache->device_counts = device_counts;
    cache->max_programs = max_programs;
    *out_cache = cache;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_gqa_replay_cache_destroy(psi_hip_gqa_replay_cache* cache) {
    if (cache == nullptr) return PSI_HIP_OK;
    for (auto& p : cache->programs)
        if (p.exec) (void)hipGraphExecDestroy(p.exec);
    delete cache;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_gqa_replay_cache_stats(const psi_hip_gqa_replay_cache* cache, uint32_t* programs,
                                              uint64_t* recordings, uint64_t* replays) {
    PSI_REQUIRE(cache != nullptr, "replay cache must not be null");
    if (programs) *programs = (uint32_t)cache->programs.size();
    if (recordings) *recordings = cache->recordings;
    if (replays) *replays = cache->replays;
    return PSI_HIP_OK;
}

// Records the layer at the capacities of `input` into a new program.
static int record_program(psi_hip_gqa_replay_cache* cache, const psi_hip_gqa_layer_input* input, hipGraphExec_t* out) {
    psi_hip_ctx* ctx = cache->ctx;
    // by-value counts = the capacities (they cut the grids and bound the device-side counts)
    psi_hip_gqa_batch_metadata md = *input->batch_metadata;
    md.shape.num_tokens = md.shape.num_total_tokens;
    md.shape.num_q_token_tiles = md.shape.num_total_q_token_tiles;
    md.shape.num_kv_splits = md.shape.num_total_kv_splits;
    psi_hip_gqa_layer_input at_capacity = *input;
    at_capacity.batch_metadata = &md;

    const uint32_t* bound_before = ctx->replay_counts;
    const bool timing_before = ctx->timing;
    ctx->replay_counts = md.replay_counts != nullptr ? md.replay_counts : cache->device_counts;
    ctx->timing = false;  // event records would become nodes of the program
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    int rc = PSI_HIP_OK;
    if (e != hipSuccess) {
        rc = fail(PSI_HIP_ERR_RUNTIME, "hipStreamBeginCapture failed: %s", hipGetErrorString(e));
    } else {
        rc = record_layer(ctx, &cache->cfg, &at_capacity);
        e = hipStreamEndCapture(ctx->stream, &graph);  // always ends the capture, also after a failed recording
        if (rc == PSI_HIP_OK && e != hipSuccess)
            rc = fail(PSI_HIP_ERR_RUNTIME, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
    }
    ctx->replay_counts = bound_before;
    ctx->timing = timing_before;
    if (rc == PSI_HIP_OK) {
        e = hipGraphInstantiate(out, graph, nullptr, nullptr, 0);
        if (e != hipSuccess) rc = fail(PSI_HIP_ERR_RUNTIME, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
    }
    if (graph) (void)hipGraphDestroy(graph);
    return rc;
}

extern "C" int psi_hip_gqa_replay_cache_submit(psi_hip_gqa_replay_cache* cache, const psi_hip_gqa_layer_input* input,
                                               uint32_t gqa_layer_parameter, int* out_recorded) {
    PSI_REQUIRE(cache != nullptr, "replay cache must not be null");
    psi_hip_ctx* ctx = cache->ctx;
    PSI_REQUIRE(ctx->stream != nullptr, "the replay cache records by stream capture: the context needs a created stream");
    int rc = check_input(input);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(gqa_layer_parameter <= input->page_table_layout.num_gqa_layers,
                "GQA page-table index exceeds layer count");
    if (out_recorded) *out_recorded = 0;
    const ProgramKey key = make_key(*ctx, *input, gqa_layer_parameter != 0);
    auto it = cache->programs.begin();
    for (; it != cache->programs.end(); ++it)
        if (std::memcmp(&it->key, &key, sizeof(key)) == 0) break;
    if (it == cache->programs.end()) {
        Program p;
        p.key = key;
        rc = record_program(cache, input, &p.exec);
        if (rc != PSI_HIP_OK) return rc;
        cache->programs.push_front(p);
        cache->recordings += 1;
        if (out_recorded) *out_recorded = 1;
        while (cache->programs.size() > cache->max_programs) {
            // a dropped program may still be running: wait for the stream before its nodes go away
            PSI_HIP_CHECK(hipStreamSynchronize(ctx->stream));
            (void)hipGraphExecDestroy(cache->programs.back().exec);
            cache->programs.pop_back();
        }
    } else if (it != cache->programs.begin()) {
        cache->programs.splice(cache->programs.begin(), cache->programs, it);
    }
    if (input->batch_metadata->replay_counts == nullptr) {
        // the counts the program reads: one small launch ahead of it (a caller that places them itself saves it)
        const psi_hip_gqa_replay_shape& s = input->batch_metadata->shape;
        hipLaunchKernelGGL(set_replay_counts_kernel, dim3(1), dim3(64), 0, ctx->stream, cache->device_counts,
                           s.num_tokens, s.num_q_token_tiles, s.num_kv_splits, gqa_layer_parameter);
        PSI_HIP_CHECK(hipGetLastError());
    }
    PSI_HIP_CHECK(hipGraphLaunch(cache->programs.front().exec, ctx->stream));
    cache->replays += 1;
    return PSI_HIP_OK;
}
