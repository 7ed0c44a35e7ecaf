// Kernels a gated GQA layer runs around the attention proper, and their C-ABI entry points:
//   QGKV split            crates/inference-backend-metal/src/components/metal/gqa_qgkv_split.metal:5-43
//   RMSNorm + RoPE        crates/inference-backend-metal/src/components/metal/rms_norm_rope.metal:7-82
//                         (host parameters: components/rms_norm_rope.rs:170-238)
//   sigmoid gate          crates/inference-backend-metal/src/components/metal/gqa_activation_gate.metal:13-38
// plus the K-side RMSNorm + RoPE fused into the KV append.  All of them move a few hundred KB per
// decode step: they are launch-latency bound, so the design goal is fewer launches and no extra
// round trip through HBM, not bandwidth.  One wave handles one (token, head) row.
#include <cmath>
#include <cstring>

#include "common.h"
#include "device_types.h"

namespace psi {

constexpr uint32_t kMaxRopeHalf = 128;  // rope_dim <= 256: the frequency table travels as a kernel argument

struct RopeTable {
    float inverse_frequencies[kMaxRopeHalf];
};

struct NormRopeArgs {
    const void* input;
    const uint16_t* norm_weight;
    const uint32_t* positions;
    void* output;
    uint64_t in_token_stride, in_head_stride;
    uint32_t num_active_tokens, num_heads, head_dim, rope_dim;
    float eps, attention_factor;
    const uint32_t* replay_counts = nullptr;  // see active_count()
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Normalises and rotates one row; `emit(d, value)` receives every output element once, value already
// in f32 and about to be rounded to the storage type by the caller.
template <typename Tag, typename Emit>
__device__ __forceinline__ void norm_rope_row(const void* row, const uint16_t* norm_weight, float position,
                                              uint32_t head_dim, uint32_t rope_dim, float eps, float attention_factor,
                                              const RopeTable& table, uint32_t lane, Emit emit) {
    float acc = 0.0f;
    for (uint32_t d = lane; d < head_dim; d += 64) {
        const float x = load_as_f32<Tag>(row, d);
        acc = fmaf(x, x, acc);
    }
    acc = wave_sum(acc);
    const float inv = 1.0f / sqrtf(acc / (float)head_dim + eps);
    const uint32_t half = rope_dim / 2;
    auto normalised = [&](uint32_t d) {
        return round_through<Tag>(round_through<Tag>(bf16_bits_to_f32(norm_weight[d])) *
                                  round_through<Tag>(load_as_f32<Tag>(row, d) * inv));
    };
    for (uint32_t d = lane; d < head_dim; d += 64) {
        if (d < half) {
            const float x1 = normalised(d), x2 = normalised(d + half);
            float s, c;
            sincosf(position * table.inverse_frequencies[d], &s, &c);
            emit(d, attention_factor * (x1 * c - x2 * s));
            emit(d + half, attention_factor * (x1 * s + x2 * c));
        } else if (d >= rope_dim) {
            emit(d, normalised(d));
        }
    }
}

template <typename Tag>
__global__ __launch_bounds__(256) void rms_norm_rope_kernel(NormRopeArgs a, RopeTable table) {
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t row = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= (uint64_t)active_count(a.replay_counts, kReplayTokens, a.num_active_tokens) * a.num_heads) return;
    const uint32_t token = (uint32_t)(row / a.num_heads), head = (uint32_t)(row % a.num_heads);
    const char* in = static_cast<const char*>(a.input) +
                     (token * a.in_token_stride + head * a.in_head_stride) * sizeof(typename Tag::storage);
    const uint64_t out_base = row * a.head_dim;
    norm_rope_row<Tag>(in, a.norm_weight, (float)a.positions[token], a.head_dim, a.rope_dim, a.eps,
                       a.attention_factor, table, lane,
                       [&](uint32_t d, float v) { store_from_f32<Tag>(a.output, out_base + d, v); });
}

struct FusedAppendArgs {
    void* pages;
    const void* raw_k;
    const void* flat_v;
    const uint16_t* norm_weight;
    const uint32_t* req_slots;
    const uint32_t* flat_token_indices;
    const uint32_t* page_ids;
    uint64_t k_token_stride, v_token_stride;
    uint32_t num_active, layer;
    uint32_t num_layers, num_blocks, ids_per_block;
    uint32_t hkv, d, tokens_per_page, rope_dim;
    uint64_t page_elems;
    float eps, attention_factor;
    const uint32_t* replay_counts = nullptr;  // see active_count()
};

// One wave per (token write, kv_head): the K row is normalised and rotated on its way into its page
// line, the V row is copied.  Page index contract of gqa_kv_page_write.metal:29-47.
template <typename Tag>
__device__ __forceinline__ void append_row(const FusedAppendArgs& a, const RopeTable& table, uint64_t item, uint32_t lane) {
    using Elem = typename Tag::storage;
    const uint32_t write = (uint32_t)(item / a.hkv), head = (uint32_t)(item % a.hkv);
    const uint32_t req_slot = a.req_slots[write];
    const uint32_t token = a.flat_token_indices[write];
    const uint32_t block = token / (a.tokens_per_page * a.ids_per_block);
    const uint32_t id_index = (token / a.tokens_per_page) % a.ids_per_block;
    const uint32_t page_token = token % a.tokens_per_page;
    const uint64_t table_index =
        (((uint64_t)req_slot * a.num_layers + active_layer(a.replay_counts, a.layer, a.num_layers)) * a.num_blocks + block) *
            a.ids_per_block +
        id_index;
    const uint64_t page_base = (uint64_t)a.page_ids[table_index] * a.page_elems;
    const uint64_t k_line = page_base + ((uint64_t)head * a.tokens_per_page + page_token) * a.d;
    const uint64_t v_line = page_base + ((uint64_t)(a.hkv + head) * a.tokens_per_page + page_token) * a.d;
    const Elem* k_row = static_cast<const Elem*>(a.raw_k) + write * a.k_token_stride + (uint64_t)head * a.d;
    const Elem* v_row = static_cast<const Elem*>(a.flat_v) + write * a.v_token_stride + (uint64_t)head * a.d;
    norm_rope_row<Tag>(k_row, a.norm_weight, (float)token, a.d, a.rope_dim, a.eps, a.attention_factor, table, lane,
                       [&](uint32_t d, float v) { store_from_f32<Tag>(a.pages, k_line + d, v); });
    Elem* v_dst = static_cast<Elem*>(a.pages) + v_line;
    for (uint32_t d = lane; d < a.d; d += 64) v_dst[d] = v_row[d];
}

template <typename Tag>
__global__ __launch_bounds__(256) void kv_page_write_norm_rope_kernel(FusedAppendArgs a, RopeTable table) {
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t item = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= (uint64_t)active_count(a.replay_counts, kReplayTokens, a.num_active) * a.hkv) return;
    append_row<Tag>(a, table, item, lane);
}

// The whole pre-attention step of a gated GQA layer in one launch: waves [0, T * Hq) normalise and
// rotate the query rows into the dense Q buffer, waves [T * Hq, T * (Hq + Hkv)) do the fused append.
template <typename Tag>
__global__ __launch_bounds__(256) void qk_norm_rope_append_kernel(NormRopeArgs q, FusedAppendArgs kv, RopeTable table) {
    using Elem = typename Tag::storage;
    const uint32_t lane = threadIdx.x & 63;
    const uint64_t wave_id = (uint64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    // the grid is cut for the capacity: Q rows first, then the K / V rows
    const uint64_t q_rows = (uint64_t)q.num_active_tokens * q.num_heads;
    const uint32_t active = active_count(q.replay_counts, kReplayTokens, q.num_active_tokens);
    if (wave_id < q_rows) {
        if (wave_id >= (uint64_t)active * q.num_heads) return;
        const uint32_t token = (uint32_t)(wave_id / q.num_heads), head = (uint32_t)(wave_id % q.num_heads);
        const char* in = static_cast<const char*>(q.input) +
                         (token * q.in_token_stride + head * q.in_head_stride) * sizeof(Elem);
        const uint64_t out_base = wave_id * q.head_dim;
        norm_rope_row<Tag>(in, q.norm_weight, (float)q.positions[token], q.head_dim, q.rope_dim, q.eps,
                           q.attention_factor, table, lane,
                           [&](uint32_t d, float v) { store_from_f32<Tag>(q.output, out_base + d, v); });
        return;
    }
    const uint64_t item = wave_id - q_rows;
    if (item >= (uint64_t)active * kv.hkv) return;
    append_row<Tag>(kv, table, item, lane);
}

template <typename Elem>
__global__ __launch_bounds__(256) void qgkv_split_kernel(const Elem* qgkv, Elem* q, Elem* g, Elem* k, Elem* v,
                                                         uint32_t num_active_tokens, uint32_t hq, uint32_t hkv,
                                                         uint32_t d, const uint32_t* replay_counts) {
    const uint64_t q_slots = (uint64_t)hq * d, kv_slots = (uint64_t)hkv * d;
    const uint64_t width = 2 * q_slots + 2 * kv_slots;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)active_count(replay_counts, kReplayTokens, num_active_tokens) * width) return;
    const uint64_t token = gid / width;
    uint64_t slot = gid - token * width;
    const Elem value = qgkv[gid];
    if (slot < 2 * q_slots) {
        const uint64_t pair = slot / (2 * d), in_pair = slot - pair * 2 * d;
        const uint64_t dst = (token * hq + pair) * d + in_pair % d;
        (in_pair < d ? q : g)[dst] = value;
        return;
    }
    slot -= 2 * q_slots;
    if (slot < kv_slots) {
        k[token * kv_slots + slot] = value;
        return;
    }
    v[token * kv_slots + slot - kv_slots] = value;
}

template <typename Tag>
__global__ __launch_bounds__(256) void activation_gate_kernel(const void* attention_output, const void* gates,
                                                              void* output, uint32_t num_active_tokens,
                                                              uint64_t per_token, const uint32_t* replay_counts) {
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= active_count(replay_counts, kReplayTokens, num_active_tokens) * per_token) return;
    store_from_f32<Tag>(output, gid,
                        load_as_f32<Tag>(attention_output, gid) * gate_sigmoid<Tag>(load_as_f32<Tag>(gates, gid)));
}

static int check_norm_config(const psi_hip_rms_norm_rope_config* cfg) {
    PSI_REQUIRE(cfg != nullptr, "RMSNorm/RoPE config must not be null");
    PSI_REQUIRE(cfg->num_heads > 0 && cfg->head_dim > 0, "RMSNorm/RoPE needs heads and a head_dim");
    PSI_REQUIRE(cfg->rope_dim > 0 && cfg->rope_dim <= cfg->head_dim && cfg->rope_dim % 2 == 0,
                "RMSNorm/RoPE rope_dim must be even and in 2..head_dim");
    PSI_REQUIRE(std::isfinite(cfg->eps) && cfg->eps > 0.0f, "RMSNorm/RoPE eps must be finite and positive");
    PSI_REQUIRE(std::isfinite(cfg->rope_theta) && cfg->rope_theta > 0.0f,
                "RMSNorm/RoPE rope_theta must be finite and positive");
    PSI_REQUIRE(cfg->dtype == PSI_HIP_F32 || cfg->dtype == PSI_HIP_BF16 || cfg->dtype == PSI_HIP_F16,
                "unsupported RMSNorm/RoPE dtype %u", cfg->dtype);
    const psi_hip_rope_scaling& s = cfg->scaling;
    PSI_REQUIRE(s.kind == PSI_HIP_ROPE_DEFAULT || s.kind == PSI_HIP_ROPE_YARN, "unknown RoPE scaling kind %u", s.kind);
    if (s.kind == PSI_HIP_ROPE_YARN) {
        PSI_REQUIRE(std::isfinite(s.factor) && s.factor >= 1.0f, "Yarn factor must be finite and >= 1");
        PSI_REQUIRE(std::isfinite(s.attention_factor) && s.attention_factor > 0.0f,
                    "Yarn attention_factor must be finite and positive");
        PSI_REQUIRE(std::isfinite(s.beta_fast) && s.beta_fast > 0.0f && std::isfinite(s.beta_slow) && s.beta_slow > 0.0f &&
                        s.beta_fast >= s.beta_slow,
                    "Yarn beta_fast >= beta_slow > 0 required");
        PSI_REQUIRE(s.original_max_position_embeddings > 0, "Yarn original_max_position_embeddings must be positive");
        PSI_REQUIRE(cfg->rope_theta > 1.0f, "Yarn rope_theta must be greater than 1");
    }
    return PSI_HIP_OK;
}

// rms_norm_rope.rs:170-238
static int rope_parameters(const psi_hip_rms_norm_rope_config* cfg, float* inverse_frequencies, float* attention_factor,
                           float* correction) {
    const psi_hip_rope_scaling& s = cfg->scaling;
    const bool yarn = s.kind == PSI_HIP_ROPE_YARN;
    float low = 0.0f, high = 0.0f;
    if (yarn) {
        auto bound = [&](float rotations) {
            const double dimension = cfg->rope_dim, base = cfg->rope_theta;
            const double original_length = s.original_max_position_embeddings;
            constexpr double kTau = 6.283185307179586476925286766559;
            return (float)(dimension * std::log(original_length / ((double)rotations * kTau)) / (2.0 * std::log(base)));
        };
        low = std::max(bound(s.beta_fast), 0.0f);
        high = std::min(bound(s.beta_slow), (float)(cfg->rope_dim - 1));
        if (s.truncate) {
            low = std::floor(low);
            high = std::ceil(high);
        }
        PSI_REQUIRE(low <= high, "Yarn correction range must be ordered");
        if (low == high) high += 0.001f;
        if (correction != nullptr) {
            correction[0] = low;
            correction[1] = high;
        }
    }
    const uint32_t half = cfg->rope_dim / 2;
    for (uint32_t d = 0; d < half; ++d) {
        float inv = std::pow(cfg->rope_theta, -((float)d / (float)half));
        if (yarn) {
            const float ramp = std::min(std::max(((float)d - low) / (high - low), 0.0f), 1.0f);
            inv *= 1.0f + ramp * (1.0f / s.factor - 1.0f);
        }
        PSI_REQUIRE(std::isfinite(inv) && inv > 0.0f, "RMSNorm/RoPE inverse frequency must be finite and positive");
        inverse_frequencies[d] = inv;
    }
    *attention_factor = yarn ? s.attention_factor : 1.0f;
    return PSI_HIP_OK;
}

static int fill_table(const psi_hip_rms_norm_rope_config* cfg, RopeTable* table, float* attention_factor) {
    PSI_REQUIRE(cfg->rope_dim / 2 <= kMaxRopeHalf, "RMSNorm/RoPE rope_dim above %u is not built", 2 * kMaxRopeHalf);
    for (float& f : table->inverse_frequencies) f = 0.0f;
    return rope_parameters(cfg, table->inverse_frequencies, attention_factor, nullptr);
}

}  // namespace psi

using namespace psi;

extern "C" int psi_hip_rope_parameters(const psi_hip_rms_norm_rope_config* cfg, float* out_inverse_frequencies,
                                       float* out_attention_factor, float* out_correction) {
    int rc = check_norm_config(cfg);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_inverse_frequencies && out_attention_factor, "out pointers must not be null");
    return rope_parameters(cfg, out_inverse_frequencies, out_attention_factor, out_correction);
}

// Validates one RMSNorm + RoPE operand set and fills the kernel arguments (everything but the table).
static int make_norm_args(const psi_hip_rms_norm_rope_config* cfg, const void* input, uint64_t input_token_stride,
                          uint64_t input_head_stride, const void* norm_weight, const uint32_t* flat_token_indices,
                          void* output, uint32_t num_total_tokens, uint32_t num_active_tokens, NormRopeArgs* a) {
    PSI_REQUIRE(input && norm_weight && flat_token_indices && output, "RMSNorm/RoPE buffers must not be null");
    PSI_REQUIRE(num_total_tokens > 0, "RMSNorm/RoPE requires tokens");
    PSI_REQUIRE(num_active_tokens > 0 && num_active_tokens <= num_total_tokens,
                "RMSNorm/RoPE active token count must be in 1..capacity");
    PSI_REQUIRE((uint64_t)num_total_tokens * cfg->num_heads * cfg->head_dim - 1 <= UINT32_MAX,
                "RMSNorm/RoPE elements exceeds the shader u32 element-index domain");
    PSI_REQUIRE((input_token_stride == 0) == (input_head_stride == 0),
                "RMSNorm/RoPE input strides must both be given or both be 0 (dense)");
    a->input = input;
    a->norm_weight = static_cast<const uint16_t*>(norm_weight);
    a->positions = flat_token_indices;
    a->output = output;
    a->in_head_stride = input_head_stride ? input_head_stride : cfg->head_dim;
    a->in_token_stride = input_token_stride ? input_token_stride : (uint64_t)cfg->num_heads * cfg->head_dim;
    PSI_REQUIRE(a->in_head_stride >= cfg->head_dim &&
                    a->in_token_stride >= (uint64_t)(cfg->num_heads - 1) * a->in_head_stride + cfg->head_dim,
                "RMSNorm/RoPE input strides overlap rows");
    a->num_active_tokens = num_active_tokens;
    a->num_heads = cfg->num_heads;
    a->head_dim = cfg->head_dim;
    a->rope_dim = cfg->rope_dim;
    a->eps = cfg->eps;
    return PSI_HIP_OK;
}

// Validates the operands of the fused append and fills its kernel arguments (everything but the table).
static int make_append_args(const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
                            const psi_hip_rms_norm_rope_config* norm_cfg, void* pages, uint64_t pages_bytes,
                            const void* raw_k, uint64_t k_token_stride, const void* flat_v, uint64_t v_token_stride,
                            const void* norm_weight, const uint32_t* req_slots, const uint32_t* flat_token_indices,
                            const uint32_t* page_ids, uint32_t num_total_token_writes,
                            uint32_t num_active_token_writes, uint32_t gqa_layer_index, Geometry* g,
                            FusedAppendArgs* a) {
    int rc = make_geometry(cfg, g);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_layout(layout);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(norm_cfg->num_heads == g->hkv && norm_cfg->head_dim == g->d && norm_cfg->dtype == g->dtype,
                "fused append: the K norm config must match the page geometry (%u heads of %u, dtype %u)", g->hkv,
                g->d, g->dtype);
    PSI_REQUIRE(pages && raw_k && flat_v && norm_weight && req_slots && flat_token_indices && page_ids,
                "GQA KV page write buffers must not be null");
    PSI_REQUIRE(gqa_layer_index < layout->num_gqa_layers, "GQA page-table index exceeds layer count");
    PSI_REQUIRE(num_total_token_writes > 0, "GQA KV page write requires tokens");
    PSI_REQUIRE(num_active_token_writes > 0 && num_active_token_writes <= num_total_token_writes,
                "GQA KV page write active token count must be in 1..capacity");
    PSI_REQUIRE(pages_bytes == 0 || pages_bytes >= cfg->page_bytes, "GQA page arena is smaller than one page");
    const uint64_t dense = (uint64_t)g->hkv * g->d;
    PSI_REQUIRE((k_token_stride == 0 || k_token_stride >= dense) && (v_token_stride == 0 || v_token_stride >= dense),
                "fused append: token strides must cover a token's K / V rows");
    a->pages = pages;
    a->raw_k = raw_k;
    a->flat_v = flat_v;
    a->norm_weight = static_cast<const uint16_t*>(norm_weight);
    a->req_slots = req_slots;
    a->flat_token_indices = flat_token_indices;
    a->page_ids = page_ids;
    a->k_token_stride = k_token_stride ? k_token_stride : dense;
    a->v_token_stride = v_token_stride ? v_token_stride : dense;
    a->num_active = num_active_token_writes;
    a->layer = gqa_layer_index;
    a->num_layers = layout->num_gqa_layers;
    a->num_blocks = layout->num_blocks;
    a->ids_per_block = layout->num_page_ids_per_block;
    a->hkv = g->hkv;
    a->d = g->d;
    a->tokens_per_page = g->tokens_per_page;
    a->rope_dim = norm_cfg->rope_dim;
    a->page_elems = g->page_elems;
    a->eps = norm_cfg->eps;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_rms_norm_rope(psi_hip_ctx* ctx, const psi_hip_rms_norm_rope_config* cfg, const void* input,
                                     uint64_t input_token_stride, uint64_t input_head_stride,
                                     const void* norm_weight, const uint32_t* flat_token_indices, void* output,
                                     uint32_t num_total_tokens, uint32_t num_active_tokens) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    int rc = check_norm_config(cfg);
    if (rc != PSI_HIP_OK) return rc;
    NormRopeArgs a;
    rc = make_norm_args(cfg, input, input_token_stride, input_head_stride, norm_weight, flat_token_indices, output,
                        num_total_tokens, num_active_tokens, &a);
    if (rc != PSI_HIP_OK) return rc;
    a.replay_counts = ctx->replay_counts;
    RopeTable table;
    rc = fill_table(cfg, &table, &a.attention_factor);
    if (rc != PSI_HIP_OK) return rc;
    const uint64_t rows = (uint64_t)num_active_tokens * cfg->num_heads;
    const dim3 grid((uint32_t)((rows + 3) / 4)), block(256);
    LaunchScope scope(ctx, "rms_norm_rope");
    if (cfg->dtype == PSI_HIP_F32) hipLaunchKernelGGL(rms_norm_rope_kernel<F32Tag>, grid, block, 0, ctx->stream, a, table);
    else if (cfg->dtype == PSI_HIP_BF16) hipLaunchKernelGGL(rms_norm_rope_kernel<BF16Tag>, grid, block, 0, ctx->stream, a, table);
    else hipLaunchKernelGGL(rms_norm_rope_kernel<F16Tag>, grid, block, 0, ctx->stream, a, table);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_kv_page_write_norm_rope(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                               const psi_hip_page_table_layout* layout,
                                               const psi_hip_rms_norm_rope_config* norm_cfg, void* pages,
                                               uint64_t pages_bytes, const void* raw_k, uint64_t k_token_stride,
                                               const void* flat_v, uint64_t v_token_stride, const void* norm_weight,
                                               const uint32_t* req_slots, const uint32_t* flat_token_indices,
                                               const uint32_t* page_ids, uint32_t num_total_token_writes,
                                               uint32_t num_active_token_writes, uint32_t gqa_layer_index) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    int rc = check_norm_config(norm_cfg);
    if (rc != PSI_HIP_OK) return rc;
    Geometry g;
    FusedAppendArgs a;
    rc = make_append_args(cfg, layout, norm_cfg, pages, pages_bytes, raw_k, k_token_stride, flat_v, v_token_stride,
                          norm_weight, req_slots, flat_token_indices, page_ids, num_total_token_writes,
                          num_active_token_writes, gqa_layer_index, &g, &a);
    if (rc != PSI_HIP_OK) return rc;
    a.replay_counts = ctx->replay_counts;
    RopeTable table;
    rc = fill_table(norm_cfg, &table, &a.attention_factor);
    if (rc != PSI_HIP_OK) return rc;
    const uint64_t items = (uint64_t)num_active_token_writes * g.hkv;
    PSI_REQUIRE((items + 3) / 4 <= 0x7fffffffull, "GQA KV page write grid exceeds the launch domain");
    const dim3 grid((uint32_t)((items + 3) / 4)), block(256);
    LaunchScope scope(ctx, "kv_page_write");
    if (g.dtype == PSI_HIP_F32) hipLaunchKernelGGL(kv_page_write_norm_rope_kernel<F32Tag>, grid, block, 0, ctx->stream, a, table);
    else if (g.dtype == PSI_HIP_BF16) hipLaunchKernelGGL(kv_page_write_norm_rope_kernel<BF16Tag>, grid, block, 0, ctx->stream, a, table);
    else hipLaunchKernelGGL(kv_page_write_norm_rope_kernel<F16Tag>, grid, block, 0, ctx->stream, a, table);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_qk_norm_rope_kv_page_write(
    psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
    const psi_hip_rms_norm_rope_config* q_norm_cfg, const psi_hip_rms_norm_rope_config* k_norm_cfg, const void* raw_q,
    uint64_t q_token_stride, uint64_t q_head_stride, const void* q_norm_weight, void* q_output, void* pages,
    uint64_t pages_bytes, const void* raw_k, uint64_t k_token_stride, const void* flat_v, uint64_t v_token_stride,
    const void* k_norm_weight, const uint32_t* req_slots, const uint32_t* flat_token_indices, const uint32_t* page_ids,
    uint32_t num_total_tokens, uint32_t num_active_tokens, uint32_t gqa_layer_index) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    int rc = check_norm_config(q_norm_cfg);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_norm_config(k_norm_cfg);
    if (rc != PSI_HIP_OK) return rc;
    Geometry g;
    FusedAppendArgs kv;
    rc = make_append_args(cfg, layout, k_norm_cfg, pages, pages_bytes, raw_k, k_token_stride, flat_v, v_token_stride,
                          k_norm_weight, req_slots, flat_token_indices, page_ids, num_total_tokens, num_active_tokens,
                          gqa_layer_index, &g, &kv);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(q_norm_cfg->num_heads == g.hq && q_norm_cfg->head_dim == g.d && q_norm_cfg->dtype == g.dtype,
                "the Q norm config must match the attention geometry (%u heads of %u, dtype %u)", g.hq, g.d, g.dtype);
    // one rotation table serves both operands
    PSI_REQUIRE(q_norm_cfg->rope_dim == k_norm_cfg->rope_dim && q_norm_cfg->rope_theta == k_norm_cfg->rope_theta &&
                    std::memcmp(&q_norm_cfg->scaling, &k_norm_cfg->scaling, sizeof(psi_hip_rope_scaling)) == 0,
                "the Q and K norm configs must share rope_dim, rope_theta and scaling");
    NormRopeArgs qa;
    rc = make_norm_args(q_norm_cfg, raw_q, q_token_stride, q_head_stride, q_norm_weight, flat_token_indices, q_output,
                        num_total_tokens, num_active_tokens, &qa);
    if (rc != PSI_HIP_OK) return rc;
    qa.replay_counts = ctx->replay_counts;
    RopeTable table;
    rc = fill_table(k_norm_cfg, &table, &kv.attention_factor);
    if (rc != PSI_HIP_OK) return rc;
    qa.attention_factor = kv.attention_factor;
    const uint64_t waves = (uint64_t)num_active_tokens * (g.hq + g.hkv);
    PSI_REQUIRE((waves + 3) / 4 <= 0x7fffffffull, "GQA prepare grid exceeds the launch domain");
    const dim3 grid((uint32_t)((waves + 3) / 4)), block(256);
    LaunchScope scope(ctx, "qk_norm_rope_kv_page_write");
    if (g.dtype == PSI_HIP_F32) hipLaunchKernelGGL(qk_norm_rope_append_kernel<F32Tag>, grid, block, 0, ctx->stream, qa, kv, table);
    else if (g.dtype == PSI_HIP_BF16) hipLaunchKernelGGL(qk_norm_rope_append_kernel<BF16Tag>, grid, block, 0, ctx->stream, qa, kv, table);
    else hipLaunchKernelGGL(qk_norm_rope_append_kernel<F16Tag>, grid, block, 0, ctx->stream, qa, kv, table);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_qgkv_split(psi_hip_ctx* ctx, uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim,
                                  uint32_t dtype, const void* qgkv, void* q, void* g, void* k, void* v,
                                  uint32_t num_total_tokens, uint32_t num_active_tokens) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    PSI_REQUIRE(num_q_heads > 0 && num_kv_heads > 0 && head_dim > 0, "GQA QGKV split needs heads and a head_dim");
    PSI_REQUIRE(dtype == PSI_HIP_F32 || dtype == PSI_HIP_BF16 || dtype == PSI_HIP_F16, "unsupported GQA QGKV split dtype %u",
                dtype);
    PSI_REQUIRE(qgkv && q && g && k && v, "GQA QGKV split buffers must not be null");
    PSI_REQUIRE(num_total_tokens > 0, "GQA QGKV split requires tokens");
    PSI_REQUIRE(num_active_tokens > 0 && num_active_tokens <= num_total_tokens,
                "GQA QGKV split active token count must be in 1..capacity");
    const uint64_t width = 2ull * ((uint64_t)num_q_heads + num_kv_heads) * head_dim;
    PSI_REQUIRE((uint64_t)num_total_tokens * width <= UINT32_MAX, "GQA QGKV split exceeds the shader u32 count domain");
    const uint64_t count = (uint64_t)num_active_tokens * width;
    const dim3 grid((uint32_t)((count + 255) / 256)), block(256);
    LaunchScope scope(ctx, "qgkv_split");
    if (dtype == PSI_HIP_F32)
        hipLaunchKernelGGL(qgkv_split_kernel<float>, grid, block, 0, ctx->stream, static_cast<const float*>(qgkv),
                           static_cast<float*>(q), static_cast<float*>(g), static_cast<float*>(k), static_cast<float*>(v),
                           num_active_tokens, num_q_heads, num_kv_heads, head_dim, ctx->replay_counts);
    else
        hipLaunchKernelGGL(qgkv_split_kernel<uint16_t>, grid, block, 0, ctx->stream, static_cast<const uint16_t*>(qgkv),
                           static_cast<uint16_t*>(q), static_cast<uint16_t*>(g), static_cast<uint16_t*>(k),
                           static_cast<uint16_t*>(v), num_active_tokens, num_q_heads, num_kv_heads, head_dim,
                           ctx->replay_counts);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

extern "C" int psi_hip_activation_gate(psi_hip_ctx* ctx, uint32_t num_q_heads, uint32_t head_dim, uint32_t dtype,
                                       const void* attention_output, const void* gates, void* output,
                                       uint32_t num_total_tokens, uint32_t num_active_tokens) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    PSI_REQUIRE(num_q_heads > 0 && head_dim > 0, "GQA activation gate needs heads and a head_dim");
    PSI_REQUIRE(dtype == PSI_HIP_F32 || dtype == PSI_HIP_BF16 || dtype == PSI_HIP_F16,
                "unsupported GQA activation gate dtype %u", dtype);
    PSI_REQUIRE(attention_output && gates && output, "GQA activation gate buffers must not be null");
    PSI_REQUIRE(num_total_tokens > 0, "GQA activation gate requires tokens");
    PSI_REQUIRE(num_active_tokens > 0 && num_active_tokens <= num_total_tokens,
                "GQA activation-gate active token count must be in 1..capacity");
    PSI_REQUIRE((uint64_t)num_total_tokens * num_q_heads * head_dim <= UINT32_MAX,
                "GQA activation/gate exceeds the shader u32 count domain");
    const uint64_t count = (uint64_t)num_active_tokens * num_q_heads * head_dim;
    const dim3 grid((uint32_t)((count + 255) / 256)), block(256);
    LaunchScope scope(ctx, "activation_gate");
    const uint64_t per_token = (uint64_t)num_q_heads * head_dim;
    if (dtype == PSI_HIP_F32) hipLaunchKernelGGL(activation_gate_kernel<F32Tag>, grid, block, 0, ctx->stream, attention_output, gates, output, num_active_tokens, per_token, ctx->replay_counts);
    else if (dtype == PSI_HIP_BF16) hipLaunchKernelGGL(activation_gate_kernel<BF16Tag>, grid, block, 0, ctx->stream, attention_output, gates, output, num_active_tokens, per_token, ctx->replay_counts);
    else hipLaunchKernelGGL(activation_gate_kernel<F16Tag>, grid, block, 0, ctx->stream, attention_output, gates, output, num_active_tokens, per_token, ctx->replay_counts);
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}
