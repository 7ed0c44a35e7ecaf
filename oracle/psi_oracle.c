/*
 * psi_oracle.c -- CPU restatement of the reference's paged KV-cache attention path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or calls this file;
 * it exists so that tests, the smoke check and the bench's CPU-baseline leg can compare the
 * HIP path with the arithmetic the reference defines.  Plain C, sequential f32 sums in the
 * reference's order, no fast-math.
 *
 * Every function cites the reference source it follows (paths relative to the reference root).
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   psi_oracle_softmax          closed form softmax([0, ln 3]) = [.25, .75]
 *                               (crates/inference-executor-core/src/reference.rs:103-108)
 *   psi_oracle_projected_gqa    the 2-token causal known answer
 *                               (crates/inference-executor-core/src/attn/gqa/reference.rs:84-115),
 *                               float64 brute force on tiny inputs, split/permutation invariants
 *   psi_oracle_kv_page_write    page known answers [0,0,10,11,0,0,20,21] and the 0x7777 canary case
 *                               (crates/inference-backend-metal/src/components/gqa_kv_page_write.rs:283-364)
 *   psi_oracle_gather_context   the reference tests' independent page packer
 *                               (crates/inference-backend-metal/src/components/gqa_split_kv_single_q_test.rs:397-424)
 *   bf16 / f16 conversions      exhaustive 65536-pattern round trip + known bit patterns
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define PSI_ORACLE_F32 0u
#define PSI_ORACLE_BF16 1u
#define PSI_ORACLE_F16 2u

/* ---------------------------------------------------------------- dtype conversion */

static inline uint32_t f32_bits(float v) {
    uint32_t b;
    memcpy(&b, &v, 4);
    return b;
}
static inline float bits_f32(uint32_t b) {
    float v;
    memcpy(&v, &b, 4);
    return v;
}

/* Round-to-nearest-even f32 -> bf16, NaN kept quiet (the behaviour of `half::bf16::from_f32`,
 * which the reference's tests use: gqa_split_kv_tiled_q_test.rs:280-316). */
uint16_t psi_oracle_f32_to_bf16(float v) {
    uint32_t b = f32_bits(v);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x0040u);
    uint32_t round = 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)((b + round) >> 16);
}
float psi_oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* IEEE binary16 <-> binary32, round-to-nearest-even, subnormals kept. */
uint16_t psi_oracle_f32_to_f16(float v) {
    uint32_t b = f32_bits(v);
    uint32_t sign = (b >> 16) & 0x8000u;
    uint32_t a = b & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((a >> 13) & 0x3ffu));
    if (a >= 0x47800000u) return (uint16_t)(sign | 0x7c00u); /* >= 65536 or inf */
    if (a >= 0x38800000u) {                                   /* normal half */
        uint32_t mant = a & 0x7fffffu;
        uint32_t exp = (a >> 23) - 112u;
        uint32_t h = (exp << 10) | (mant >> 13);
        uint32_t rem = mant & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
        return (uint16_t)(sign | h);
    }
    if (a < 0x33000000u) return (uint16_t)sign; /* rounds to zero */
    /* subnormal half: value = mant24 * 2^(e-150), unit = 2^-24 */
    uint32_t e = a >> 23;
    uint32_t mant = (a & 0x7fffffu) | 0x800000u;
    uint32_t shift = 126u - e; /* 14..24 */
    uint32_t h = mant >> shift;
    uint32_t rem = mant & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1u);
    if (rem > half || (rem == half && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}
float psi_oracle_f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t mant = h & 0x3ffu;
    if (exp == 0x1fu) return bits_f32(sign | 0x7f800000u | (mant << 13));
    if (exp != 0) return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
    if (mant == 0) return bits_f32(sign);
    float v = (float)mant * 5.9604644775390625e-08f; /* 2^-24 */
    return sign ? -v : v;
}

static size_t dtype_size(uint32_t dtype) { return dtype == PSI_ORACLE_F32 ? 4u : 2u; }

static float load_elem(const void* base, uint64_t index, uint32_t dtype) {
    if (dtype == PSI_ORACLE_F32) return ((const float*)base)[index];
    uint16_t h = ((const uint16_t*)base)[index];
    return dtype == PSI_ORACLE_BF16 ? psi_oracle_bf16_to_f32(h) : psi_oracle_f16_to_f32(h);
}

void psi_oracle_convert_from_f32(const float* src, void* dst, uint64_t count, uint32_t dtype) {
    for (uint64_t i = 0; i < count; ++i) {
        if (dtype == PSI_ORACLE_F32) ((float*)dst)[i] = src[i];
        else if (dtype == PSI_ORACLE_BF16) ((uint16_t*)dst)[i] = psi_oracle_f32_to_bf16(src[i]);
        else ((uint16_t*)dst)[i] = psi_oracle_f32_to_f16(src[i]);
    }
}
void psi_oracle_convert_to_f32(const void* src, float* dst, uint64_t count, uint32_t dtype) {
    for (uint64_t i = 0; i < count; ++i) dst[i] = load_elem(src, i, dtype);
}

/* ---------------------------------------------------------------- attention math */

/* crates/inference-executor-core/src/reference.rs:15-31 (softmax_reference):
 * max by left fold from -inf, weights exp(l - max), sequential f32 total, divide.
 * Returns -1 where the reference asserts (empty input, total not finite-positive). */
int psi_oracle_softmax(const float* logits, uint64_t n, float* out) {
    if (n == 0) return -1;
    float max_logit = -INFINITY;
    for (uint64_t i = 0; i < n; ++i) max_logit = fmaxf(max_logit, logits[i]);
    float total = 0.0f;
    for (uint64_t i = 0; i < n; ++i) {
        out[i] = expf(logits[i] - max_logit);
        total += out[i];
    }
    if (!(total > 0.0f) || !isfinite(total)) return -1;
    for (uint64_t i = 0; i < n; ++i) out[i] = out[i] / total;
    return 0;
}

/* One (token, q_head) row of crates/inference-executor-core/src/attn/gqa/reference.rs:43-73:
 * logits over the visible context (sequential dot over head_dim, then * scale), softmax,
 * then for every head_dim index a sequential sum over the context of p * v. */
static int attend_row(const float* q_row, const float* ctx_k, const float* ctx_v, uint64_t visible,
                      uint32_t num_kv_heads, uint32_t kv_head, uint32_t head_dim, float scale,
                      float* logits, float* probs, float* out_row) {
    for (uint64_t t = 0; t < visible; ++t) {
        const float* k = ctx_k + (t * num_kv_heads + kv_head) * head_dim;
        float dot = 0.0f;
        for (uint32_t d = 0; d < head_dim; ++d) dot += q_row[d] * k[d];
        logits[t] = dot * scale;
    }
    if (psi_oracle_softmax(logits, visible, probs) != 0) return -1;
    for (uint32_t d = 0; d < head_dim; ++d) {
        float weighted = 0.0f;
        for (uint64_t t = 0; t < visible; ++t)
            weighted += probs[t] * ctx_v[(t * num_kv_heads + kv_head) * head_dim + d];
        out_row[d] = weighted;
    }
    return 0;
}

/* crates/inference-executor-core/src/attn/gqa/reference.rs:15-78 (projected_gqa_reference).
 * q, out: [total_tokens, num_q_heads, head_dim] f32; ctx_k[r], ctx_v[r]: dense
 * [token_indices[r] + n_r, num_kv_heads, head_dim] f32.  Token i of request r sees
 * token_indices[r] + i + 1 context tokens.  num_threads > 1 spreads independent (token, head)
 * rows over threads; each row's arithmetic order is unchanged so results are bit-identical. */
int psi_oracle_projected_gqa(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim, float scale,
                             uint32_t num_reqs, const uint32_t* cu_tokens, const uint32_t* token_indices,
                             const float* q, const float* const* ctx_k, const float* const* ctx_v, float* out,
                             int num_threads) {
    if (num_q_heads == 0 || num_kv_heads == 0 || head_dim == 0 || num_q_heads % num_kv_heads != 0) return -1;
    if (!(scale > 0.0f)) return -1;
    if (cu_tokens[0] != 0) return -1;
    for (uint32_t r = 0; r < num_reqs; ++r)
        if (cu_tokens[r] > cu_tokens[r + 1]) return -1;
    const uint32_t group = num_q_heads / num_kv_heads;
    int status = 0;
    for (uint32_t r = 0; r < num_reqs; ++r) {
        const uint32_t req_start = cu_tokens[r], n_r = cu_tokens[r + 1] - cu_tokens[r];
        const uint64_t max_visible = (uint64_t)token_indices[r] + n_r;
        const int64_t rows = (int64_t)n_r * num_q_heads;
        if (num_threads < 1) num_threads = 1;
#pragma omp parallel num_threads(num_threads)
        {
            float* logits = (float*)malloc(sizeof(float) * (max_visible ? max_visible : 1));
            float* probs = (float*)malloc(sizeof(float) * (max_visible ? max_visible : 1));
#pragma omp for schedule(dynamic, 1)
            for (int64_t row = 0; row < rows; ++row) {
                uint32_t i = (uint32_t)(row / num_q_heads), h = (uint32_t)(row % num_q_heads);
                uint64_t token = (uint64_t)req_start + i;
                uint64_t visible = (uint64_t)token_indices[r] + i + 1;
                int rc = attend_row(q + (token * num_q_heads + h) * head_dim, ctx_k[r], ctx_v[r], visible,
                                    num_kv_heads, h / group, head_dim, scale, logits, probs,
                                    out + (token * num_q_heads + h) * head_dim);
                if (rc != 0) {
#pragma omp atomic write
                    status = -1;
                }
            }
            free(logits);
            free(probs);
        }
    }
    return status;
}

/* ---------------------------------------------------------------- page layout */

/* Index math of crates/inference-backend-metal/src/components/metal/gqa_kv_page_write.metal:29-47
 * (the same expressions reappear in gqa_split_kv_single_q_map.metal:96-111).  Returns the element
 * offset of (kind, kv_head, token, dim 0) in the page arena; kind 0 = K, 1 = V. */
static uint64_t page_elem_offset(const uint32_t* page_ids, uint32_t req_slot, uint32_t layer, uint32_t token,
                                 uint32_t num_gqa_layers, uint32_t num_blocks, uint32_t ids_per_block,
                                 uint32_t tokens_per_page, uint64_t page_elems, uint32_t num_kv_heads,
                                 uint32_t head_dim, uint32_t kind, uint32_t kv_head) {
    uint32_t block_index = token / (tokens_per_page * ids_per_block);
    uint32_t page_id_index = (token / tokens_per_page) % ids_per_block;
    uint32_t page_token = token % tokens_per_page;
    uint64_t table_index =
        (((uint64_t)req_slot * num_gqa_layers + layer) * num_blocks + block_index) * ids_per_block + page_id_index;
    uint64_t page_id = page_ids[table_index];
    return page_id * page_elems +
           (((uint64_t)kind * num_kv_heads + kv_head) * tokens_per_page + page_token) * head_dim;
}

/* crates/inference-backend-metal/src/components/gqa_kv_page_write.rs:57-70: tokens per page =
 * page_bytes / (2 * num_kv_heads * head_dim * elem), and it must divide exactly. */
int psi_oracle_tokens_per_page(uint32_t num_kv_heads, uint32_t head_dim, uint32_t page_bytes, uint32_t dtype,
                               uint32_t* out) {
    uint64_t per_token = (uint64_t)num_kv_heads * head_dim * 2u * dtype_size(dtype);
    if (per_token == 0 || per_token > UINT32_MAX || page_bytes % per_token != 0) return -1;
    *out = (uint32_t)(page_bytes / per_token);
    return *out > 0 ? 0 : -1;
}

/* crates/inference-backend-metal/src/components/metal/gqa_kv_page_write.metal:5-53: for every
 * active write w, kv head and dim, copy flat_k/flat_v[(w*Hkv + head)*D + d] bit-for-bit into the
 * K / V slot of the page the table names for (req_slots[w], layer, flat_token_indices[w]). */
int psi_oracle_kv_page_write(void* pages, const void* flat_k, const void* flat_v, const uint32_t* req_slots,
                             const uint32_t* flat_token_indices, const uint32_t* page_ids,
                             uint32_t num_active_token_writes, uint32_t gqa_layer_index, uint32_t num_gqa_layers,
                             uint32_t num_blocks, uint32_t num_page_ids_per_block, uint32_t num_kv_heads,
                             uint32_t head_dim, uint32_t page_bytes, uint32_t dtype) {
    uint32_t tokens_per_page;
    if (psi_oracle_tokens_per_page(num_kv_heads, head_dim, page_bytes, dtype, &tokens_per_page) != 0) return -1;
    const size_t es = dtype_size(dtype);
    const uint64_t page_elems = page_bytes / es;
    for (uint32_t w = 0; w < num_active_token_writes; ++w)
        for (uint32_t head = 0; head < num_kv_heads; ++head)
            for (uint32_t kind = 0; kind < 2; ++kind) {
                uint64_t dst = page_elem_offset(page_ids, req_slots[w], gqa_layer_index, flat_token_indices[w],
                                                num_gqa_layers, num_blocks, num_page_ids_per_block, tokens_per_page,
                                                page_elems, num_kv_heads, head_dim, kind, head);
                uint64_t src = ((uint64_t)w * num_kv_heads + head) * head_dim;
                memcpy((char*)pages + dst * es, (const char*)(kind ? flat_v : flat_k) + src * es, head_dim * es);
            }
    return 0;
}

/* Reads `context_len` tokens of one request back out of the pages through the table into the
 * dense [context_len, num_kv_heads, head_dim] f32 layout projected_gqa_reference consumes; the
 * inverse of the page packer in gqa_split_kv_single_q_test.rs:397-424. */
int psi_oracle_gather_context(const void* pages, const uint32_t* page_ids, uint32_t req_slot,
                              uint32_t gqa_layer_index, uint32_t context_len, uint32_t num_gqa_layers,
                              uint32_t num_blocks, uint32_t num_page_ids_per_block, uint32_t num_kv_heads,
                              uint32_t head_dim, uint32_t page_bytes, uint32_t dtype, float* ctx_k, float* ctx_v) {
    uint32_t tokens_per_page;
    if (psi_oracle_tokens_per_page(num_kv_heads, head_dim, page_bytes, dtype, &tokens_per_page) != 0) return -1;
    const uint64_t page_elems = page_bytes / dtype_size(dtype);
    for (uint32_t t = 0; t < context_len; ++t)
        for (uint32_t head = 0; head < num_kv_heads; ++head) {
            uint64_t k_off = page_elem_offset(page_ids, req_slot, gqa_layer_index, t, num_gqa_layers, num_blocks,
                                              num_page_ids_per_block, tokens_per_page, page_elems, num_kv_heads,
                                              head_dim, 0, head);
            uint64_t v_off = page_elem_offset(page_ids, req_slot, gqa_layer_index, t, num_gqa_layers, num_blocks,
                                              num_page_ids_per_block, tokens_per_page, page_elems, num_kv_heads,
                                              head_dim, 1, head);
            float* kd = ctx_k + ((uint64_t)t * num_kv_heads + head) * head_dim;
            float* vd = ctx_v + ((uint64_t)t * num_kv_heads + head) * head_dim;
            for (uint32_t d = 0; d < head_dim; ++d) {
                kd[d] = load_elem(pages, k_off + d, dtype);
                vd[d] = load_elem(pages, v_off + d, dtype);
            }
        }
    return 0;
}

/* The whole decode/verify step on the CPU: per request gather the context through the page table,
 * widen q to f32 and run projected_gqa_reference.  req_slots_by_req[r] is the request's table row;
 * q is [total_tokens, Hq, D] in `dtype`; out is f32. */
int psi_oracle_paged_gqa(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim, float scale,
                         uint32_t page_bytes, uint32_t dtype, uint32_t num_req_slots, uint32_t num_gqa_layers,
                         uint32_t num_blocks, uint32_t num_page_ids_per_block, uint32_t gqa_layer_index,
                         uint32_t num_reqs, const uint32_t* req_slots_by_req, const uint32_t* token_indices,
                         const uint32_t* cu_tokens, const void* q, const void* pages, const uint32_t* page_ids,
                         float* out, int num_threads) {
    (void)num_req_slots;
    const uint64_t total_tokens = cu_tokens[num_reqs];
    const uint64_t q_elems = total_tokens * num_q_heads * head_dim;
    float* qf = (float*)malloc(sizeof(float) * (q_elems ? q_elems : 1));
    psi_oracle_convert_to_f32(q, qf, q_elems, dtype);
    int status = 0;
    for (uint32_t r = 0; r < num_reqs && status == 0; ++r) {
        uint32_t n_r = cu_tokens[r + 1] - cu_tokens[r];
        uint32_t ctx = token_indices[r] + n_r;
        uint64_t ctx_elems = (uint64_t)ctx * num_kv_heads * head_dim;
        float* ck = (float*)malloc(sizeof(float) * (ctx_elems ? ctx_elems : 1));
        float* cv = (float*)malloc(sizeof(float) * (ctx_elems ? ctx_elems : 1));
        status = psi_oracle_gather_context(pages, page_ids, req_slots_by_req[r], gqa_layer_index, ctx,
                                           num_gqa_layers, num_blocks, num_page_ids_per_block, num_kv_heads,
                                           head_dim, page_bytes, dtype, ck, cv);
        if (status == 0) {
            /* Run the dense reference on this request alone; its outputs land at the request's rows. */
            uint32_t cu_one[2] = {0, n_r};
            uint32_t ti_one[1] = {token_indices[r]};
            const float* kk[1] = {ck};
            const float* vv[1] = {cv};
            uint64_t row0 = (uint64_t)cu_tokens[r] * num_q_heads * head_dim;
            status = psi_oracle_projected_gqa(num_q_heads, num_kv_heads, head_dim, scale, 1, cu_one, ti_one,
                                              qf + row0, kk, vv, out + row0, num_threads);
        }
        free(ck);
        free(cv);
    }
    free(qf);
    return status;
}

/* ---------------------------------------------------------------- projections around the attention
 *
 * Restated from the reference's pre / post kernels of a gated GQA layer:
 *   psi_oracle_qgkv_split            crates/inference-backend-metal/src/components/metal/gqa_qgkv_split.metal:5-43
 *   psi_oracle_rope_parameters       crates/inference-backend-metal/src/components/rms_norm_rope.rs:170-238
 *   psi_oracle_rms_norm_rope         crates/inference-backend-metal/src/components/metal/rms_norm_rope.metal:7-82
 *   psi_oracle_activation_gate       crates/inference-backend-metal/src/components/metal/gqa_activation_gate.metal:13-38
 * What pins them (tests/test_oracle.py): the two-token split / norm_rope_2 / gate closed forms of
 * crates/inference-executor-metal/src/attn/gqa/backend.rs:883-1027, the Yarn correction range 14 / 29 and the
 * long-context Yarn closed form of rms_norm_rope.rs:395-470, and the bf16 rounding-order vector of
 * rms_norm_rope.rs:472-517.  The reference's kernels call Metal's fast cos / sin / exp; this file uses libm, and
 * the reference's own tests allow 1e-3 (long context) and 2e-5 (small positions) for that.
 */

/* One token row [q_0 | g_0 | q_1 | g_1 | ... | k | v] -> q, g [Hq][D] and k, v [Hkv][D]. */
int psi_oracle_qgkv_split(const void* qgkv, void* q, void* g, void* k, void* v, uint32_t num_active_tokens,
                          uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim, uint32_t dtype) {
    const size_t es = dtype_size(dtype);
    const uint64_t q_slots = (uint64_t)num_q_heads * head_dim, kv_slots = (uint64_t)num_kv_heads * head_dim;
    const uint64_t width = 2 * q_slots + 2 * kv_slots;
    for (uint64_t gid = 0; gid < (uint64_t)num_active_tokens * width; ++gid) {
        const uint64_t token = gid / width;
        uint64_t slot = gid - token * width;
        const char* src = (const char*)qgkv + gid * es;
        if (slot < 2 * q_slots) {
            const uint64_t pair = slot / (2 * head_dim), in_pair = slot - pair * 2 * head_dim;
            const uint64_t dst = (token * num_q_heads + pair) * head_dim + in_pair % head_dim;
            memcpy((char*)(in_pair < head_dim ? q : g) + dst * es, src, es);
            continue;
        }
        slot -= 2 * q_slots;
        if (slot < kv_slots) {
            memcpy((char*)k + (token * kv_slots + slot) * es, src, es);
            continue;
        }
        slot -= kv_slots;
        memcpy((char*)v + (token * kv_slots + slot) * es, src, es);
    }
    return 0;
}

/* Inverse frequencies [rope_dim / 2] and the attention factor.  yarn == 0: plain RoPE.
 * correction[2] receives the (low, high) Yarn correction range when yarn != 0. */
int psi_oracle_rope_parameters(uint32_t rope_dim, float rope_theta, int yarn, float factor, float attention_factor,
                               float beta_fast, float beta_slow, uint32_t original_max_position_embeddings,
                               int truncate, float* inverse_frequencies, float* out_attention_factor,
                               float* correction) {
    if (rope_dim == 0 || rope_dim % 2 != 0 || !(rope_theta > 0.0f)) return -1;
    float low = 0.0f, high = 0.0f;
    if (yarn) {
        const double dimension = (double)rope_dim, base = (double)rope_theta;
        const double original_length = (double)original_max_position_embeddings;
        const double tau = 6.283185307179586476925286766559;
        low = (float)(dimension * log(original_length / ((double)beta_fast * tau)) / (2.0 * log(base)));
        high = (float)(dimension * log(original_length / ((double)beta_slow * tau)) / (2.0 * log(base)));
        if (low < 0.0f) low = 0.0f;
        const float cap = (float)(rope_dim > 0 ? rope_dim - 1 : 0);
        if (high > cap) high = cap;
        if (truncate) {
            low = floorf(low);
            high = ceilf(high);
        }
        if (low > high) return -1;
        if (low == high) high += 0.001f;
        if (correction) {
            correction[0] = low;
            correction[1] = high;
        }
    }
    const uint32_t half = rope_dim / 2;
    for (uint32_t d = 0; d < half; ++d) {
        float inv = powf(rope_theta, -((float)d / (float)half));
        if (yarn) {
            float ramp = ((float)d - low) / (high - low);
            ramp = ramp < 0.0f ? 0.0f : (ramp > 1.0f ? 1.0f : ramp);
            inv *= 1.0f + ramp * (1.0f / factor - 1.0f);
        }
        inverse_frequencies[d] = inv;
    }
    *out_attention_factor = yarn ? attention_factor : 1.0f;
    return 0;
}

/* Rounds through the storage type: T(x) of the Metal source. */
static float round_to(float v, uint32_t dtype) {
    if (dtype == PSI_ORACLE_BF16) return psi_oracle_bf16_to_f32(psi_oracle_f32_to_bf16(v));
    if (dtype == PSI_ORACLE_F16) return psi_oracle_f16_to_f32(psi_oracle_f32_to_f16(v));
    return v;
}
static void store_elem(void* base, uint64_t index, uint32_t dtype, float v) {
    if (dtype == PSI_ORACLE_F32) ((float*)base)[index] = v;
    else if (dtype == PSI_ORACLE_BF16) ((uint16_t*)base)[index] = psi_oracle_f32_to_bf16(v);
    else ((uint16_t*)base)[index] = psi_oracle_f32_to_f16(v);
}

/* rows = num_active_tokens * num_heads; input / output [tokens][heads][head_dim] in `dtype`; norm_weight is bf16
 * bits.  Per row: inv = 1 / sqrt(mean(x^2) + eps) in f32 (sequential sum); normalised element
 * T(T(w) * T(x * inv)); dims d < rope_dim / 2 rotate with their partner d + rope_dim / 2 in f32 at angle
 * position * inverse_frequencies[d]; dims >= rope_dim are the normalised element.  The weight product is
 * formed in the storage type: for bf16, a product of two bf16 values rounded once. */
int psi_oracle_rms_norm_rope(const void* input, const uint16_t* norm_weight, const uint32_t* flat_token_indices,
                             void* output, uint32_t num_active_tokens, uint32_t num_heads, uint32_t head_dim,
                             uint32_t rope_dim, float eps, const float* inverse_frequencies, float attention_factor,
                             uint32_t dtype) {
    if (rope_dim > head_dim || rope_dim % 2 != 0) return -1;
    const uint32_t half = rope_dim / 2;
    for (uint64_t row = 0; row < (uint64_t)num_active_tokens * num_heads; ++row) {
        const uint64_t base = row * head_dim;
        float acc = 0.0f;
        for (uint32_t d = 0; d < head_dim; ++d) {
            const float x = load_elem(input, base + d, dtype);
            acc += x * x;
        }
        const float inv = 1.0f / sqrtf(acc / (float)head_dim + eps);
        const float position = (float)flat_token_indices[row / num_heads];
        for (uint32_t d = 0; d < head_dim; ++d) {
            if (d < half) {
                const uint32_t d2 = d + half;
                const float x1 = round_to(round_to(psi_oracle_bf16_to_f32(norm_weight[d]), dtype) *
                                              round_to(load_elem(input, base + d, dtype) * inv, dtype), dtype);
                const float x2 = round_to(round_to(psi_oracle_bf16_to_f32(norm_weight[d2]), dtype) *
                                              round_to(load_elem(input, base + d2, dtype) * inv, dtype), dtype);
                const float theta = position * inverse_frequencies[d];
                const float c = cosf(theta), s = sinf(theta);
                store_elem(output, base + d, dtype, attention_factor * (x1 * c - x2 * s));
                store_elem(output, base + d2, dtype, attention_factor * (x1 * s + x2 * c));
            } else if (d >= rope_dim) {
                store_elem(output, base + d, dtype,
                           round_to(psi_oracle_bf16_to_f32(norm_weight[d]), dtype) *
                               round_to(load_elem(input, base + d, dtype) * inv, dtype));
            }
        }
    }
    return 0;
}

/* sigmoid(x) = y or 1 - y with y = 1 / (1 + exp(-|x|)); the bf16 variant rounds to bf16 after every step
 * (gqa_activation_gate.metal:13-27).  output = T(attention_output * sigmoid(gate)). */
int psi_oracle_activation_gate(const void* attention_output, const void* gates, void* output, uint64_t count,
                               uint32_t dtype) {
    for (uint64_t i = 0; i < count; ++i) {
        const float a = load_elem(attention_output, i, dtype), x = load_elem(gates, i, dtype);
        float s;
        if (dtype == PSI_ORACLE_F32) {
            const float y = 1.0f / (1.0f + expf(-fabsf(x)));
            s = x < 0.0f ? 1.0f - y : y;
        } else {
            const float abs_x = round_to(fabsf(x), dtype);
            const float exp_x = round_to(expf(-abs_x), dtype);
            const float denom = round_to(1.0f + exp_x, dtype);
            const float y = round_to(1.0f / denom, dtype);
            s = x < 0.0f ? round_to(1.0f - y, dtype) : y;
        }
        store_elem(output, i, dtype, a * s);
    }
    return 0;
}
