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
