/*
 * psi_hip.h -- C ABI of the MI355X (gfx950) paged KV-cache attention path.
 *
 * This is the layer an `inference-backend-hip` crate (a sibling of the reference's
 * `inference-backend-metal`) binds: every entry point takes plain pointers and sizes, returns an
 * `int` status, never throws and never aborts.  Device pointers are ordinary HIP device
 * addresses owned by the caller; the library allocates no device memory in any entry point below.
 *
 * Status codes: 0 = ok; negative = error, text available from psi_hip_last_error() (per thread).
 * Contract violations that make the reference `panic!`/`assert!` come back as
 * PSI_HIP_ERR_INVALID_ARGUMENT with the reference's message.
 *
 * Each declaration cites the reference interface it replaces (paths relative to the reference
 * repository root).
 */
#ifndef PSI_HIP_H
#define PSI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PSI_HIP_OK 0
#define PSI_HIP_ERR_INVALID_ARGUMENT (-1)
#define PSI_HIP_ERR_RESOURCE_EXHAUSTED (-2)
#define PSI_HIP_ERR_RUNTIME (-3)
#define PSI_HIP_ERR_UNSUPPORTED (-4)

/* Element type of q / K / V / pages / output.  The reference's `Dtype::{Float32, Bfloat16}`
 * (crates/inference-backend-metal/src/components/gqa_split_kv.rs:33); F16 is added for the
 * fp16-page configuration and is byte-compatible with the u16 page write. */
#define PSI_HIP_F32 0u
#define PSI_HIP_BF16 1u
#define PSI_HIP_F16 2u

#define PSI_HIP_SENTINEL 0xffffffffu /* padding value of kv_splits rows (u32::MAX) */

/* SplitKV variant tags, `GQASplitKVVariant` (gqa_split_kv.rs:8-19). */
#define PSI_HIP_VARIANT_SINGLE_Q 0u
#define PSI_HIP_VARIANT_TILED_Q 1u

typedef struct psi_hip_ctx psi_hip_ctx;

/* Fixed workload facts: `GQASplitKVConfig` / `GQAKVPageWriteConfig` / `GQASplitKVSingleQConfig`
 * (gqa_split_kv.rs:23-29, gqa_kv_page_write.rs:42-48, gqa_split_kv_single_q.rs:47-58).  `scale`
 * is the model's attention scale; kernels never substitute 1/sqrt(head_dim). */
typedef struct psi_hip_gqa_config {
    uint32_t num_q_heads;
    uint32_t num_kv_heads;
    uint32_t head_dim;
    float scale;
    uint32_t page_bytes;
    uint32_t dtype;
} psi_hip_gqa_config;

/* `GQAPageTableLayout`: u32 page_ids[num_req_slots][num_gqa_layers][num_blocks][num_page_ids_per_block]
 * (crates/inference-executor-core/src/attn/gqa/core.rs:146-183). */
typedef struct psi_hip_page_table_layout {
    uint32_t num_req_slots;
    uint32_t num_gqa_layers;
    uint32_t num_blocks;
    uint32_t num_page_ids_per_block;
} psi_hip_page_table_layout;

/* `GQASplitKVVariant` with its geometry (gqa_split_kv.rs:8-19).  SingleQ uses kv_token_tile_size,
 * num_threads_per_threadblock, q_head_tile_size; TiledQ uses q_token_tile_size,
 * kv_token_tile_size, q_head_tile_size.  The tile fields drive the metadata planner (split
 * boundaries fall on kv_token_tile_size multiples); the HIP kernels choose their own launch shape. */
typedef struct psi_hip_split_kv_variant {
    uint32_t kind;
    uint32_t q_token_tile_size;
    uint32_t kv_token_tile_size;
    uint32_t num_threads_per_threadblock;
    uint32_t q_head_tile_size;
} psi_hip_split_kv_variant;

/* `GQAReplayShape` (core.rs:94-143). */
typedef struct psi_hip_gqa_replay_shape {
    uint32_t num_tokens;
    uint32_t num_total_tokens;
    uint32_t num_q_token_tiles;
    uint32_t num_total_q_token_tiles;
    uint32_t num_kv_splits;       /* num_sdpa_map_task_templates */
    uint32_t num_total_kv_splits; /* num_total_sdpa_map_task_templates */
    uint32_t reduce_sdpa_partial_outputs;
} psi_hip_gqa_replay_shape;

/* ------------------------------------------------------------------ library / context */

const char* psi_hip_last_error(void);
const char* psi_hip_version(void);

/* Replaces `Device::system_default()` + `Stream::new` (crates/inference-backend-metal/src/metal/mod.rs:12-40).
 * `stream` is a hipStream_t (NULL = the default stream); every launch of this context goes to
 * it.  A context is confined to one thread, like the reference's executor.  The context owns 64 bytes of pinned
 * host memory (the device error words) and 64 bytes of device memory (the counters through which the workgroups of
 * a prefill-chunk map share out its work: zero between launches, so the launches of one context must follow one
 * another on its stream, as they do, and two contexts never share them); both are allocated here and freed by
 * psi_hip_ctx_destroy, no launch allocates. */
int psi_hip_ctx_create(int device, void* stream, psi_hip_ctx** out_ctx);
int psi_hip_ctx_destroy(psi_hip_ctx* ctx);
/* Later launches go to `stream`.  They are ordered behind what the context has launched on its previous stream (an
 * event recorded there, awaited here: no host synchronisation), so the one-after-the-other rule above survives the
 * switch.  Not while either stream is being captured into a graph: then the order is the capturing caller's. */
int psi_hip_ctx_set_stream(psi_hip_ctx* ctx, void* stream);
/* `ReplaySubmission::wait` (stream synchronisation). */
int psi_hip_sync(psi_hip_ctx* ctx);
/* Per-kernel timing for measurement harnesses: when enabled, every launch is bracketed by HIP
 * events on the context's stream; psi_hip_ctx_kernel_time_ms drains them (synchronises) and
 * returns the accumulated milliseconds and launch count of the kernel with that name
 * ("kv_page_write", "split_kv_map", "split_kv_reduce", "tiled_q_map", "tiled_q_reduce"). */
int psi_hip_ctx_set_timing(psi_hip_ctx* ctx, int enabled);
int psi_hip_ctx_kernel_time_ms(psi_hip_ctx* ctx, const char* kernel, double* out_total_ms, uint64_t* out_launches);
int psi_hip_ctx_reset_timing(psi_hip_ctx* ctx);
/* Behaviour switches.  FORCE_GENERIC routes every attention launch to the shape-generic kernels
 * (the cross-check variant, like the reference's `--validate` runs that compare two variants). */
#define PSI_HIP_FLAG_FORCE_GENERIC 1u
/* F32_OUTPUT makes the combine kernels store the attention output as f32 [tokens, Hq, D] instead of
 * the io dtype, so a harness can check the f32-accumulated result before output rounding. */
#define PSI_HIP_FLAG_F32_OUTPUT 2u
/* MUTE_LOADERS is for harnesses: while it is set, the loading waves of the multi-query map never say that a
 * tile has landed, so that the other waves' waits (bounded at 65536 polls) run out, which sets
 * PSI_HIP_DEVICE_ERR_WAIT_GAVE_UP below while every kernel still runs to its end.  (The prefill-chunk map
 * has no such waits: its waves meet at workgroup barriers only.) */
#define PSI_HIP_FLAG_MUTE_LOADERS 3u
int psi_hip_ctx_set_flag(psi_hip_ctx* ctx, uint32_t flag, uint32_t value);

/* Errors a kernel found while it ran.  The reference has no counterpart: its Metal kernels have no
 * waits between simdgroups and multiply K and V in the storage type.  Here a kernel that could not
 * compute a row reports it in a word of pinned host memory that belongs to the context (written by the
 * GPU, read by the host after a synchronisation), and stores the affected partial rows as empty states
 * (maximum -inf, sum 0), so that no stale or half-computed row is merged.
 *   WAIT_GAVE_UP  a wave's bounded wait for another wave of its workgroup ran out (multi-query map);
 *   V_RANGE       the prefill-chunk map met a V element of a bf16 cache that f16 cannot hold (finite
 *                 |v| > 65504, Inf or NaN): that map multiplies V as f16.  Run the batch through
 *                 psi_hip_split_kv_tiled_q_map instead, which keeps V in the storage type -- except for tiles of
 *                 more than 48 query columns, which that entry point hands to the same kernel: for those, set
 *                 PSI_HIP_FLAG_FORCE_GENERIC for the step (the shape-generic kernels multiply in f32).
 * psi_hip_sync returns PSI_HIP_ERR_RUNTIME while a bit is set; psi_hip_ctx_take_device_error
 * synchronises the context's stream, returns the bits and clears them. */
#define PSI_HIP_DEVICE_ERR_WAIT_GAVE_UP 1u
#define PSI_HIP_DEVICE_ERR_V_RANGE 2u
int psi_hip_ctx_take_device_error(psi_hip_ctx* ctx, uint32_t* out_bits);

/* Device-side active counts for captured launches: the counterpart of `ReplayU32::Parameter`
 * (crates/inference-backend-metal/src/metal/replay.rs; bound at submit by `ReplayArguments::with_u32`).
 * device_counts: device u32[4] = {num_active_tokens (= token writes), num_active_q_token_tiles,
 * num_active_kv_splits, gqa_layer_index + 1}, or null to unbind.  The last word binds the page-table layer the
 * same way (`qwen3.5.mtp.gqa_layer_index`, crates/inference-executor-metal/src/model/qwen/v3_5/mtp/layer.rs:88,
 * mtp/mod.rs:335-339: one recorded program serves every MTP step): 0 keeps the gqa_layer_index argument of the
 * entry point, n > 0 selects layer n - 1 (clamped to the table's layers) for the append and the maps.  While bound, every kernel launched through this
 * context reads its active counts from the block when it RUNS; the num_active_* arguments of the entry
 * points then are upper bounds (pass the capacities): grids are cut for them and the device values are
 * clamped to them.  A HIP graph captured with the block bound therefore serves every batch of its
 * capacity bucket: refresh the metadata arrays and the block, replay.  Lanes beyond the device counts
 * touch nothing, as with the by-value counts. */
int psi_hip_ctx_bind_replay_counts(psi_hip_ctx* ctx, const uint32_t* device_counts);

/* ------------------------------------------------------------------ geometry (host only) */

/* `GQAKVPageWriteConfig::num_tokens_per_page` (gqa_kv_page_write.rs:57-70). */
int psi_hip_gqa_tokens_per_page(const psi_hip_gqa_config* cfg, uint32_t* out_tokens_per_page);

/* `GQASplitKV::new(config).select(num_tokens, num_q_token_tiles)` (gqa_split_kv.rs:86-156);
 * dspark_history != 0 selects `new_dspark_history` (SingleQ partial layout only). */
int psi_hip_split_kv_select(const psi_hip_gqa_config* cfg, int dspark_history, uint32_t num_tokens,
                            uint32_t num_q_token_tiles, psi_hip_split_kv_variant* out_variant);
/* `GQASplitKV::max_q_tokens_per_partial_output` (gqa_split_kv.rs:127-133). */
int psi_hip_split_kv_max_q_tokens_per_partial_output(const psi_hip_gqa_config* cfg, int dspark_history,
                                                     uint32_t* out);
/* `select_split_kv_variant` (crates/inference-executor-metal/src/attn/gqa/mod.rs:64-94), including
 * the (head_dim 256, 8 tokens/page) work model of mod.rs:96-316.  bucket_max_tokens = 0 means no
 * replay bucket policy (exact power-of-two padding). */
int psi_hip_split_kv_select_batch(const psi_hip_gqa_config* cfg, uint32_t max_tokens, uint32_t bucket_max_tokens,
                                  const uint32_t* token_indices, const uint32_t* cu_tokens, uint32_t num_reqs,
                                  psi_hip_split_kv_variant* out_variant);

/* `ReplayBucketPolicy::with_topology_boundaries(max, boundaries).buckets()` and `.capacity(active)`
 * (crates/inference-executor-core/src/replay.rs:4-87).  out_buckets may be NULL to query the count. */
int psi_hip_replay_buckets(uint32_t max_capacity, const uint32_t* topology_boundaries, uint32_t num_boundaries,
                           uint32_t* out_buckets, uint32_t buckets_capacity, uint32_t* out_num_buckets);
int psi_hip_replay_bucket_capacity(uint32_t max_capacity, const uint32_t* topology_boundaries,
                                   uint32_t num_boundaries, uint32_t active, uint32_t* out_capacity);

/* ------------------------------------------------------------------ batch metadata (host only) */

#define PSI_HIP_CAPACITY_EXACT 0u             /* `GQAMetadataBuffers::update` */
#define PSI_HIP_CAPACITY_BUCKETED 1u          /* `update_bucketed` */
#define PSI_HIP_CAPACITY_CALLER_TOKENS 2u     /* `update_bucketed_with_token_capacity` */
#define PSI_HIP_CAPACITY_FIXED_PARTITION 3u   /* fixed-length partitions; not in the reference */

/* `GQAMetadataBuffers::update*` (crates/inference-executor-metal/src/attn/gqa/batch_metadata.rs:128-317)
 * with `build_single_q_kv_splits` (:352-424) and `build_tiled_q_kv_splits` (:433-523).
 * Host arrays, each with capacity for max_tokens entries as in `GQAMetadataBuffers::new` (:92-126):
 *   req_slots_by_token[max_tokens], flat_token_indices[max_tokens], q_token_tiles[max_tokens][2],
 *   kv_splits[max_tokens][3], cu_kv_splits[max_tokens + 1].
 * Only the ranges the reference writes are written (tails keep the caller's bytes); kv_splits is
 * padded with PSI_HIP_SENTINEL up to shape->num_total_kv_splits rows.
 * capacity_mode FIXED_PARTITION ignores the greedy budget: token t gets ceil(ctx_t / partition_tokens)
 * splits of partition_tokens (a multiple of variant->kv_token_tile_size); kv_splits must then hold
 * `kv_splits_capacity` rows (>= the plan) and is padded to the bucketed/exact capacity within it. */
int psi_hip_gqa_metadata_update(uint32_t max_tokens, const uint32_t* req_slots, const uint32_t* token_indices,
                                const uint32_t* cu_tokens, uint32_t num_reqs,
                                const psi_hip_split_kv_variant* variant, uint32_t capacity_mode,
                                uint32_t caller_num_total_tokens, const uint32_t* topology_boundaries,
                                uint32_t num_boundaries, uint32_t partition_tokens, uint32_t kv_splits_capacity,
                                uint32_t* req_slots_by_token, uint32_t* flat_token_indices,
                                uint32_t* q_token_tiles, uint32_t* kv_splits, uint32_t* cu_kv_splits,
                                psi_hip_gqa_replay_shape* out_shape);

/* Dispatch order (no counterpart in the reference, which launches rows in plan order): sorts the
 * first num_kv_splits rows of kv_splits in place by descending length (stable; padding rows last) so
 * that the map's longest workgroups start first and the short ones fill the end of the launch.  The
 * rows of a token are then no longer adjacent: partial_row_index[i] (host u32[num_kv_splits]) is the
 * new position of original row i.  Upload it and pass it to the combine entry points as
 * `partial_row_index`; cu_kv_splits keeps indexing the original order.  The map entry points need
 * nothing: they treat rows independently. */
int psi_hip_split_kv_order_longest_first(uint32_t* kv_splits, uint32_t num_kv_splits, uint32_t* partial_row_index);

/* Balanced decode plan (no counterpart in the reference, whose planner budgets partial states, not
 * device occupancy).  Re-cuts the rows of an existing SingleQ plan at 16-token tile boundaries into
 * `num_workers` consecutive groups of equal cost (tiles, plus five tiles' worth for every row started); a map
 * workgroup then serves one group per KV head and all workgroups finish together.  Inside a group, adjacent pieces of one token
 * are one row -- one pass through the keys, one partial state -- whatever the partition of the input plan,
 * so the output has at most num_workers + num_tokens rows (fewer row starts and partial states than a
 * workgroup per input row: the launch streams faster and the combine reads less).
 * kv_splits_in[num_rows_in][3] / cu_in[num_tokens + 1] -> kv_splits_out (capacity rows_capacity rows),
 * cu_out[num_tokens + 1], worker_cu_out[num_workers + 1].  The rows of a token still tile [0, context)
 * in order. */
int psi_hip_split_kv_balance_plan(const uint32_t* kv_splits_in, uint32_t num_rows_in, const uint32_t* cu_in,
                                  uint32_t num_tokens, uint32_t num_workers, uint32_t* kv_splits_out,
                                  uint32_t rows_capacity, uint32_t* cu_out, uint32_t* worker_cu_out,
                                  uint32_t* out_num_rows);
/* Workers per KV head for the balanced plan: 256 / num_kv_heads, i.e. one map workgroup per compute unit over
 * all KV heads (more workgroups mean more rows and partial states for the same bytes and measure slower). */
int psi_hip_split_kv_balanced_workers(const psi_hip_gqa_config* cfg, uint32_t* out_num_workers);

/* ------------------------------------------------------------------ projections around the attention
 *
 * The kernels a gated GQA layer records before and after the attention proper
 * (crates/inference-executor-metal/src/attn/gqa/backend.rs:394-658): QGKV split, Q / K RMSNorm + RoPE, sigmoid
 * gate.  Each has a stand-alone entry point with the reference component's meaning; the K side is also fused
 * into the append (psi_hip_kv_page_write_norm_rope) and the gate into the combine (`gate` argument of the two
 * reduce entry points), which removes a global round trip of K and of the attention output.  Inputs may be
 * strided views of the projection output, so the split itself is optional. */

#define PSI_HIP_ROPE_DEFAULT 0u
#define PSI_HIP_ROPE_YARN 1u

/* `RopeScaling` (crates/inference-backend-metal/src/components/rms_norm_rope.rs:16-27). */
typedef struct psi_hip_rope_scaling {
    uint32_t kind; /* PSI_HIP_ROPE_DEFAULT: the other fields are ignored */
    float factor;
    float attention_factor;
    float beta_fast;
    float beta_slow;
    uint32_t original_max_position_embeddings;
    uint32_t truncate;
} psi_hip_rope_scaling;

/* `RMSNormRopeConfig` (rms_norm_rope.rs:40-49; validate :81-96).  dtype: f32 or bf16 like the reference, or f16. */
typedef struct psi_hip_rms_norm_rope_config {
    uint32_t num_heads;
    uint32_t head_dim;
    uint32_t rope_dim; /* even, 2 .. min(head_dim, 256) */
    float eps;
    float rope_theta;
    psi_hip_rope_scaling scaling;
    uint32_t dtype;
} psi_hip_rms_norm_rope_config;

/* Attention-output gate for the combine: gates in the IO dtype, element (token, q_head, d) at
 * gates[token * token_stride + q_head * head_stride + d].  [T][Hq][D] from a split: strides Hq*D and D; the
 * projection output in place: pointer qgkv + D, strides 2*(Hq+Hkv)*D and 2*D. */
typedef struct psi_hip_output_gate {
    const void* gates;
    uint64_t token_stride;
    uint64_t head_stride;
} psi_hip_output_gate;

/* Host helper: `RopeScaling::kernel_parameters` (rms_norm_rope.rs:170-238): the f32 inverse frequencies
 * [rope_dim / 2] the kernels use (theta^(-d / half), Yarn ramp applied), the attention factor, and the Yarn
 * correction range (low, high) when out_correction is not null and the scaling is Yarn. */
int psi_hip_rope_parameters(const psi_hip_rms_norm_rope_config* cfg, float* out_inverse_frequencies,
                            float* out_attention_factor, float* out_correction);

/* `RMSNormRopeKernel::invoke_bucketed` (rms_norm_rope.rs:273-296; kernel metal/rms_norm_rope.metal:7-82).
 * input: device, row (token, head) at input + (token * input_token_stride + head * input_head_stride) elements;
 * strides 0 = dense [T][heads][head_dim].  norm_weight: device bf16[head_dim].  flat_token_indices: device
 * u32[T], the rotary position of each token.  output: device, dense [T][heads][head_dim]; may alias a dense
 * input.  Per row: x * rsqrt(mean(x^2) + eps) rounded to dtype, times the weight rounded to dtype (product in
 * dtype), dims below rope_dim rotated in f32 as pairs (d, d + rope_dim / 2).  Rows of tokens >=
 * num_active_tokens keep their bytes. */
int psi_hip_rms_norm_rope(psi_hip_ctx* ctx, const psi_hip_rms_norm_rope_config* cfg, const void* input,
                          uint64_t input_token_stride, uint64_t input_head_stride, const void* norm_weight,
                          const uint32_t* flat_token_indices, void* output, uint32_t num_total_tokens,
                          uint32_t num_active_tokens);

/* `GQAQGKVSplitKernel::invoke_bucketed` (crates/inference-backend-metal/src/components/gqa_qgkv_split.rs; kernel
 * metal/gqa_qgkv_split.metal:5-43).  qgkv: device [T][q_0|g_0|q_1|g_1|...|k|v]; q, g: device [T][Hq][D];
 * k, v: device [T][Hkv][D]. */
int psi_hip_qgkv_split(psi_hip_ctx* ctx, uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t head_dim,
                       uint32_t dtype, const void* qgkv, void* q, void* g, void* k, void* v,
                       uint32_t num_total_tokens, uint32_t num_active_tokens);

/* `GQAActivationGateKernel::invoke_bucketed` (gqa_split_kv_single_q.rs:453-543; kernel
 * metal/gqa_activation_gate.metal:13-38): output = attention_output * sigmoid(gates), all [T][Hq][D] in dtype;
 * the 2-byte variants round after every step of the sigmoid.  output may alias attention_output. */
int psi_hip_activation_gate(psi_hip_ctx* ctx, uint32_t num_q_heads, uint32_t head_dim, uint32_t dtype,
                            const void* attention_output, const void* gates, void* output,
                            uint32_t num_total_tokens, uint32_t num_active_tokens);

/* ------------------------------------------------------------------ KV append */

/* `GQAKVPageWrite::invoke_bucketed(...)` recorded and submitted
 * (crates/inference-backend-metal/src/components/gqa_kv_page_write.rs:130-234; kernel
 * metal/gqa_kv_page_write.metal:5-53).  Argument order follows the Metal binding indices 0..10.
 * pages: device, the page arena (written); pages_bytes bounds it (0 = unchecked).
 * flat_k, flat_v: device [num_total_token_writes, num_kv_heads, head_dim].
 * req_slots, flat_token_indices: device u32[num_total_token_writes].
 * page_ids: device u32 table laid out per `layout`.
 * Writes with index >= num_active_token_writes touch nothing. */
int psi_hip_kv_page_write(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
                          void* pages, uint64_t pages_bytes, const void* flat_k, const void* flat_v,
                          const uint32_t* req_slots, const uint32_t* flat_token_indices, const uint32_t* page_ids,
                          uint32_t num_total_token_writes, uint32_t num_active_token_writes,
                          uint32_t gqa_layer_index);

/* The K-side RMSNorm + RoPE (psi_hip_rms_norm_rope with num_heads = num_kv_heads, positions =
 * flat_token_indices) fused into the append: the raw K rows are normalised, rotated and written straight into
 * their page lines; V rows are copied.  No counterpart as one kernel in the reference, which records
 * RMSNormRope(k) then GQAKVPageWrite (backend.rs:470-560).  raw_k / flat_v: row (token, kv_head) at
 * base + token * token_stride + kv_head * head_dim elements (token strides 0 = dense [T][Hkv][D]; the projection
 * output in place: pointers qgkv + 2*Hq*D and qgkv + (2*Hq + Hkv)*D, strides 2*(Hq+Hkv)*D).
 * norm_cfg->num_heads must equal cfg->num_kv_heads, head_dim and dtype must match cfg. */
int psi_hip_kv_page_write_norm_rope(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                    const psi_hip_page_table_layout* layout,
                                    const psi_hip_rms_norm_rope_config* norm_cfg, void* pages, uint64_t pages_bytes,
                                    const void* raw_k, uint64_t k_token_stride, const void* flat_v,
                                    uint64_t v_token_stride, const void* norm_weight, const uint32_t* req_slots,
                                    const uint32_t* flat_token_indices, const uint32_t* page_ids,
                                    uint32_t num_total_token_writes, uint32_t num_active_token_writes,
                                    uint32_t gqa_layer_index);

/* Everything a gated GQA layer does between its projection and the attention, in one launch: the Q-side
 * RMSNorm + RoPE (psi_hip_rms_norm_rope on raw_q with its strides, into the dense q_output [T][Hq][D]) and the
 * fused append above.  The two norm configs differ in num_heads (Hq / Hkv), eps and weights at most: rope_dim,
 * rope_theta and scaling must be equal.  No single-kernel counterpart in the reference (backend.rs:470-560
 * records four operators). */
int psi_hip_qk_norm_rope_kv_page_write(
    psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
    const psi_hip_rms_norm_rope_config* q_norm_cfg, const psi_hip_rms_norm_rope_config* k_norm_cfg, const void* raw_q,
    uint64_t q_token_stride, uint64_t q_head_stride, const void* q_norm_weight, void* q_output, void* pages,
    uint64_t pages_bytes, const void* raw_k, uint64_t k_token_stride, const void* flat_v, uint64_t v_token_stride,
    const void* k_norm_weight, const uint32_t* req_slots, const uint32_t* flat_token_indices, const uint32_t* page_ids,
    uint32_t num_total_tokens, uint32_t num_active_tokens, uint32_t gqa_layer_index);

/* ------------------------------------------------------------------ split-KV decode (SingleQ) */

/* Which kernels a geometry gets (all map and combine entry points below, SingleQ and TiledQ):
 *   bf16 / f16 K/V, head_dim 128 or 256, tokens_per_page a power of two  -> the gfx950 kernels (HBM-bound
 *       decode map, matrix-core multi-query map; prefill-chunk map for pages of at least 8 tokens);
 *   anything else the reference's config admits (f32 K/V, other head dims, other page sizes)  -> the
 *       shape-generic kernels: the same results, correct for every shape, not tuned (a batch of 8
 *       sequences in f32 runs at about 1 % of the HBM peak);
 *   PSI_HIP_FLAG_FORCE_GENERIC sends every geometry to the generic kernels (the cross-check variant). */

/* Scratch for the partial states of `num_total_kv_splits` splits: replaces `GQASplitKVSingleQScratch::new`
 * (gqa_split_kv_single_q.rs:236-246).  The layout is private to the library. */
int psi_hip_split_kv_single_q_scratch_bytes(const psi_hip_gqa_config* cfg, uint32_t num_total_kv_splits,
                                            uint64_t* out_bytes);

/* `GQASplitKVSingleQKernels::invoke_map_bucketed` (gqa_split_kv_single_q.rs:320-351; kernel
 * metal/gqa_split_kv_single_q_map.metal:31-253).  q: device [num_total_tokens, Hq, D];
 * kv_splits: device u32[num_total_kv_splits][3] = {q_token, kv_begin, kv_end}; rows whose
 * q_token >= num_active_tokens (sentinel padding) and rows >= num_active_kv_splits write nothing. */
int psi_hip_split_kv_single_q_map(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                  const psi_hip_page_table_layout* layout, const void* q, const void* kv_pages,
                                  uint64_t kv_pages_bytes, const uint32_t* req_slots, const uint32_t* page_ids,
                                  const uint32_t* kv_splits, void* scratch, uint64_t scratch_bytes,
                                  uint32_t gqa_layer_index, uint32_t num_total_tokens,
                                  uint32_t num_total_kv_splits, uint32_t num_active_tokens,
                                  uint32_t num_active_kv_splits);

/* The append and the map of a decode step in one launch (no counterpart as one kernel in the reference, which
 * records gqa_kv_page_write and then gqa_split_kv_single_q_map, attn/gqa/backend.rs:394-658): the page arena ends
 * up as after psi_hip_kv_page_write, bit for bit, and the partial states as after psi_hip_split_kv_single_q_map up
 * to the order of summation.  The workgroup whose kv_splits row ends at a token's own position
 * (flat_token_indices[t] + 1) writes that token's K/V lines; every position appended in this step is read from
 * flat_k / flat_v instead of its page, after the paged positions of the row.
 * Requires what the two calls require plus: each active token owns a row that ends at its position + 1 (true of
 * every plan of psi_hip_gqa_metadata_update), and the tokens of a request are adjacent and in position order.
 * worker_cu / num_workers: null / 0 for a workgroup per row, or the worker table of a balanced plan as for
 * psi_hip_split_kv_single_q_map_balanced.  Shapes outside the gfx950 decode kernel run the two launches. */
int psi_hip_kv_page_write_split_kv_single_q_map(
    psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout, const void* q,
    void* kv_pages, uint64_t kv_pages_bytes, const void* flat_k, const void* flat_v, const uint32_t* req_slots,
    const uint32_t* flat_token_indices, const uint32_t* page_ids, const uint32_t* kv_splits,
    const uint32_t* worker_cu, uint32_t num_workers, void* scratch, uint64_t scratch_bytes, uint32_t gqa_layer_index,
    uint32_t num_total_tokens, uint32_t num_total_kv_splits, uint32_t num_active_tokens,
    uint32_t num_active_kv_splits);

/* The same map launched over a balanced plan: workgroup w of each KV head serves kv_splits rows
 * [worker_cu[w], worker_cu[w + 1]) (device u32[num_workers + 1], from psi_hip_split_kv_balance_plan).
 * Falls back to the row-per-workgroup launch for shapes outside the gfx950 kernels' domain. */
int psi_hip_split_kv_single_q_map_balanced(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                           const psi_hip_page_table_layout* layout, const void* q,
                                           const void* kv_pages, uint64_t kv_pages_bytes,
                                           const uint32_t* req_slots, const uint32_t* page_ids,
                                           const uint32_t* kv_splits, const uint32_t* worker_cu,
                                           uint32_t num_workers, void* scratch, uint64_t scratch_bytes,
                                           uint32_t gqa_layer_index, uint32_t num_total_tokens,
                                           uint32_t num_total_kv_splits, uint32_t num_active_tokens,
                                           uint32_t num_active_kv_splits);

/* `GQASplitKVSingleQKernels::invoke_reduce_bucketed` (gqa_split_kv_single_q.rs:353-383; kernel
 * metal/gqa_split_kv_single_q_reduce.metal:10-49).  cu_kv_splits: device u32[num_total_tokens + 1];
 * output: device [num_total_tokens, Hq, D]; rows >= num_active_tokens keep their bytes. */
/* partial_row_index: device u32[num_total_kv_splits] from psi_hip_split_kv_order_longest_first, or null
 * when the rows of a token are adjacent as planned.
 * gate: null, or the attention-output gate of a gated GQA layer (metal/gqa_activation_gate.metal:13-38) applied
 * to each output element right after it is rounded to the IO dtype -- the result of the combine followed by
 * psi_hip_activation_gate, without the round trip. */
int psi_hip_split_kv_single_q_reduce(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const void* scratch,
                                     uint64_t scratch_bytes, const uint32_t* cu_kv_splits, void* output,
                                     uint32_t num_total_tokens, uint32_t num_total_kv_splits,
                                     uint32_t num_active_tokens, const uint32_t* partial_row_index,
                                     const psi_hip_output_gate* gate);

/* A partial result another attention task produced for each token, entered into the split row the map leaves
 * alone for it.  Replaces the direct writes of a second producer into the SingleQ partial arrays
 * (metal/gqa_block_sdpa.metal:47-76, the block attention of the second speculator) under the rule of
 * metal/gqa_split_kv_single_q_map.metal:49-53: a kv_splits row whose first field is >= num_active_tokens is
 * skipped by the map and may be filled by someone else before the combine, which merges every row of
 * [cu_kv_splits[t], cu_kv_splits[t + 1]).  Call between the map and the reduce, on the same stream.
 * slot_rows: device u32[num_total_tokens], the kv_splits row reserved for token t
 * (`block_sdpa_map_task_template_indices`, crates/inference-executor-metal/src/attn/dspark/metadata.rs:207-212);
 * a value >= num_total_kv_splits means the token has none.  partial_exp_sums / partial_max_logits: device
 * f32[num_total_tokens, Hq] in the reference's form (sum of exp(logit - max); max of the scaled natural-log
 * logits).  partial_output: device [num_total_tokens, Hq, D] in the IO dtype, already divided by the exp sum.
 * partial_row_index: as for the reduce. */
int psi_hip_split_kv_single_q_store_partials(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, void* scratch,
                                             uint64_t scratch_bytes, const uint32_t* slot_rows,
                                             const float* partial_exp_sums, const float* partial_max_logits,
                                             const void* partial_output, uint32_t num_total_tokens,
                                             uint32_t num_total_kv_splits, uint32_t num_active_tokens,
                                             const uint32_t* partial_row_index);

/* ------------------------------------------------------------------ split-KV verify / prefill (TiledQ) */

/* `GQASplitKVTiledQConfig::partial_output_bytes + 2 * partial_output_stats_bytes`
 * (gqa_split_kv_tiled_q.rs:131-157). */
int psi_hip_split_kv_tiled_q_scratch_bytes(const psi_hip_gqa_config* cfg, uint32_t q_token_tile_size,
                                           uint32_t num_total_kv_splits, uint64_t* out_bytes);

/* `GQASplitKVTiledQKernels::invoke_map_bucketed` (gqa_split_kv_tiled_q.rs:279-300; kernel
 * metal/gqa_split_kv_tiled_q.metal:49-319).  q_token_tiles: device u32[num_total_q_token_tiles][2];
 * kv_splits rows index q-token tiles.  Causal mask: key position > flat_token_indices[q] is hidden.
 * max_active_q_tile_tokens (no counterpart in the reference): the largest number of tokens any active
 * tile holds, e.g. 2 for a verify step with one draft; it sizes the kernel's query-column blocks.
 * 0 = unknown, any tile may hold q_token_tile_size tokens.  It is a contract, not a hint: it must bound every
 * batch the launch serves, including every batch later replayed on a graph captured from this call.  A row whose
 * tile holds more tokens is entered as an empty partial state (its keys are not attended).
 * Kernels, for bf16 / f16 with head_dim 128 or 256 and pages of 8 * 2^k tokens: up to 48 query columns per tile
 * (max_active_q_tile_tokens x Q heads per KV head) the multi-query pipeline; 49 to 64 the row-group kernel with every
 * row a group of its own (for bf16 K/V, too, it rounds the probabilities to f16 and multiplies V as f16, reporting
 * V values beyond f16's range as PSI_HIP_DEVICE_ERR_V_RANGE; it uses the context's work counters: see
 * psi_hip_ctx_create).  Everything else: the shape-generic kernel. */
int psi_hip_split_kv_tiled_q_map(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                 const psi_hip_page_table_layout* layout, uint32_t q_token_tile_size,
                                 const void* q, const void* kv_pages, uint64_t kv_pages_bytes,
                                 const uint32_t* req_slots, const uint32_t* page_ids,
                                 const uint32_t* flat_token_indices, const uint32_t* q_token_tiles,
                                 const uint32_t* kv_splits, void* scratch, uint64_t scratch_bytes,
                                 uint32_t gqa_layer_index, uint32_t num_total_tokens,
                                 uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits,
                                 uint32_t num_active_tokens, uint32_t num_active_q_token_tiles,
                                 uint32_t num_active_kv_splits, uint32_t max_active_q_tile_tokens);

/* Row groups for prefill chunks (no counterpart in the reference, whose TiledQ map launches one
 * threadgroup per (row, Q-head tile), gqa_split_kv_tiled_q.rs:402-409).  Host helper: gathers the
 * kv_split rows of consecutive Q-token tiles of one request that start at the same key (the rows of one
 * KV partition of a fixed-partition plan) into groups of up to *out_group_tiles rows, the group with the
 * longest KV range first (its work items walk that range whatever the number of its tokens).  row_groups:
 * host u32[row_groups_capacity], written as [*out_num_groups][*out_group_tiles] row indices padded with PSI_HIP_SENTINEL; capacity of num_kv_splits * 32 words always suffices.  req_slots
 * is the per-token slot array of psi_hip_gqa_metadata_update.  Every non-padding row lands in exactly
 * one group.  *out_group_tiles = 0 when the geometry has no grouped kernel (use the plain map then).
 * With more than five Q heads per KV head a group's heads are dealt to two or three work items, so that an item's
 * tokens x heads fit the 256 query columns of a workgroup -- unless no group of the batch is wider than
 * 256 / (heads per KV head * q_token_tile_size) tiles (short chunks, verify steps): then *out_group_tiles is that
 * number, and the launch, which goes by the table's width, lets one work item serve all the heads of its KV head and
 * read its KV range once.
 * When to use row groups: for requests of more than one Q-token tile (the plain map walks a request's KV range once per
 * tile), and for single tiles of more than 48 query columns (8 tokens x 7 or 8 heads per KV head): the plain and the
 * balanced map hand those to the same kernel, every row a group of its own, but cut for another kernel's shares --
 * 64 sequences of 2048..16384 tokens with 8 new tokens each at 32 Q / 4 KV heads of 256 take 487 us as row groups over
 * the planned partition against 661 us over a balanced plan; with 16 new tokens 529 us against 1534 us.  Single tiles
 * of up to 48 columns are faster through the plain map with a balanced plan (447 us against 483 us at 24 Q heads). */
int psi_hip_split_kv_tiled_q_group_rows(const psi_hip_gqa_config* cfg, uint32_t q_token_tile_size,
                                        const uint32_t* kv_splits, uint32_t num_kv_splits,
                                        const uint32_t* q_token_tiles, uint32_t num_q_token_tiles,
                                        const uint32_t* req_slots, uint32_t* row_groups,
                                        uint64_t row_groups_capacity, uint32_t* out_group_tiles,
                                        uint32_t* out_num_groups);

/* Partition length for a batch of prefill chunks (no counterpart in the reference, which has no fixed partitions).
 * Host helper: the `partition_tokens` of a FIXED_PARTITION plan, a multiple of 256 tokens, with which the work items of
 * psi_hip_split_kv_tiled_q_map_grouped -- (token group, partition, KV head, head subset) -- and the combine behind it
 * end soonest on `num_compute_units` compute units (0 = 256), by a model of that launch: an item costs its KV tiles
 * plus a fixed share, a unit that is through takes the heaviest item left, and every item's partial rows are written
 * and read once.  token_indices[r] is the position of request r's first new token and cu_tokens[r + 1] - cu_tokens[r]
 * the number of its new tokens, as for psi_hip_gqa_metadata_update.  On the shape this library is measured on (2048
 * tokens on a 4096-token prefix, 24 Q / 4 KV heads of 256) it answers 4096; for 512 tokens on the same prefix 1024,
 * where 4096 leaves 96 items for 256 units and takes three times as long; for 64 verify requests of 8 tokens on
 * 2048..16384 cached ones 10240.  The answer depends on the batch's lengths only: cache it per shape class.  *out_partition_tokens = 0 when the geometry has no grouped kernel or the batch
 * is empty. */
int psi_hip_split_kv_chunk_partition_tokens(const psi_hip_gqa_config* cfg, uint32_t q_token_tile_size,
                                            const uint32_t* token_indices, const uint32_t* cu_tokens,
                                            uint32_t num_reqs, uint32_t num_compute_units,
                                            uint32_t* out_partition_tokens);

/* The multi-query map launched over a balanced plan (psi_hip_split_kv_balance_plan on the TiledQ tables: its
 * `num_tokens` is then the number of Q-token tiles and cu_in the per-tile cu_kv_splits): workgroup w of each KV head
 * serves kv_splits rows [worker_cu[w], worker_cu[w + 1]).  Same results as psi_hip_split_kv_tiled_q_map up to the
 * order of summation; shapes outside the gfx950 kernels run one workgroup per row. */
int psi_hip_split_kv_tiled_q_map_balanced(
    psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, const psi_hip_page_table_layout* layout,
    uint32_t q_token_tile_size, const void* q, const void* kv_pages, uint64_t kv_pages_bytes,
    const uint32_t* req_slots, const uint32_t* page_ids, const uint32_t* flat_token_indices,
    const uint32_t* q_token_tiles, const uint32_t* kv_splits, const uint32_t* worker_cu, uint32_t num_workers,
    void* scratch, uint64_t scratch_bytes, uint32_t gqa_layer_index, uint32_t num_total_tokens,
    uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits, uint32_t num_active_tokens,
    uint32_t num_active_q_token_tiles, uint32_t num_active_kv_splits, uint32_t max_active_q_tile_tokens);

/* psi_hip_split_kv_tiled_q_map with one work item per (row group, KV head [, half or a third of the Q heads, by the
 * width of the table: see psi_hip_split_kv_tiled_q_group_rows]):
 * the group's K/V tiles are staged once in LDS for up to 256 query columns and both contractions run
 * on the matrix cores.  The launch is one workgroup per compute unit; a workgroup takes items, in the table's
 * order, until none is left.  Same arguments, scratch layout and results (within rounding) as the plain map;
 * row_groups: device copy of the table of psi_hip_split_kv_tiled_q_group_rows for the same kv_splits.
 * Geometries outside the grouped kernel (other than bf16 / f16, head_dim 128 or 256, pages of 8*2^k
 * tokens) run the plain map. */
int psi_hip_split_kv_tiled_q_map_grouped(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                         const psi_hip_page_table_layout* layout, uint32_t q_token_tile_size,
                                         const void* q, const void* kv_pages, uint64_t kv_pages_bytes,
                                         const uint32_t* req_slots, const uint32_t* page_ids,
                                         const uint32_t* flat_token_indices, const uint32_t* q_token_tiles,
                                         const uint32_t* kv_splits, void* scratch, uint64_t scratch_bytes,
                                         uint32_t gqa_layer_index, uint32_t num_total_tokens,
                                         uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits,
                                         uint32_t num_active_tokens, uint32_t num_active_q_token_tiles,
                                         uint32_t num_active_kv_splits, uint32_t max_active_q_tile_tokens,
                                         const uint32_t* row_groups, uint32_t group_tiles, uint32_t num_groups);

/* `GQASplitKVTiledQKernels::invoke_reduce_bucketed` (gqa_split_kv_tiled_q.rs:314-327; kernel
 * metal/gqa_split_kv_tiled_q.metal:324-378). */
int psi_hip_split_kv_tiled_q_reduce(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg, uint32_t q_token_tile_size,
                                    const void* scratch, uint64_t scratch_bytes, const uint32_t* q_token_tiles,
                                    const uint32_t* cu_kv_splits, void* output, uint32_t num_total_tokens,
                                    uint32_t num_total_q_token_tiles, uint32_t num_total_kv_splits,
                                    uint32_t num_active_q_token_tiles, const uint32_t* partial_row_index,
                                    const psi_hip_output_gate* gate);

/* ------------------------------------------------------------------ the attention layer
 *
 * `GQA::record(GQAInput)` / `UngatedGQA::record` (crates/inference-executor-metal/src/attn/gqa/backend.rs:394-658,
 * ungated_backend.rs:182-380; `ReplayLayer`, src/def/layer.rs:12-23) without the two quantised matmuls around it:
 * one call takes the QGKV projection output and the batch metadata and issues, on the context's stream, what the
 * reference records between them -- QGKV split, Q / K RMSNorm + RoPE, KV page write, SplitKV map of the batch's
 * variant, combine, sigmoid gate -- in this library's fused form: one prepare launch (Q and K normalised and
 * rotated from strided views of the projection output, K and V written straight into their page lines), the map,
 * and the combine with the gate applied to each element as it is stored.  Stream order stands for the barriers the
 * reference records.  Results equal the operator-by-operator sequence bit for bit in the arena and in the output. */

/* Device copies of one batch's `GQAMetadataBuffers` arrays (batch_metadata.rs:22-46) with the shape and variant
 * psi_hip_gqa_metadata_update returned for them, plus this library's optional launch plans for the same rows. */
typedef struct psi_hip_gqa_batch_metadata {
    psi_hip_gqa_replay_shape shape;
    psi_hip_split_kv_variant variant;
    const uint32_t* req_slots;          /* u32[num_total_tokens] */
    const uint32_t* flat_token_indices; /* u32[num_total_tokens] */
    const uint32_t* q_token_tiles;      /* u32[num_total_q_token_tiles][2]; TiledQ only */
    const uint32_t* kv_splits;          /* u32[num_total_kv_splits][3] */
    const uint32_t* cu_kv_splits;       /* u32[num_total_tokens + 1] (SingleQ) / [num_total_q_token_tiles + 1] */
    const uint32_t* partial_row_index;  /* null, or the row order of psi_hip_split_kv_order_longest_first */
    const uint32_t* worker_cu;          /* null, or the worker table of psi_hip_split_kv_balance_plan */
    uint32_t num_workers;
    const uint32_t* row_groups;         /* null, or the table of psi_hip_split_kv_tiled_q_group_rows (TiledQ) */
    uint32_t group_tiles;
    uint32_t num_row_groups;
    uint32_t max_active_q_tile_tokens;  /* TiledQ: bound on the tokens of any tile (0 = q_token_tile_size) */
    /* null, or device u32[4] = {tokens, q-token tiles, KV splits, layer + 1 or 0} that the caller has already filled
     * for this batch, e.g. as four more words of the copy that brings the arrays above to the device: the replay
     * cache then reads its programs' counts there and a submit is the program's launch alone. */
    const uint32_t* replay_counts;
} psi_hip_gqa_batch_metadata;

/* `GQACore` + `GQAMetalConfig` (backend.rs:114-146) as far as the attention needs them. */
typedef struct psi_hip_gqa_layer_config {
    psi_hip_gqa_config attention;
    uint32_t gated; /* 1: `GQA`, projection rows [q_0|g_0|q_1|g_1|...|k|v]; 0: `UngatedGQA`, rows [q|k|v] */
    uint32_t rope_dim;
    float norm_eps;
    float rope_theta;
    psi_hip_rope_scaling rope_scaling;
} psi_hip_gqa_layer_config;

#define PSI_HIP_REPLAY_EXACT 0u    /* `GQAReplayMode::Exact`: active counts equal the recorded capacities */
#define PSI_HIP_REPLAY_BUCKETED 1u /* `GQAReplayMode::Bucketed`: active counts within the capacities */

/* `GQAInput` (backend.rs:169-182).  Activations come either as `qgkv`, the projection output the reference keeps in
 * `scratch.qgkv` ([num_total_tokens] rows in the layer's layout), or -- qgkv null -- as rows that are already
 * split, normalised and rotated: q [T][Hq][D], k and v [T][Hkv][D], optionally gates g [T][Hq][D] (the attention
 * core alone: append, map, combine [, gate]; the decode step then folds the append into the map launch). */
typedef struct psi_hip_gqa_layer_input {
    psi_hip_page_table_layout page_table_layout;
    uint32_t gqa_layer_index;
    uint32_t replay_mode; /* PSI_HIP_REPLAY_* */
    const psi_hip_gqa_batch_metadata* batch_metadata;
    const void* qgkv;
    const void* q;
    const void* k;
    const void* v;
    const void* g;
    void* kv_pages; /* `GQAKVCacheBindings` */
    uint64_t kv_pages_bytes;
    const uint32_t* page_ids;
    const void* q_norm_weight; /* `GQAWeights::{q,k}_norm_weight`: bf16[head_dim]; unused with split inputs */
    const void* k_norm_weight;
    void* q_norm_rope;     /* `scratch.q_norm_rope` [num_total_tokens][Hq][D]; unused with split inputs */
    void* partial_scratch; /* the `scratch.sdpa_partial_*` buffers as one, sized by psi_hip_gqa_layer_scratch_bytes */
    uint64_t partial_scratch_bytes;
    void* output; /* `scratch.gated_attention_output` / `scratch.attention_output`: [num_total_tokens][Hq][D] */
} psi_hip_gqa_layer_input;

/* How the planned rows are dispatched (this library's launch plans; PLAN_ORDER is the reference's). */
#define PSI_HIP_DISPATCH_PLAN_ORDER 0u    /* one workgroup per row, rows as planned */
#define PSI_HIP_DISPATCH_LONGEST_FIRST 1u /* psi_hip_split_kv_order_longest_first */
#define PSI_HIP_DISPATCH_BALANCED 2u      /* psi_hip_split_kv_balance_plan */
#define PSI_HIP_DISPATCH_ROW_GROUPS 3u    /* psi_hip_split_kv_tiled_q_group_rows (TiledQ; SingleQ batches get BALANCED) */
#define PSI_HIP_DISPATCH_AUTO 4u          /* per batch: ROW_GROUPS over the partition length of
                                             psi_hip_split_kv_chunk_partition_tokens when the batch is TiledQ with
                                             FIXED_PARTITION capacities, the host arrays hold a row-group table, and a
                                             request brings more than one Q-token tile or a tile more than 48 query
                                             columns (new tokens x Q heads per KV head); BALANCED over
                                             partition_tokens otherwise */

typedef struct psi_hip_gqa_plan_options {
    uint32_t capacity_mode;           /* PSI_HIP_CAPACITY_* */
    uint32_t partition_tokens;        /* FIXED_PARTITION; with ROW_GROUPS 0 = what
                                         psi_hip_split_kv_chunk_partition_tokens answers for the batch */
    uint32_t caller_num_total_tokens; /* CALLER_TOKENS */
    uint32_t dispatch;                /* PSI_HIP_DISPATCH_* */
    uint32_t num_workers;             /* BALANCED: workers per KV head, 0 = psi_hip_split_kv_balanced_workers */
    uint32_t bucket_max_tokens;       /* variant selection: `GQAReplayBucketPolicy::max_tokens`, 0 = none */
    const uint32_t* topology_boundaries;
    uint32_t num_boundaries;
    uint32_t bucket_capacities;       /* FIXED_PARTITION only: 1 = the recorded capacities of the shape (tokens, Q-token
                                         tiles, KV splits -- the re-cut rows of a balanced plan included -- and the
                                         number of row groups) are rounded up to `ReplayBucketPolicy` buckets of
                                         host->max_tokens (with the topology boundaries), host->max_tokens,
                                         host->kv_splits_capacity and the row-group table's capacity, and the arrays
                                         are padded with PSI_HIP_SENTINEL up to them: a replay cache then sees one key
                                         per bucket instead of one per batch */
} psi_hip_gqa_plan_options;

/* Host arrays of one batch's metadata with their capacities (e.g. views of one pinned staging block that is then
 * uploaded in one copy).  partial_row_index / worker_cu / row_groups may be null when the dispatch does not use
 * them. */
typedef struct psi_hip_gqa_host_metadata {
    uint32_t max_tokens;          /* req_slots_by_token, flat_token_indices [max_tokens]; q_token_tiles [max_tokens][2];
                                     cu_kv_splits [max_tokens + 1] */
    uint32_t kv_splits_capacity;  /* rows of kv_splits ([rows][3]) and of partial_row_index */
    uint32_t max_workers;         /* worker_cu [max_workers + 1] */
    uint64_t row_groups_capacity; /* words of row_groups */
    uint32_t* req_slots_by_token;
    uint32_t* flat_token_indices;
    uint32_t* q_token_tiles;
    uint32_t* kv_splits;
    uint32_t* cu_kv_splits;
    uint32_t* partial_row_index;
    uint32_t* worker_cu;
    uint32_t* row_groups;
} psi_hip_gqa_host_metadata;

/* `GQA::prepare` / `prepare_bucketed` / `prepare_bucketed_with_token_capacity` (backend.rs:289-364): selects the
 * batch's SplitKV variant (`select_split_kv_variant`, variant null) or takes the caller's, updates the metadata
 * arrays, and -- beyond the reference -- adds the dispatch plan, all on the host in one call.  out_plan receives
 * shape, variant, num_workers, group_tiles, num_row_groups and max_active_q_tile_tokens; its pointer fields are
 * left to the caller (they name the device copies).  out_uses (may be null): bit 0 partial_row_index is in use,
 * bit 1 worker_cu, bit 2 row_groups. */
int psi_hip_gqa_layer_prepare(const psi_hip_gqa_layer_config* cfg, const psi_hip_gqa_plan_options* options,
                              const uint32_t* req_slots, const uint32_t* token_indices, const uint32_t* cu_tokens,
                              uint32_t num_reqs, const psi_hip_split_kv_variant* variant,
                              const psi_hip_gqa_host_metadata* host, psi_hip_gqa_batch_metadata* out_plan,
                              uint32_t* out_uses);

/* The next decode step of the batch psi_hip_gqa_layer_prepare planned last into `host` -- the same requests in the
 * same order, one new token each at the next position -- without planning again: positions and the end of every
 * token's last row move on by one, in place.  That equals a fresh preparation bit for bit as long as no sequence
 * starts a new 16-token tile (a plan with fixed partitions, in plan order or balanced, depends on the tile counts
 * alone); when one does, or when the plan is of another kind (greedy capacities, a row index, TiledQ), nothing is
 * touched and *out_advanced is 0: prepare again.  `plan` is the preparation's output; its shape stays as it is.
 * No counterpart in the reference, which plans every batch anew (batch_metadata.rs:128-317). */
int psi_hip_gqa_layer_advance_decode(const psi_hip_gqa_plan_options* options, const psi_hip_gqa_host_metadata* host,
                                     const psi_hip_gqa_batch_metadata* plan, uint32_t plan_uses, int* out_advanced);

/* Bytes of `partial_scratch` for a variant and split capacity (`GQAScratch::new`, scratch.rs:48-92). */
int psi_hip_gqa_layer_scratch_bytes(const psi_hip_gqa_layer_config* cfg, const psi_hip_split_kv_variant* variant,
                                    uint32_t num_total_kv_splits, uint64_t* out_bytes);

/* `GQA::record` (backend.rs:394-658).  With device-side counts bound to the context the launches are valid for
 * every batch of the capacity bucket (psi_hip_ctx_bind_replay_counts). */
int psi_hip_gqa_layer_record(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg,
                             const psi_hip_gqa_layer_input* input);

/* A batch that holds prefill chunks and decode requests at once.  The reference runs such a batch through one
 * SplitKV variant (`select_split_kv_variant`, crates/inference-executor-metal/src/attn/gqa/mod.rs:64-94, then
 * `GQA::record`, backend.rs:394-658), and its server caps a request at 64 tokens per batch; here the requests with more
 * than chunk_min_tokens new tokens go through the TiledQ kernels with the row-group plan (matrix-core bound) and the
 * others through the variant psi_hip_split_kv_select_batch picks for them (HBM bound): two parts of one batch,
 * planned by one call and recorded by one call.  The chunk requests must come first in the batch, so that either
 * part's tokens are one run of the flat q / k / v / output rows; a batch with only one kind has one empty part.
 *
 * psi_hip_gqa_layer_prepare_mixed is psi_hip_gqa_layer_prepare for both parts (chunk_options / decode_options and
 * chunk_host / decode_host as there; the chunk part's dispatch is ROW_GROUPS whatever chunk_options->dispatch says,
 * its variant TiledQ with 8-token tiles).  out_plan->chunk and ->decode receive what psi_hip_gqa_layer_prepare writes
 * to its out_plan (the pointer fields are left to the caller), ->chunk_uses and ->decode_uses its out_uses. */
typedef struct psi_hip_gqa_mixed_plan {
    uint32_t num_chunk_reqs;   /* the batch's first requests: the prefill chunks */
    uint32_t num_chunk_tokens; /* their tokens: rows [0, num_chunk_tokens) of q / k / v / output */
    uint32_t chunk_uses;
    uint32_t decode_uses;
    psi_hip_gqa_batch_metadata chunk;
    psi_hip_gqa_batch_metadata decode;
} psi_hip_gqa_mixed_plan;
int psi_hip_gqa_layer_prepare_mixed(const psi_hip_gqa_layer_config* cfg, const psi_hip_gqa_plan_options* chunk_options,
                                    const psi_hip_gqa_plan_options* decode_options, uint32_t chunk_min_tokens,
                                    const uint32_t* req_slots, const uint32_t* token_indices, const uint32_t* cu_tokens,
                                    uint32_t num_reqs, const psi_hip_gqa_host_metadata* chunk_host,
                                    const psi_hip_gqa_host_metadata* decode_host, psi_hip_gqa_mixed_plan* out_plan);
/* Bytes of `partial_scratch` for a mixed batch: the chunk part's partial states, then the decode part's. */
int psi_hip_gqa_layer_mixed_scratch_bytes(const psi_hip_gqa_layer_config* cfg, const psi_hip_gqa_mixed_plan* plan,
                                          uint64_t* out_bytes);
/* `GQA::record` for a mixed batch: the chunk part, then the decode part, on the context's stream (input->
 * batch_metadata is not used; the row pointers of the input name the whole batch and the decode part's rows start
 * num_chunk_tokens rows in).  Both parts' kernels need a compute unit to themselves and scale with the compute
 * units they get, so running them side by side on two streams gains nothing (measured: 1622 us at best against
 * 1643 us one after the other on a 2048-token chunk next to 128 decode sequences); they are issued in turn. */
int psi_hip_gqa_layer_record_mixed(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg,
                                   const psi_hip_gqa_layer_input* input, const psi_hip_gqa_mixed_plan* plan);

/* psi_hip_gqa_layer_record with the partial states in a buffer built into the library instead of
 * input->partial_scratch (which is ignored, as is partial_scratch_bytes).  No counterpart in the reference.  It is
 * for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid allocation.  The call allocates nothing on the host or the device and only launches kernels; the
 * buffer is a static device array of PSI_HIP_STATIC_SCRATCH_BYTES that every GPU the library runs on holds until
 * the process ends (its address is looked up when a context is created on that GPU).  A batch whose partial
 * states need more (psi_hip_gqa_layer_scratch_bytes for the variant and num_total_kv_splits) is rejected with
 * PSI_HIP_ERR_INVALID_ARGUMENT.  All calls on one GPU share the one buffer, which keeps the previous call's
 * contents: nothing in it has to start at zero (the combine only reads rows the same call's map wrote), but two
 * calls that overlap on one GPU -- on different streams or from different contexts -- race. */
#define PSI_HIP_STATIC_SCRATCH_BYTES (16u << 20)
int psi_hip_gqa_layer_record_static_scratch(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg,
                                            const psi_hip_gqa_layer_input* input);

/* One recorded program per capacity bucket: the counterpart of the reference's replay-program store, which keeps a
 * recorded program per `(variant, total tokens, total Q-token tiles, total KV splits)` key and binds the active
 * counts at submission (crates/inference-executor-core/src/replay.rs:4-87; parameter keys backend.rs:55-57;
 * `Stream::submit_replay_with_arguments`).  Here a program is a HIP graph captured from psi_hip_gqa_layer_record
 * with the counts block bound.  The context's stream must be a created stream (capture is not possible on the
 * null stream).  device_counts: caller-owned device u32[4], written by the cache at every submission.
 * max_programs: programs kept; the least recently used one is dropped beyond that. */
typedef struct psi_hip_gqa_replay_cache psi_hip_gqa_replay_cache;
int psi_hip_gqa_replay_cache_create(psi_hip_ctx* ctx, const psi_hip_gqa_layer_config* cfg, uint32_t* device_counts,
                                    uint32_t max_programs, psi_hip_gqa_replay_cache** out_cache);
int psi_hip_gqa_replay_cache_destroy(psi_hip_gqa_replay_cache* cache);
/* Replays the program of the input's bucket, recording it first if the cache has none: key = variant and geometry,
 * the three capacities of input->batch_metadata->shape, the layer index (when by value), and every buffer address
 * of the input (a program holds addresses).  The active counts of the shape go to the counts block, stream-ordered
 * ahead of the program; gqa_layer_parameter > 0 binds the page-table layer gqa_layer_parameter - 1 the same way
 * (`ReplayU32::Parameter`) instead of the input's gqa_layer_index.  When input->batch_metadata->replay_counts is
 * set, the caller has placed the four words itself (the fourth as gqa_layer_parameter says): the program reads them
 * there, nothing is launched ahead of it, and the address is part of the key.  *out_recorded (may be null): 1 if
 * this call recorded. */
int psi_hip_gqa_replay_cache_submit(psi_hip_gqa_replay_cache* cache, const psi_hip_gqa_layer_input* input,
                                    uint32_t gqa_layer_parameter, int* out_recorded);
/* Programs held, recordings and replays so far; any out pointer may be null. */
int psi_hip_gqa_replay_cache_stats(const psi_hip_gqa_replay_cache* cache, uint32_t* programs, uint64_t* recordings,
                                   uint64_t* replays);

/* ------------------------------------------------------------------ request page table */

/* `GQARequestPageTable::write_page_ids` (crates/inference-executor-metal/src/attn/gqa/request_page_table.rs:58-69):
 * copies `count` (= num_page_ids_per_block) host IDs into the device table row
 * (req_slot, layer_index, block_index) on the context's stream.  IDs >= num_cache_pages are
 * rejected (crates/inference-executor-metal/src/model/qwen/v3_x/state/gqa.rs:97-102); 0 = unchecked. */
int psi_hip_page_table_write_page_ids(psi_hip_ctx* ctx, const psi_hip_page_table_layout* layout,
                                      uint32_t* page_ids_device, uint32_t req_slot, uint32_t layer_index,
                                      uint32_t block_index, const uint32_t* ids, uint32_t count,
                                      uint32_t num_cache_pages);
/* `GQARequestPageTable::reset_req_slot` (request_page_table.rs:71-77): zeroes one slot's rows. */
int psi_hip_page_table_reset_req_slot(psi_hip_ctx* ctx, const psi_hip_page_table_layout* layout,
                                      uint32_t* page_ids_device, uint32_t req_slot);
/* Flat index of (req_slot, layer, block, 0), `page_ids_start_index` (request_page_table.rs:112-117). */
int psi_hip_page_table_start_index(const psi_hip_page_table_layout* layout, uint32_t req_slot,
                                   uint32_t layer_index, uint32_t block_index, uint64_t* out_index);
/* `page_ids_by_layer_for_lane` (crates/inference-executor-core/src/model/replayable_model.rs:182-212):
 * splits one synced block's flat list [layer][id] into per-layer rows; block_ids has
 * num_gqa_layers * num_page_ids_per_block entries, out_by_layer the same count (layer-major). */
int psi_hip_page_ids_by_layer(const uint32_t* block_ids, uint32_t block_ids_len, uint32_t num_gqa_layers,
                              uint32_t num_page_ids_per_block, uint32_t* out_by_layer);

/* ---------------------------------------------------------------------------------------------
 * Cache ownership on the host: page-ID allocator and the per-request token window.  No device work.
 * ------------------------------------------------------------------------------------------- */

/* `U32IDAllocator` (crates/inference-runtime-core/src/memory/u32_id_allocator.rs:40-173): IDs in
 * [0, capacity); freed IDs are re-issued first, in the order they were freed, before never-used
 * ones; a bitmap records what is allocated.  Thread-safe.  Exhaustion returns
 * PSI_HIP_ERR_RESOURCE_EXHAUSTED ("not enough ID") and leaves the allocator unchanged apart from
 * the order of the free queue (popped IDs go back to its tail, as in the reference).  Ownership is
 * shared like the reference's Arc: destroy drops the creator's handle, the allocator itself lives
 * until every decoder-blocks object created on it has been destroyed. */
typedef struct psi_hip_id_allocator psi_hip_id_allocator;
int psi_hip_id_allocator_create(uint64_t capacity, psi_hip_id_allocator** out);
int psi_hip_id_allocator_destroy(psi_hip_id_allocator* allocator);
int psi_hip_id_allocator_alloc_one(psi_hip_id_allocator* allocator, uint32_t* id);
int psi_hip_id_allocator_alloc_many(psi_hip_id_allocator* allocator, size_t count, uint32_t* ids);
int psi_hip_id_allocator_free_one(psi_hip_id_allocator* allocator, uint32_t id);
int psi_hip_id_allocator_free_many(psi_hip_id_allocator* allocator, const uint32_t* ids, size_t count);
/* `used` / `free` / `capacity` (u32_id_allocator.rs:143-153); any out pointer may be null. */
int psi_hip_id_allocator_counts(psi_hip_id_allocator* allocator, uint64_t* used, uint64_t* free_count,
                                uint64_t* capacity);
/* `allocated_ids_bitmap_iter` (u32_id_allocator.rs:62-66): num_words must be ceil(capacity / 64). */
int psi_hip_id_allocator_bitmap(psi_hip_id_allocator* allocator, uint64_t* words, size_t num_words);
/* Runs of set bits as [begin, end) pairs, the scan the reference's hibernation uses to copy only
 * allocated pages (crates/inference-runtime-core/src/runtime/scheduler/executor_hibernate.rs:15-47).
 * ranges may be null to count only. */
int psi_hip_bitmap_allocated_ranges(const uint64_t* words, size_t num_words, uint32_t* ranges, size_t capacity_pairs,
                                    size_t* num_pairs);

/* `TrieDecoderBlocks<N, P, L, BC>` (crates/inference-runtime-core/src/runtime/decoder/trie_cache/blocks/trie/
 * mod.rs:17-39, api.rs:34-571) without prefix sharing: one request's tokens move
 * queued -> ready -> scheduled -> cached through blocks of `tokens_per_block` tokens; each block owns
 * `pages_per_kv_block` page IDs per cache lane (`TPKVBlockAllocator::allocate`,
 * .../decoder/allocator/tp_kv_block_allocator.rs:24-36), drawn lane by lane and released when the
 * block is.  Lane 0 is the main model, lanes 1.. the MTP modules, each one token ahead of the last.
 * Not thread-safe (the allocator it draws from is). */
typedef struct psi_hip_decoder_blocks psi_hip_decoder_blocks;
typedef struct psi_hip_decoder_blocks_config {
    uint32_t tokens_per_block;   /* N */
    uint32_t num_cache_lanes;    /* L >= 1 */
    uint32_t pages_per_kv_block; /* layers * N / tokens_per_page */
} psi_hip_decoder_blocks_config;

enum { PSI_HIP_QUERY_PREFILL = 0, PSI_HIP_QUERY_DECODE = 1 };
/* `QueryTokens` (crates/inference-runtime-core/src/compute/request/decoder/query_tokens.rs:4-17).
 * The token buffers belong to the caller; prepare fills them and the counts. */
typedef struct psi_hip_query_tokens {
    uint32_t kind;        /* PSI_HIP_QUERY_* */
    uint32_t window;      /* prefill only: tokens that advance the cache (= num_tokens - (L - 1)) */
    uint64_t epoch;
    uint64_t token_index; /* absolute position of tokens[0] */
    uint32_t* tokens;
    size_t num_tokens, tokens_capacity;
    uint32_t* spec_tokens; /* decode only: drafts to verify after `tokens` */
    size_t num_spec_tokens, spec_tokens_capacity;
} psi_hip_query_tokens;
/* `SampledTokens` (.../request/decoder/sample_tokens.rs:6-20) minus the probabilities, which the
 * token window never reads. */
typedef struct psi_hip_sampled_tokens {
    uint32_t kind; /* must equal the query's */
    uint32_t sampled_token;
    uint64_t epoch;
    const uint32_t* validated_tokens; /* accepted prefix of the query's spec_tokens */
    size_t num_validated_tokens;
    const uint32_t* spec_tokens; /* drafts for the next step */
    size_t num_spec_tokens;
} psi_hip_sampled_tokens;
enum {
    PSI_HIP_TOKENS_CACHED = 0,
    PSI_HIP_TOKENS_SCHEDULED = 1,
    PSI_HIP_TOKENS_READY = 2,
    PSI_HIP_TOKENS_QUEUED = 3,
    PSI_HIP_TOKENS_SPEC = 4
};

/* `TrieDecoderBlocks::new` (mod.rs:47-82): history, prompt and sampled tokens concatenated. */
int psi_hip_decoder_blocks_create(psi_hip_id_allocator* allocator, const psi_hip_decoder_blocks_config* cfg,
                                  const uint32_t* tokens, size_t num_tokens, psi_hip_decoder_blocks** out);
/* Drop (mod.rs:299-311): releases mutable then semi-immutable blocks, last to first; with no trie
 * to keep them, committed blocks are released as well. */
int psi_hip_decoder_blocks_destroy(psi_hip_decoder_blocks* blocks);
/* `ready_token_slots` (api.rs:35-46). */
int psi_hip_decoder_blocks_ready_token_slots(const psi_hip_decoder_blocks* blocks, size_t* out);
/* `init_block_once` (api.rs:48-136): adds one block and moves up to N queued tokens into it.
 * PSI_HIP_ERR_RESOURCE_EXHAUSTED (state unchanged) when the allocator cannot cover every lane. */
int psi_hip_decoder_blocks_init_block_once(psi_hip_decoder_blocks* blocks, size_t* ready_token_slots);
/* `uninit_block_once` (api.rs:138-153): releases the last block, its tokens return to the queue. */
int psi_hip_decoder_blocks_uninit_block_once(psi_hip_decoder_blocks* blocks, size_t* cached_token_slots);
/* Stored drafts as a resumed request would carry them (the reference's tests assign the field). */
int psi_hip_decoder_blocks_set_spec_tokens(psi_hip_decoder_blocks* blocks, const uint32_t* spec_tokens, size_t count);
/* `prepare` (api.rs:184-273): schedules up to `token_budget` ready tokens; a budget below
 * ready + queued yields a prefill chunk, otherwise a decode step whose spare budget selects stored
 * drafts (the rest are dropped). */
int psi_hip_decoder_blocks_prepare(psi_hip_decoder_blocks* blocks, size_t token_budget, psi_hip_query_tokens* out);
/* `cancel` (api.rs:276-331): un-schedules the newest outstanding query. */
int psi_hip_decoder_blocks_cancel(psi_hip_decoder_blocks* blocks, const psi_hip_query_tokens* query);
/* `commit` (api.rs:334-549): the query's window becomes cached; for a decode step the validated
 * drafts and the sampled token are appended, and as many of them as every lane has seen go to the
 * cache directly.  validated_tokens must be a prefix of the query's spec_tokens. */
int psi_hip_decoder_blocks_commit(psi_hip_decoder_blocks* blocks, const psi_hip_query_tokens* query,
                                  const psi_hip_sampled_tokens* sampled);
/* `prepare_blocks` (mod.rs:176-229) -> `DecoderSyncBlocks` (.../request/decoder/decoder_sync_blocks.rs:2-6):
 * page IDs of the blocks the executor has not seen yet, kv_page_ids[lane][block][pages_per_kv_block];
 * with kv_page_ids null only the counts are returned and nothing is marked as synced. */
int psi_hip_decoder_blocks_prepare_blocks(psi_hip_decoder_blocks* blocks, size_t* block_index, size_t* num_blocks,
                                          uint32_t* kv_page_ids, size_t capacity_ids);
/* `cancel_blocks` (mod.rs:231-233). */
int psi_hip_decoder_blocks_cancel_blocks(psi_hip_decoder_blocks* blocks, size_t block_index);
/* Block counts by kind and the number already synced; any out pointer may be null. */
int psi_hip_decoder_blocks_counts(const psi_hip_decoder_blocks* blocks, size_t* immutable_blocks,
                                  size_t* semi_immutable_blocks, size_t* mutable_blocks, size_t* in_sync_blocks);
/* Lane-0 view of one token class (PSI_HIP_TOKENS_*), `cached_tokens()` .. `spec_tokens()`
 * (blocks/trie/token.rs:10-181); out may be null to count only. */
int psi_hip_decoder_blocks_tokens(const psi_hip_decoder_blocks* blocks, uint32_t which, uint32_t* out,
                                  size_t capacity, size_t* count);

/* ------------------------------------------------------------------ state snapshot of selected entries
 * A snapshot of selected state stores, for a buffer of fixed-size entries, the bytes of the selected entry
 * ranges concatenated in order (`StateSnapshotWriter::write_selected_buffer` /
 * `StateSnapshotReader::read_selected_buffer`, crates/inference-executor-metal/src/model/state_snapshot.rs:249-304,
 * :533-591, ranges from :743-772).  The page arena is selected by page-ID ranges with entry_bytes = page_bytes
 * (model/page_arena/file_io.rs:28-49), the GQA page table by request-slot ranges with entry_bytes =
 * page IDs per request * 4 (attn/gqa/request_page_table/file_io.rs:28-59).  The reference streams each range
 * between unified memory and the file; here the ranges are gathered into (scattered from) one payload in device
 * memory, which then crosses the host link in a single transfer.  File layout, manifest and publishing stay with
 * the caller.
 * entry_ranges: host u32[num_ranges][2] = [begin, end) entry indices, in the reference's canonical form (every
 * range non-empty; sorted, disjoint and not adjacent; state_snapshot.rs:774-776) and inside the buffer, else
 * PSI_HIP_ERR_INVALID_ARGUMENT with the reference's message. */

/* Bytes of the payload of a selection (also validates it). */
int psi_hip_selected_ranges_payload_bytes(const uint32_t* entry_ranges, uint32_t num_ranges, uint64_t entry_bytes,
                                          uint64_t buffer_bytes, uint64_t* out_payload_bytes);

/* buffer (device) -> payload (device, payload_bytes must equal the selection's size), on the context's stream. */
int psi_hip_buffer_pack_selected(psi_hip_ctx* ctx, const void* buffer, uint64_t buffer_bytes,
                                 const uint32_t* entry_ranges, uint32_t num_ranges, uint64_t entry_bytes,
                                 void* payload, uint64_t payload_bytes);

/* payload -> buffer; bytes of the buffer outside the selection are left as they are.  A payload whose size is not
 * the selection's is the reference's "file length mismatch" (state_snapshot.rs:549-559). */
int psi_hip_buffer_unpack_selected(psi_hip_ctx* ctx, void* buffer, uint64_t buffer_bytes,
                                   const uint32_t* entry_ranges, uint32_t num_ranges, uint64_t entry_bytes,
                                   const void* payload, uint64_t payload_bytes);

#ifdef __cplusplus
}
#endif
#endif /* PSI_HIP_H */
