/* Plain C11 consumer of include/psi_hip.h: proves the header is C (not only C++), links
 * libpsi_hip.so and calls entry points that need no GPU.  Exit status 0 = every check passed. */
#include <stdio.h>
#include <string.h>

#include "psi_hip.h"

#define CHECK(cond)                                                      \
    do {                                                                 \
        if (!(cond)) {                                                   \
            fprintf(stderr, "%s:%d: %s failed (%s)\n", __FILE__, __LINE__, #cond, psi_hip_last_error()); \
            return 1;                                                    \
        }                                                                \
    } while (0)

int main(void) {
    CHECK(strstr(psi_hip_version(), "gfx950") != NULL);

    /* page geometry: bf16, 4 KV heads, head_dim 256, 64 KiB pages -> 16 tokens per page */
    psi_hip_gqa_config cfg = {24u, 4u, 256u, 0.0625f, 65536u, PSI_HIP_BF16};
    uint32_t tokens_per_page = 0;
    CHECK(psi_hip_gqa_tokens_per_page(&cfg, &tokens_per_page) == PSI_HIP_OK && tokens_per_page == 16u);
    cfg.page_bytes = 65537u;
    CHECK(psi_hip_gqa_tokens_per_page(&cfg, &tokens_per_page) == PSI_HIP_ERR_INVALID_ARGUMENT);
    CHECK(strlen(psi_hip_last_error()) > 0);
    cfg.page_bytes = 65536u;

    /* variant selection: a decode batch stays SingleQ, a two-token verify batch goes TiledQ */
    psi_hip_split_kv_variant variant;
    CHECK(psi_hip_split_kv_select(&cfg, 0, 32u, 32u, &variant) == PSI_HIP_OK);
    CHECK(variant.kind == PSI_HIP_VARIANT_SINGLE_Q);
    CHECK(psi_hip_split_kv_select(&cfg, 0, 128u, 64u, &variant) == PSI_HIP_OK);
    CHECK(variant.kind == PSI_HIP_VARIANT_TILED_Q && variant.q_token_tile_size == 8u);

    /* capacity buckets */
    uint32_t capacity = 0;
    CHECK(psi_hip_replay_bucket_capacity(128u, NULL, 0u, 25u, &capacity) == PSI_HIP_OK && capacity == 32u);

    /* metadata of a two-request decode batch (reference vector: tile 8, slots [2,5], starts [7,20]) */
    const uint32_t slots[2] = {2u, 5u}, starts[2] = {7u, 20u}, cu[3] = {0u, 2u, 5u};
    psi_hip_split_kv_variant single = {PSI_HIP_VARIANT_SINGLE_Q, 1u, 8u, 256u, 6u};
    uint32_t by_token[8], flat[8], tiles[16], splits[24], cu_splits[9];
    psi_hip_gqa_replay_shape shape;
    CHECK(psi_hip_gqa_metadata_update(8u, slots, starts, cu, 2u, &single, PSI_HIP_CAPACITY_EXACT, 0u, NULL, 0u, 0u, 8u,
                                      by_token, flat, tiles, splits, cu_splits, &shape) == PSI_HIP_OK);
    CHECK(shape.num_tokens == 5u && shape.num_kv_splits == 8u && cu_splits[5] == 8u);
    CHECK(flat[0] == 7u && flat[4] == 22u && by_token[2] == 5u);

    /* scratch size query */
    uint64_t bytes = 0;
    CHECK(psi_hip_split_kv_single_q_scratch_bytes(&cfg, 8u, &bytes) == PSI_HIP_OK && bytes >= 8u * 24u * 258u * 4u);

    /* page-ID allocator: fresh IDs ascend, freed IDs come back first and in order */
    psi_hip_id_allocator* allocator = NULL;
    CHECK(psi_hip_id_allocator_create(65u, &allocator) == PSI_HIP_OK);
    uint32_t ids[4];
    CHECK(psi_hip_id_allocator_alloc_many(allocator, 4u, ids) == PSI_HIP_OK && ids[0] == 0u && ids[3] == 3u);
    CHECK(psi_hip_id_allocator_free_one(allocator, 2u) == PSI_HIP_OK);
    CHECK(psi_hip_id_allocator_free_one(allocator, 0u) == PSI_HIP_OK);
    CHECK(psi_hip_id_allocator_alloc_many(allocator, 3u, ids) == PSI_HIP_OK);
    CHECK(ids[0] == 2u && ids[1] == 0u && ids[2] == 4u);
    uint64_t used = 0;
    CHECK(psi_hip_id_allocator_counts(allocator, &used, NULL, NULL) == PSI_HIP_OK && used == 5u);
    CHECK(psi_hip_id_allocator_destroy(allocator) == PSI_HIP_OK);

    /* page-table index math */
    psi_hip_page_table_layout layout = {4u, 3u, 6u, 2u};
    uint64_t index = 0;
    CHECK(psi_hip_page_table_start_index(&layout, 1u, 2u, 3u, &index) == PSI_HIP_OK && index == ((1u * 3u + 2u) * 6u + 3u) * 2u);

    printf("abi_c11 ok\n");
    return 0;
}
