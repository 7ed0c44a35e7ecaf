// Request page table helpers: the table itself is a caller-owned device buffer of u32 page IDs,
// [num_req_slots][num_gqa_layers][num_blocks][num_page_ids_per_block]; these entry points do the
// index arithmetic and the small host-to-device updates.  Follows
// crates/inference-executor-metal/src/attn/gqa/request_page_table.rs:8-122.
#include "common.h"

using namespace psi;

static int check_row(const psi_hip_page_table_layout* layout, uint32_t req_slot, uint32_t layer_index,
                     uint32_t block_index) {
    int rc = check_layout(layout);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(req_slot < layout->num_req_slots,
                "GQA request page table req_slot out of range: req_slot=%u num_req_slots=%u", req_slot,
                layout->num_req_slots);
    PSI_REQUIRE(layer_index < layout->num_gqa_layers,
                "GQA request page table layer out of range: layer_index=%u num_layers=%u", layer_index,
                layout->num_gqa_layers);
    PSI_REQUIRE(block_index < layout->num_blocks,
                "GQA request page table block out of range: block_index=%u num_blocks=%u", block_index,
                layout->num_blocks);
    return PSI_HIP_OK;
}

extern "C" int psi_hip_page_table_start_index(const psi_hip_page_table_layout* layout, uint32_t req_slot,
                                              uint32_t layer_index, uint32_t block_index, uint64_t* out_index) {
    int rc = check_row(layout, req_slot, layer_index, block_index);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_index != nullptr, "out pointer must not be null");
    *out_index = (((uint64_t)req_slot * layout->num_gqa_layers + layer_index) * layout->num_blocks + block_index) *
                 layout->num_page_ids_per_block;
    return PSI_HIP_OK;
}

extern "C" int psi_hip_page_table_write_page_ids(psi_hip_ctx* ctx, const psi_hip_page_table_layout* layout,
                                                 uint32_t* page_ids_device, uint32_t req_slot, uint32_t layer_index,
                                                 uint32_t block_index, const uint32_t* ids, uint32_t count,
                                                 uint32_t num_cache_pages) {
    PSI_REQUIRE(ctx != nullptr && page_ids_device != nullptr && ids != nullptr, "page-table pointers must not be null");
    uint64_t start;
    int rc = psi_hip_page_table_start_index(layout, req_slot, layer_index, block_index, &start);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(count == layout->num_page_ids_per_block,
                "GQA page-id count must match one request/GQA-layer/block entry");
    if (num_cache_pages > 0)
        for (uint32_t i = 0; i < count; ++i)
            PSI_REQUIRE(ids[i] < num_cache_pages, "GQA page id %u exceeds the cache page count %u", ids[i],
                        num_cache_pages);
    // The source is pageable host memory: the runtime stages it before returning, so the caller
    // may reuse `ids` immediately.
    PSI_HIP_CHECK(hipMemcpyAsync(page_ids_device + start, ids, (size_t)count * sizeof(uint32_t),
                                 hipMemcpyHostToDevice, ctx->stream));
    return PSI_HIP_OK;
}

extern "C" int psi_hip_page_table_reset_req_slot(psi_hip_ctx* ctx, const psi_hip_page_table_layout* layout,
                                                 uint32_t* page_ids_device, uint32_t req_slot) {
    PSI_REQUIRE(ctx != nullptr && page_ids_device != nullptr, "page-table pointers must not be null");
    uint64_t start;
    int rc = psi_hip_page_table_start_index(layout, req_slot, 0, 0, &start);
    if (rc != PSI_HIP_OK) return rc;
    const size_t per_request =
        (size_t)layout->num_gqa_layers * layout->num_blocks * layout->num_page_ids_per_block * sizeof(uint32_t);
    PSI_HIP_CHECK(hipMemsetAsync(page_ids_device + start, 0, per_request, ctx->stream));
    return PSI_HIP_OK;
}

extern "C" int psi_hip_page_ids_by_layer(const uint32_t* block_ids, uint32_t block_ids_len, uint32_t num_gqa_layers,
                                         uint32_t num_page_ids_per_block, uint32_t* out_by_layer) {
    PSI_REQUIRE(block_ids != nullptr && out_by_layer != nullptr, "page-id arrays must not be null");
    PSI_REQUIRE((uint64_t)num_gqa_layers * num_page_ids_per_block == block_ids_len,
                "expects %llu page ids for each synced kv block, got %u",
                (unsigned long long)((uint64_t)num_gqa_layers * num_page_ids_per_block), block_ids_len);
    // The runtime's per-block list is already layer-major: layer l owns [l*ids, (l+1)*ids).
    for (uint32_t i = 0; i < block_ids_len; ++i) out_by_layer[i] = block_ids[i];
    return PSI_HIP_OK;
}
