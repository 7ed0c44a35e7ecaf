// KV append: scatters the projected K and V of the current tokens into their pages through the
// request page table.  Replaces crates/inference-backend-metal/src/components/metal/gqa_kv_page_write.metal:5-53
// (one thread per element there); here one work-item moves one 16-byte chunk of a
// (token, K|V, kv_head) line, so a 512-byte line is written by 32 adjacent lanes with 128-bit
// stores.  Pure bit copy: the destination bytes equal the source bytes.
#include "common.h"
#include "device_types.h"

namespace psi {

struct PageWriteArgs {
    void* pages;
    const void* flat_k;
    const void* flat_v;
    const uint32_t* req_slots;
    const uint32_t* flat_token_indices;
    const uint32_t* page_ids;
    uint32_t num_active;
    uint32_t layer;
    uint32_t num_layers, num_blocks, ids_per_block;
    uint32_t hkv, d, tokens_per_page;
    uint64_t page_elems;
    uint32_t units_per_line;  // chunks (vector path) or elements (scalar path) per (token, head) line
    const uint32_t* replay_counts;  // see active_count()
};

// Element offset of (kind, head, token, 0) -- the index contract shared with the attention
// kernels (gqa_kv_page_write.metal:29-47).
__device__ __forceinline__ uint64_t line_offset(const PageWriteArgs& a, uint32_t write, uint32_t kind, uint32_t head) {
    const uint32_t req_slot = a.req_slots[write];
    const uint32_t token = a.flat_token_indices[write];
    const uint32_t block = token / (a.tokens_per_page * a.ids_per_block);
    const uint32_t id_index = (token / a.tokens_per_page) % a.ids_per_block;
    const uint32_t page_token = token % a.tokens_per_page;
    const uint64_t table_index =
        (((uint64_t)req_slot * a.num_layers + active_layer(a.replay_counts, a.layer, a.num_layers)) * a.num_blocks + block) *
            a.ids_per_block +
        id_index;
    const uint64_t page_id = a.page_ids[table_index];
    return page_id * a.page_elems + (((uint64_t)kind * a.hkv + head) * a.tokens_per_page + page_token) * a.d;
}

template <typename Unit, int kUnitsAreChunks>
__global__ __launch_bounds__(256) void kv_page_write_kernel(PageWriteArgs a, uint32_t elems_per_unit) {
    const uint32_t per_write = 2u * a.hkv * a.units_per_line;
    const uint64_t gid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= (uint64_t)active_count(a.replay_counts, kReplayTokens, a.num_active) * per_write) return;
    const uint32_t write = (uint32_t)(gid / per_write);
    uint32_t rest = (uint32_t)(gid - (uint64_t)write * per_write);
    const uint32_t kind = rest / (a.hkv * a.units_per_line);
    rest -= kind * a.hkv * a.units_per_line;
    const uint32_t head = rest / a.units_per_line;
    const uint32_t unit = rest - head * a.units_per_line;
    const uint64_t dst_elem = line_offset(a, write, kind, head) + (uint64_t)unit * elems_per_unit;
    const uint64_t src_elem = ((uint64_t)write * a.hkv + head) * a.d + (uint64_t)unit * elems_per_unit;
    const Unit* src = reinterpret_cast<const Unit*>(kind ? a.flat_v : a.flat_k);
    Unit* dst = reinterpret_cast<Unit*>(a.pages);
    dst[dst_elem / elems_per_unit] = src[src_elem / elems_per_unit];
}

}  // namespace psi

extern "C" int psi_hip_kv_page_write(psi_hip_ctx* ctx, const psi_hip_gqa_config* cfg,
                                     const psi_hip_page_table_layout* layout, void* pages, uint64_t pages_bytes,
                                     const void* flat_k, const void* flat_v, const uint32_t* req_slots,
                                     const uint32_t* flat_token_indices, const uint32_t* page_ids,
                                     uint32_t num_total_token_writes, uint32_t num_active_token_writes,
                                     uint32_t gqa_layer_index) {
    using namespace psi;
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    Geometry g;
    int rc = make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    rc = check_layout(layout);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(pages && flat_k && flat_v && req_slots && flat_token_indices && page_ids,
                "GQA KV page-write buffers must not be null");
    // gqa_kv_page_write.rs:104-112, :208-216
    PSI_REQUIRE(num_total_token_writes > 0, "GQA KV page-write requires token writes");
    PSI_REQUIRE((uint64_t)num_total_token_writes * g.hkv * g.d <= UINT32_MAX,
                "GQA KV page-write threads exceeds the shader u32 count domain: count=%llu",
                (unsigned long long)((uint64_t)num_total_token_writes * g.hkv * g.d));
    PSI_REQUIRE(num_active_token_writes > 0, "GQA KV page-write active count must be positive");
    PSI_REQUIRE(num_active_token_writes <= num_total_token_writes,
                "GQA KV page-write active count exceeds recorded capacity");
    PSI_REQUIRE(gqa_layer_index < layout->num_gqa_layers, "GQA page-table index exceeds layer count");
    PSI_REQUIRE(pages_bytes == 0 || pages_bytes >= cfg->page_bytes, "GQA page arena is smaller than one page");

    PageWriteArgs a;
    a.pages = pages;
    a.flat_k = flat_k;
    a.flat_v = flat_v;
    a.req_slots = req_slots;
    a.flat_token_indices = flat_token_indices;
    a.page_ids = page_ids;
    a.num_active = num_active_token_writes;
    a.replay_counts = ctx->replay_counts;
    a.layer = gqa_layer_index;
    a.num_layers = layout->num_gqa_layers;
    a.num_blocks = layout->num_blocks;
    a.ids_per_block = layout->num_page_ids_per_block;
    a.hkv = g.hkv;
    a.d = g.d;
    a.tokens_per_page = g.tokens_per_page;
    a.page_elems = g.page_elems;

    const uint32_t line_bytes = g.d * g.elem;
    const bool aligned16 = line_bytes % 16 == 0 && (reinterpret_cast<uintptr_t>(pages) % 16 == 0) &&
                           (reinterpret_cast<uintptr_t>(flat_k) % 16 == 0) &&
                           (reinterpret_cast<uintptr_t>(flat_v) % 16 == 0);
    LaunchScope scope(ctx, "kv_page_write");
    if (aligned16) {
        a.units_per_line = line_bytes / 16;
        const uint64_t total = (uint64_t)num_active_token_writes * 2u * g.hkv * a.units_per_line;
        const uint32_t grid = (uint32_t)((total + 255) / 256);
        hipLaunchKernelGGL((kv_page_write_kernel<uint4, 1>), dim3(grid), dim3(256), 0, ctx->stream, a, 16u / g.elem);
    } else {
        a.units_per_line = g.d;
        const uint64_t total = (uint64_t)num_active_token_writes * 2u * g.hkv * g.d;
        const uint32_t grid = (uint32_t)((total + 255) / 256);
        if (g.elem == 4)
            hipLaunchKernelGGL((kv_page_write_kernel<uint32_t, 0>), dim3(grid), dim3(256), 0, ctx->stream, a, 1u);
        else
            hipLaunchKernelGGL((kv_page_write_kernel<uint16_t, 0>), dim3(grid), dim3(256), 0, ctx->stream, a, 1u);
    }
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}
