// Selected entries of a device buffer (pages of the arena, request rows of the page table) packed into one
// contiguous payload in HBM, and restored from it.  The payload is what a state snapshot stores: the byte
// ranges [begin * entry_bytes, end * entry_bytes) of each selected entry range, concatenated in order
// (crates/inference-executor-metal/src/model/state_snapshot.rs:249-304 and :743-776; used for the page arena by
// model/page_arena/file_io.rs:28-49 and for the page table by attn/gqa/request_page_table/file_io.rs:28-59).
// The reference streams each range between unified memory and a file; on a discrete GPU the ranges are first
// gathered on the device so that one large transfer crosses the host link instead of one per range.
#include <algorithm>

#include "common.h"

namespace psi {

constexpr int kRangesPerLaunch = 128;
constexpr uint64_t kBytesPerWorkgroup = 64 * 1024;  // of the longest range of a launch; shorter ranges finish early
constexpr uint32_t kMaxWorkgroupsPerRange = 2048;

// A batch of ranges handed over with the launch: no table in device memory, nothing to upload.
struct RangeBatch {
    uint64_t buffer_offset[kRangesPerLaunch];   // bytes
    uint64_t payload_offset[kRangesPerLaunch];  // bytes
    uint64_t bytes[kRangesPerLaunch];
};

// kToPayload: buffer -> payload, else payload -> buffer.  Unit: the widest of 16, 4, 1 bytes that divides every
// offset and length of the call.
template <typename Unit, bool kToPayload>
__global__ __launch_bounds__(256) void move_ranges_kernel(RangeBatch batch, char* buffer, char* payload) {
    const uint32_t r = blockIdx.y;
    const uint64_t units = batch.bytes[r] / sizeof(Unit);
    Unit* in_buffer = reinterpret_cast<Unit*>(buffer + batch.buffer_offset[r]);
    Unit* in_payload = reinterpret_cast<Unit*>(payload + batch.payload_offset[r]);
    const Unit* src = kToPayload ? in_buffer : in_payload;
    Unit* dst = kToPayload ? in_payload : in_buffer;
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < units; i += (uint64_t)gridDim.x * 256)
        dst[i] = src[i];
}

// The canonical form the reference asserts (state_snapshot.rs:774-776): every range non-empty, ranges sorted,
// disjoint and not adjacent; and each inside the buffer (:762-768).
static int check_ranges(const uint32_t* entry_ranges, uint32_t num_ranges, uint64_t entry_bytes, uint64_t buffer_bytes,
                        uint64_t* payload_bytes) {
    PSI_REQUIRE(entry_bytes > 0, "model state snapshot buffer entry size must be positive");
    PSI_REQUIRE(num_ranges == 0 || entry_ranges != nullptr, "entry ranges must not be null");
    uint64_t total = 0;
    for (uint32_t r = 0; r < num_ranges; ++r) {
        const uint32_t begin = entry_ranges[2 * r], end = entry_ranges[2 * r + 1];
        PSI_REQUIRE(begin < end && (r == 0 || entry_ranges[2 * r - 1] < begin),
                    "model state snapshot buffer entry ranges must be nonempty, sorted, disjoint, and nonadjacent");
        PSI_REQUIRE((uint64_t)end * entry_bytes <= buffer_bytes,
                    "model state snapshot buffer entry range is out of bounds: entry_range=%u..%u entry_bytes=%llu "
                    "buffer_bytes=%llu",
                    begin, end, (unsigned long long)entry_bytes, (unsigned long long)buffer_bytes);
        total += (uint64_t)(end - begin) * entry_bytes;
    }
    if (payload_bytes != nullptr) *payload_bytes = total;
    return PSI_HIP_OK;
}

template <bool kToPayload>
static int move_ranges(psi_hip_ctx* ctx, void* buffer, uint64_t buffer_bytes, const uint32_t* entry_ranges,
                       uint32_t num_ranges, uint64_t entry_bytes, void* payload, uint64_t payload_bytes) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    uint64_t needed = 0;
    int rc = check_ranges(entry_ranges, num_ranges, entry_bytes, buffer_bytes, &needed);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(payload_bytes == needed, "model state snapshot file length mismatch: expected=%llu actual=%llu",
                (unsigned long long)needed, (unsigned long long)payload_bytes);
    if (num_ranges == 0) return PSI_HIP_OK;
    PSI_REQUIRE(buffer != nullptr && payload != nullptr, "snapshot buffers must not be null");
    const uint64_t both = reinterpret_cast<uintptr_t>(buffer) | reinterpret_cast<uintptr_t>(payload) | entry_bytes;
    const int unit = both % 16 == 0 ? 16 : both % 4 == 0 ? 4 : 1;

    LaunchScope scope(ctx, kToPayload ? "state_pack_ranges" : "state_unpack_ranges");
    uint64_t payload_offset = 0;
    for (uint32_t first = 0; first < num_ranges; first += kRangesPerLaunch) {
        const uint32_t count = std::min<uint32_t>(kRangesPerLaunch, num_ranges - first);
        RangeBatch batch = {};
        uint64_t longest = 0;
        for (uint32_t i = 0; i < count; ++i) {
            const uint32_t begin = entry_ranges[2 * (first + i)], end = entry_ranges[2 * (first + i) + 1];
            batch.buffer_offset[i] = (uint64_t)begin * entry_bytes;
            batch.payload_offset[i] = payload_offset;
            batch.bytes[i] = (uint64_t)(end - begin) * entry_bytes;
            payload_offset += batch.bytes[i];
            longest = std::max(longest, batch.bytes[i]);
        }
        const dim3 grid((uint32_t)std::min<uint64_t>((longest + kBytesPerWorkgroup - 1) / kBytesPerWorkgroup,
                                                     kMaxWorkgroupsPerRange),
                        count);
        char* b = static_cast<char*>(buffer);
        char* p = static_cast<char*>(payload);
        if (unit == 16)
            hipLaunchKernelGGL((move_ranges_kernel<uint4, kToPayload>), grid, dim3(256), 0, ctx->stream, batch, b, p);
        else if (unit == 4)
            hipLaunchKernelGGL((move_ranges_kernel<uint32_t, kToPayload>), grid, dim3(256), 0, ctx->stream, batch, b, p);
        else
            hipLaunchKernelGGL((move_ranges_kernel<uint8_t, kToPayload>), grid, dim3(256), 0, ctx->stream, batch, b, p);
    }
    PSI_HIP_CHECK(hipGetLastError());
    return PSI_HIP_OK;
}

}  // namespace psi

using namespace psi;

extern "C" int psi_hip_selected_ranges_payload_bytes(const uint32_t* entry_ranges, uint32_t num_ranges,
                                                     uint64_t entry_bytes, uint64_t buffer_bytes,
                                                     uint64_t* out_payload_bytes) {
    PSI_REQUIRE(out_payload_bytes != nullptr, "out pointer must not be null");
    return check_ranges(entry_ranges, num_ranges, entry_bytes, buffer_bytes, out_payload_bytes);
}

extern "C" int psi_hip_buffer_pack_selected(psi_hip_ctx* ctx, const void* buffer, uint64_t buffer_bytes,
                                            const uint32_t* entry_ranges, uint32_t num_ranges, uint64_t entry_bytes,
                                            void* payload, uint64_t payload_bytes) {
    return move_ranges<true>(ctx, const_cast<void*>(buffer), buffer_bytes, entry_ranges, num_ranges, entry_bytes,
                             payload, payload_bytes);
}

extern "C" int psi_hip_buffer_unpack_selected(psi_hip_ctx* ctx, void* buffer, uint64_t buffer_bytes,
                                              const uint32_t* entry_ranges, uint32_t num_ranges, uint64_t entry_bytes,
                                              const void* payload, uint64_t payload_bytes) {
    return move_ranges<false>(ctx, buffer, buffer_bytes, entry_ranges, num_ranges, entry_bytes,
                              const_cast<void*>(payload), payload_bytes);
}
