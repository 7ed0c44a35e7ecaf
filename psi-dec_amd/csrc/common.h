// Shared host-side helpers of the paged-attention library: error reporting, config checks,
// launch bookkeeping.  Host code only; kernels live in the *.hip files.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <string>
#include <vector>

#include "../../include/psi_hip.h"

namespace psi {

// Thread-local message behind psi_hip_last_error().
void set_error(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define PSI_REQUIRE(cond, ...)                                         \
    do {                                                               \
        if (!(cond)) return ::psi::fail(PSI_HIP_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

#define PSI_HIP_CHECK(expr)                                                                       \
    do {                                                                                          \
        hipError_t e_ = (expr);                                                                   \
        if (e_ != hipSuccess)                                                                     \
            return ::psi::fail(PSI_HIP_ERR_RUNTIME, "%s failed: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

inline uint32_t dtype_size(uint32_t dtype) { return dtype == PSI_HIP_F32 ? 4u : 2u; }

// Derived geometry, validated once per call.
struct Geometry {
    uint32_t hq, hkv, d, group, tokens_per_page, elem;
    uint64_t page_elems;
    float scale;
    uint32_t dtype;
};

int make_geometry(const psi_hip_gqa_config* cfg, Geometry* g);
// Device address of the library's built-in partial-state array on `device` (the calling thread's current device).
int resolve_static_scratch(int device);
int check_layout(const psi_hip_page_table_layout* layout);

constexpr uint32_t kDeviceStatusWords = 2;
constexpr uint32_t kDefaultWaitPolls = 1u << 16;

struct KernelTimer {
    double total_ms = 0;
    uint64_t launches = 0;
    std::vector<std::pair<hipEvent_t, hipEvent_t>> pending;
};

}  // namespace psi

struct psi_hip_ctx {
    int device = 0;
    hipStream_t stream = nullptr;
    bool timing = false;
    bool force_generic = false;  // route every launch to the shape-generic kernels
    bool f32_output = false;     // combine kernels store f32 instead of the io dtype
    // Device u32[4] = {active tokens, active Q-token tiles, active KV splits, reserved} read by every
    // kernel when it runs (graph replay); null: the counts passed by value apply.
    const uint32_t* replay_counts = nullptr;
    // Errors found by running kernels: kDeviceStatusWords words of pinned host memory mapped into the GPU's address
    // space (word i set to 1 by a kernel = bit i of the PSI_HIP_DEVICE_ERR_* mask).  One word per kind, written
    // with plain stores: nothing on the GPU reads or clears them.
    volatile uint32_t* status_host = nullptr;
    uint32_t* status_device = nullptr;
    // Two zeroed words of device memory through which the workgroups of a prefill-chunk map launch share out its work
    // items; the launch leaves them zero again.  One launch at a time uses them: the context's launches run on its
    // stream, one after the other.
    uint32_t* work_claim = nullptr;
    int num_cus = 0;  // compute units of the device
    hipEvent_t order_event = nullptr;  // psi_hip_ctx_set_stream: the old stream's work before the new stream's
    bool mute_loaders = false;  // harness switch: the maps' loading waves announce nothing, so that waits run out
    std::map<std::string, psi::KernelTimer> timers;
    std::vector<hipEvent_t> event_pool;
};

namespace psi {

// RAII bracket: records events around one launch when timing is on.
class LaunchScope {
  public:
    LaunchScope(psi_hip_ctx* ctx, const char* name);
    ~LaunchScope();

  private:
    psi_hip_ctx* ctx_;
    KernelTimer* timer_ = nullptr;
    hipEvent_t start_ = nullptr, stop_ = nullptr;
};

}  // namespace psi
