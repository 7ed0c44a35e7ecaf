// Context, error reporting, geometry validation and per-kernel event timing.
#include <cstring>

#include "common.h"

namespace psi {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

// Mirrors the validate() chain of the reference configs
// (crates/inference-backend-metal/src/components/gqa_split_kv.rs:32-66,
//  gqa_kv_page_write.rs:50-70, gqa_split_kv_single_q.rs:61-92).
int make_geometry(const psi_hip_gqa_config* cfg, Geometry* g) {
    PSI_REQUIRE(cfg != nullptr, "GQA config must not be null");
    PSI_REQUIRE(cfg->num_q_heads > 0, "GQA num_q_heads must be positive");
    PSI_REQUIRE(cfg->num_kv_heads > 0, "GQA num_kv_heads must be positive");
    PSI_REQUIRE(cfg->head_dim > 0, "GQA head_dim must be positive");
    PSI_REQUIRE(cfg->num_q_heads % cfg->num_kv_heads == 0, "GQA num_q_heads must be a multiple of num_kv_heads");
    PSI_REQUIRE(cfg->page_bytes > 0, "GQA page_bytes must be positive");
    PSI_REQUIRE(cfg->dtype == PSI_HIP_F32 || cfg->dtype == PSI_HIP_BF16 || cfg->dtype == PSI_HIP_F16,
                "unsupported GQA dtype %u", cfg->dtype);
    const uint64_t per_token = (uint64_t)cfg->num_kv_heads * cfg->head_dim * 2u * dtype_size(cfg->dtype);
    PSI_REQUIRE(per_token <= UINT32_MAX, "GQA K/V bytes per token must fit u32");
    PSI_REQUIRE(cfg->page_bytes % per_token == 0, "GQA page_bytes must be divisible by the K/V bytes per token");
    g->hq = cfg->num_q_heads;
    g->hkv = cfg->num_kv_heads;
    g->d = cfg->head_dim;
    g->group = cfg->num_q_heads / cfg->num_kv_heads;
    g->elem = dtype_size(cfg->dtype);
    g->tokens_per_page = (uint32_t)(cfg->page_bytes / per_token);
    g->page_elems = cfg->page_bytes / g->elem;
    g->scale = cfg->scale;
    g->dtype = cfg->dtype;
    PSI_REQUIRE(g->tokens_per_page > 0, "GQA page must hold at least one token");
    return PSI_HIP_OK;
}

int check_layout(const psi_hip_page_table_layout* layout) {
    PSI_REQUIRE(layout != nullptr, "GQA page-table layout must not be null");
    PSI_REQUIRE(layout->num_req_slots > 0 && layout->num_gqa_layers > 0 && layout->num_blocks > 0 &&
                    layout->num_page_ids_per_block > 0,
                "GQA page-table layout dimensions must be positive");
    return PSI_HIP_OK;
}

LaunchScope::LaunchScope(psi_hip_ctx* ctx, const char* name) : ctx_(ctx) {
    if (!ctx->timing) return;
    timer_ = &ctx->timers[name];
    auto take = [&](hipEvent_t* ev) {
        if (!ctx->event_pool.empty()) {
            *ev = ctx->event_pool.back();
            ctx->event_pool.pop_back();
        } else if (hipEventCreate(ev) != hipSuccess) {
            *ev = nullptr;
        }
    };
    take(&start_);
    take(&stop_);
    if (start_ && stop_) (void)hipEventRecord(start_, ctx->stream);
}

LaunchScope::~LaunchScope() {
    if (!timer_ || !start_ || !stop_) return;
    (void)hipEventRecord(stop_, ctx_->stream);
    timer_->pending.emplace_back(start_, stop_);
}

}  // namespace psi

extern "C" {

const char* psi_hip_last_error(void) { return psi::g_error; }
const char* psi_hip_version(void) { return "psi-dec_amd 0.1 (gfx950)"; }

int psi_hip_ctx_create(int device, void* stream, psi_hip_ctx** out_ctx) {
    PSI_REQUIRE(out_ctx != nullptr, "out_ctx must not be null");
    int count = 0;
    PSI_HIP_CHECK(hipGetDeviceCount(&count));
    PSI_REQUIRE(device >= 0 && device < count, "device %d out of range (%d visible)", device, count);
    PSI_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    PSI_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return psi::fail(PSI_HIP_ERR_UNSUPPORTED, "device %d is %s; this library is built for gfx950 only", device,
                         prop.gcnArchName);
    // the built-in scratch of psi_hip_gqa_layer_record_static_scratch: its address on this GPU, looked up here,
    // with this GPU current, so that the entry point itself only launches
    int rc = psi::resolve_static_scratch(device);
    if (rc != PSI_HIP_OK) return rc;
    // the words in which kernels report what they could not compute: pinned host memory, so that reading them
    // after a synchronisation costs no copy
    void* status_host = nullptr;
    void* status_device = nullptr;
    PSI_HIP_CHECK(hipHostMalloc(&status_host, 64, hipHostMallocMapped));
    if (hipHostGetDevicePointer(&status_device, status_host, 0) != hipSuccess) {
        (void)hipHostFree(status_host);
        return psi::fail(PSI_HIP_ERR_RUNTIME, "the device status words cannot be mapped into device %d", device);
    }
    memset(status_host, 0, 64);
    void* work_claim = nullptr;
    if (hipMalloc(&work_claim, 64) != hipSuccess || hipMemset(work_claim, 0, 64) != hipSuccess) {
        (void)hipHostFree(status_host);
        if (work_claim != nullptr) (void)hipFree(work_claim);
        return psi::fail(PSI_HIP_ERR_RUNTIME, "no device memory for the context's work counters on device %d", device);
    }
    auto* ctx = new psi_hip_ctx();
    ctx->work_claim = static_cast<uint32_t*>(work_claim);
    ctx->num_cus = prop.multiProcessorCount;
    ctx->status_host = static_cast<volatile uint32_t*>(status_host);
    ctx->status_device = static_cast<uint32_t*>(status_device);
    ctx->device = device;
    ctx->stream = (hipStream_t)stream;
    *out_ctx = ctx;
    return PSI_HIP_OK;
}

int psi_hip_ctx_destroy(psi_hip_ctx* ctx) {
    if (!ctx) return PSI_HIP_OK;
    for (auto& kv : ctx->timers)
        for (auto& p : kv.second.pending) {
            (void)hipEventDestroy(p.first);
            (void)hipEventDestroy(p.second);
        }
    for (auto ev : ctx->event_pool) (void)hipEventDestroy(ev);
    if (ctx->status_host != nullptr) (void)hipHostFree(const_cast<uint32_t*>(ctx->status_host));
    if (ctx->work_claim != nullptr) (void)hipFree(ctx->work_claim);
    if (ctx->order_event != nullptr) (void)hipEventDestroy(ctx->order_event);
    delete ctx;
    return PSI_HIP_OK;
}

int psi_hip_ctx_set_stream(psi_hip_ctx* ctx, void* stream) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    const hipStream_t next = (hipStream_t)stream;
    if (next == ctx->stream) return PSI_HIP_OK;
    // What the context has launched on the old stream stays ahead of what it launches on the new one: its launches
    // share the context's work counters and the arena the caller hands them, and rely on running one after the other.
    // (A stream that is being captured takes no dependency on work outside its capture, and the other way round:
    // there the order is the capturing caller's.)
    hipStreamCaptureStatus from = hipStreamCaptureStatusNone, to = hipStreamCaptureStatusNone;
    const bool plain = hipStreamIsCapturing(ctx->stream, &from) == hipSuccess &&
                       hipStreamIsCapturing(next, &to) == hipSuccess && from == hipStreamCaptureStatusNone &&
                       to == hipStreamCaptureStatusNone;
    if (plain) {
        if (ctx->order_event == nullptr)
            PSI_HIP_CHECK(hipEventCreateWithFlags(&ctx->order_event, hipEventDisableTiming));
        PSI_HIP_CHECK(hipEventRecord(ctx->order_event, ctx->stream));
        PSI_HIP_CHECK(hipStreamWaitEvent(next, ctx->order_event, 0));
    } else {
        (void)hipGetLastError();
    }
    ctx->stream = next;
    return PSI_HIP_OK;
}

static uint32_t device_error_bits(const psi_hip_ctx* ctx) {
    uint32_t bits = 0;
    for (uint32_t i = 0; i < psi::kDeviceStatusWords; ++i)
        if (ctx->status_host[i] != 0) bits |= 1u << i;
    return bits;
}

static int report_device_error(uint32_t bits) {
    if (bits == 0) return PSI_HIP_OK;
    return psi::fail(PSI_HIP_ERR_RUNTIME, "a kernel reported an error (bits 0x%x):%s%s; the affected partial rows are empty states",
                     bits, (bits & PSI_HIP_DEVICE_ERR_WAIT_GAVE_UP) ? " a bounded wait between waves ran out" : "",
                     (bits & PSI_HIP_DEVICE_ERR_V_RANGE) ? " the prefill-chunk map met V values outside the f16 range" : "");
}

int psi_hip_sync(psi_hip_ctx* ctx) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    PSI_HIP_CHECK(hipStreamSynchronize(ctx->stream));
    return report_device_error(device_error_bits(ctx));
}

int psi_hip_ctx_take_device_error(psi_hip_ctx* ctx, uint32_t* out_bits) {
    PSI_REQUIRE(ctx != nullptr && out_bits != nullptr, "ctx and out_bits must not be null");
    PSI_HIP_CHECK(hipStreamSynchronize(ctx->stream));
    *out_bits = device_error_bits(ctx);
    for (uint32_t i = 0; i < psi::kDeviceStatusWords; ++i) ctx->status_host[i] = 0;
    return PSI_HIP_OK;
}

int psi_hip_ctx_bind_replay_counts(psi_hip_ctx* ctx, const uint32_t* device_counts) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    ctx->replay_counts = device_counts;
    return PSI_HIP_OK;
}

int psi_hip_ctx_set_flag(psi_hip_ctx* ctx, uint32_t flag, uint32_t value) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    switch (flag) {
        case PSI_HIP_FLAG_FORCE_GENERIC: ctx->force_generic = value != 0; break;
        case PSI_HIP_FLAG_F32_OUTPUT: ctx->f32_output = value != 0; break;
        case PSI_HIP_FLAG_MUTE_LOADERS: ctx->mute_loaders = value != 0; break;
        default: return psi::fail(PSI_HIP_ERR_INVALID_ARGUMENT, "unknown context flag %u", flag);
    }
    return PSI_HIP_OK;
}

int psi_hip_ctx_set_timing(psi_hip_ctx* ctx, int enabled) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    ctx->timing = enabled != 0;
    return PSI_HIP_OK;
}

static int drain(psi_hip_ctx* ctx, psi::KernelTimer& t) {
    for (auto& p : t.pending) {
        PSI_HIP_CHECK(hipEventSynchronize(p.second));
        float ms = 0;
        PSI_HIP_CHECK(hipEventElapsedTime(&ms, p.first, p.second));
        t.total_ms += ms;
        t.launches += 1;
        ctx->event_pool.push_back(p.first);
        ctx->event_pool.push_back(p.second);
    }
    t.pending.clear();
    return PSI_HIP_OK;
}

int psi_hip_ctx_kernel_time_ms(psi_hip_ctx* ctx, const char* kernel, double* out_total_ms, uint64_t* out_launches) {
    PSI_REQUIRE(ctx != nullptr && kernel != nullptr, "ctx and kernel name must not be null");
    auto it = ctx->timers.find(kernel);
    if (it == ctx->timers.end()) {
        if (out_total_ms) *out_total_ms = 0;
        if (out_launches) *out_launches = 0;
        return PSI_HIP_OK;
    }
    int rc = drain(ctx, it->second);
    if (rc != PSI_HIP_OK) return rc;
    if (out_total_ms) *out_total_ms = it->second.total_ms;
    if (out_launches) *out_launches = it->second.launches;
    return PSI_HIP_OK;
}

int psi_hip_ctx_reset_timing(psi_hip_ctx* ctx) {
    PSI_REQUIRE(ctx != nullptr, "ctx must not be null");
    for (auto& kv : ctx->timers) {
        int rc = drain(ctx, kv.second);
        if (rc != PSI_HIP_OK) return rc;
        kv.second.total_ms = 0;
        kv.second.launches = 0;
    }
    return PSI_HIP_OK;
}

int psi_hip_gqa_tokens_per_page(const psi_hip_gqa_config* cfg, uint32_t* out_tokens_per_page) {
    psi::Geometry g;
    int rc = psi::make_geometry(cfg, &g);
    if (rc != PSI_HIP_OK) return rc;
    PSI_REQUIRE(out_tokens_per_page != nullptr, "out pointer must not be null");
    *out_tokens_per_page = g.tokens_per_page;
    return PSI_HIP_OK;
}

}  // extern "C"
