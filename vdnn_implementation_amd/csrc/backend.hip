// Context, pooled device memory, streams, events and copies of the device back end.
#include "backend_internal.h"

#include <cstring>

namespace vdnn {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

hipEvent_t prof_take_event(vdnn_ctx* ctx) {
    if (!ctx->prof_free_events.empty()) {
        hipEvent_t e = ctx->prof_free_events.back();
        ctx->prof_free_events.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}

// Virtual base of a plan-only pool: never dereferenced, only used for offset arithmetic.
static constexpr uintptr_t kPlanBase = uintptr_t(1) << 44;

} // namespace vdnn

using namespace vdnn;

extern "C" {

const char* vdnn_last_error(void) { return g_error; }

int vdnn_ctx_create(vdnn_ctx** out, int device, int flags) {
    if (!out) { set_error("vdnn_ctx_create: null out"); return VDNN_EINVAL; }
    *out = nullptr;
    vdnn_ctx* ctx = new vdnn_ctx();
    ctx->device = device;
    ctx->plan_only = (flags & VDNN_CTX_PLAN_ONLY) != 0;
    if (!ctx->plan_only) {
        hipError_t e = hipSetDevice(device);
        if (e != hipSuccess) {
            set_error("hipSetDevice(%d) failed: %s", device, hipGetErrorString(e));
            delete ctx;
            return VDNN_EDEVICE;
        }
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, device) == hipSuccess) ctx->num_cu = prop.multiProcessorCount;
        // default priority on every stream
        if (hipStreamCreateWithFlags(&ctx->compute, hipStreamNonBlocking) != hipSuccess ||
            hipStreamCreateWithFlags(&ctx->d2h, hipStreamNonBlocking) != hipSuccess ||
            hipStreamCreateWithFlags(&ctx->h2d, hipStreamNonBlocking) != hipSuccess ||
            hipStreamCreateWithFlags(&ctx->pack, hipStreamNonBlocking) != hipSuccess) {
            set_error("hipStreamCreate failed");
            delete ctx;
            return VDNN_EDEVICE;
        }
        if (noalloc_prepare_current_device() != VDNN_OK) {
            delete ctx;
            return VDNN_EDEVICE;
        }
    }
    *out = ctx;
    return VDNN_OK;
}

int vdnn_ctx_set_activation_dtype(vdnn_ctx* ctx, int dtype) {
    VDNN_REQUIRE(ctx != nullptr, "null context");
    VDNN_REQUIRE(dtype == VDNN_DTYPE_F32 || dtype == VDNN_DTYPE_BF16, "unknown element type");
    ctx->act_dtype = dtype;
    return VDNN_OK;
}

int vdnn_ctx_activation_dtype(vdnn_ctx* ctx) { return ctx ? ctx->act_dtype : VDNN_DTYPE_F32; }

int vdnn_ctx_destroy(vdnn_ctx* ctx) {
    if (!ctx) return VDNN_OK;
    vdnn_pool_finalize(ctx);
    if (!ctx->plan_only) {
        (void)hipDeviceSynchronize();
        for (auto& r : ctx->prof_records) { (void)hipEventDestroy(r.start); (void)hipEventDestroy(r.stop); }
        for (auto e : ctx->prof_free_events) (void)hipEventDestroy(e);
        if (ctx->zvc_counters) (void)hipFree(ctx->zvc_counters);
        if (ctx->compute) (void)hipStreamDestroy(ctx->compute);
        if (ctx->d2h) (void)hipStreamDestroy(ctx->d2h);
        if (ctx->h2d) (void)hipStreamDestroy(ctx->h2d);
        if (ctx->pack) (void)hipStreamDestroy(ctx->pack);
    }
    delete ctx;
    return VDNN_OK;
}

int vdnn_device_mem_info(vdnn_ctx* ctx, size_t* free_bytes, size_t* total_bytes) {
    VDNN_REQUIRE(ctx && free_bytes && total_bytes, "null argument");
    if (ctx->plan_only) {
        *total_bytes = size_t(288) << 30; // MI355X HBM3E
        *free_bytes = *total_bytes;
        return VDNN_OK;
    }
    VDNN_HIP(hipMemGetInfo(free_bytes, total_bytes));
    return VDNN_OK;
}

int vdnn_device_synchronize(vdnn_ctx* ctx) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only) return VDNN_OK;
    VDNN_HIP(hipDeviceSynchronize());
    return VDNN_OK;
}

vdnn_stream_t vdnn_ctx_stream_compute(vdnn_ctx* ctx) { return ctx ? ctx->compute : nullptr; }
vdnn_stream_t vdnn_ctx_stream_d2h(vdnn_ctx* ctx) { return ctx ? ctx->d2h : nullptr; }
vdnn_stream_t vdnn_ctx_stream_h2d(vdnn_ctx* ctx) { return ctx ? ctx->h2d : nullptr; }
vdnn_stream_t vdnn_ctx_stream_pack(vdnn_ctx* ctx) { return ctx ? ctx->pack : nullptr; }

/* ---- pool ----------------------------------------------------------------------------------- */
int vdnn_pool_init(vdnn_ctx* ctx, size_t bytes) {
    VDNN_REQUIRE(ctx, "null context");
    VDNN_REQUIRE(!ctx->pool.initialised(), "pool already initialised");
    VDNN_REQUIRE(bytes > kReduceScratchBytes, "pool smaller than the reduction staging area");
    if (ctx->plan_only) {
        ctx->pool.init(kPlanBase, bytes);
    } else {
        hipError_t e = hipMalloc(&ctx->pool_base, bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            set_error("vdnn_pool_init: hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
            ctx->pool_base = nullptr;
            return VDNN_OOM;
        }
        ctx->pool.init((uintptr_t)ctx->pool_base, bytes);
    }
    uintptr_t s = ctx->pool.allocate(kReduceScratchBytes);
    ctx->reduce_scratch = (float*)s;
    ctx->reduce_scratch_bytes = kReduceScratchBytes - kBiasScratchBytes;
    ctx->bias_scratch = (float*)(s + ctx->reduce_scratch_bytes);
    ctx->bias_scratch_bytes = kBiasScratchBytes;
    return VDNN_OK;
}

int vdnn_pool_finalize(vdnn_ctx* ctx) {
    VDNN_REQUIRE(ctx, "null context");
    if (!ctx->pool.initialised()) return VDNN_OK;
    if (!ctx->plan_only && ctx->pool_base) {
        (void)hipDeviceSynchronize();
        (void)hipFree(ctx->pool_base);
    }
    ctx->pool_base = nullptr;
    ctx->reduce_scratch = nullptr;
    ctx->reduce_scratch_bytes = 0;
    ctx->bias_scratch = nullptr;
    ctx->bias_scratch_bytes = 0;
    ctx->pool.clear();
    return VDNN_OK;
}

int vdnn_pool_malloc(vdnn_ctx* ctx, void** ptr, size_t bytes) {
    VDNN_REQUIRE(ctx && ptr, "null argument");
    VDNN_REQUIRE(ctx->pool.initialised(), "pool not initialised");
    uintptr_t p = ctx->pool.allocate(bytes);
    if (!p) {
        *ptr = nullptr;
        set_error("vdnn_pool_malloc: out of memory for %zu bytes (in use %zu of %zu, cap %zu, largest free %zu)",
                  bytes, ctx->pool.in_use(), ctx->pool.total(), ctx->pool.cap(), ctx->pool.largest_free());
        return VDNN_OOM;
    }
    *ptr = (void*)p;
    return VDNN_OK;
}

int vdnn_pool_free(vdnn_ctx* ctx, void* ptr) {
    VDNN_REQUIRE(ctx, "null context");
    if (!ptr) return VDNN_OK;
    VDNN_REQUIRE(ctx->pool.release((uintptr_t)ptr), "pointer is not a live pool block");
    return VDNN_OK;
}

int vdnn_pool_info(vdnn_ctx* ctx, size_t* free_bytes, size_t* total_bytes) {
    VDNN_REQUIRE(ctx && free_bytes && total_bytes, "null argument");
    *total_bytes = ctx->pool.total();
    *free_bytes = ctx->pool.total() - ctx->pool.in_use();
    return VDNN_OK;
}

int vdnn_pool_peak(vdnn_ctx* ctx, size_t* peak_in_use, size_t* peak_extent) {
    VDNN_REQUIRE(ctx, "null context");
    if (peak_in_use) *peak_in_use = ctx->pool.peak_in_use();
    if (peak_extent) *peak_extent = ctx->pool.peak_extent();
    return VDNN_OK;
}

int vdnn_pool_reset_peak(vdnn_ctx* ctx) {
    VDNN_REQUIRE(ctx, "null context");
    ctx->pool.reset_peak();
    return VDNN_OK;
}

int vdnn_pool_set_cap(vdnn_ctx* ctx, size_t cap_bytes) {
    VDNN_REQUIRE(ctx, "null context");
    ctx->pool.set_cap(cap_bytes);
    return VDNN_OK;
}

int vdnn_pool_live_blocks(vdnn_ctx* ctx, size_t* count) {
    VDNN_REQUIRE(ctx && count, "null argument");
    *count = ctx->pool.live_blocks();
    return VDNN_OK;
}

/* ---- streams, events, copies ------------------------------------------------------------------ */
int vdnn_stream_synchronize(vdnn_ctx* ctx, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only) return VDNN_OK;
    VDNN_HIP(hipStreamSynchronize(stream_of(ctx, stream)));
    return VDNN_OK;
}

int vdnn_event_create(vdnn_ctx* ctx, vdnn_event_t* out, int with_timing) {
    VDNN_REQUIRE(ctx && out, "null argument");
    *out = nullptr;
    if (ctx->plan_only) return VDNN_OK;
    hipEvent_t ev;
    VDNN_HIP(hipEventCreateWithFlags(&ev, with_timing ? hipEventDefault : hipEventDisableTiming));
    *out = ev;
    return VDNN_OK;
}

int vdnn_event_destroy(vdnn_ctx* ctx, vdnn_event_t ev) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only || !ev) return VDNN_OK;
    VDNN_HIP(hipEventDestroy((hipEvent_t)ev));
    return VDNN_OK;
}

int vdnn_event_record(vdnn_ctx* ctx, vdnn_event_t ev, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only) return VDNN_OK;
    VDNN_REQUIRE(ev, "null event");
    VDNN_HIP(hipEventRecord((hipEvent_t)ev, stream_of(ctx, stream)));
    return VDNN_OK;
}

int vdnn_stream_wait_event(vdnn_ctx* ctx, vdnn_stream_t stream, vdnn_event_t ev) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only) return VDNN_OK;
    VDNN_REQUIRE(ev, "null event");
    VDNN_HIP(hipStreamWaitEvent(stream_of(ctx, stream), (hipEvent_t)ev, 0));
    return VDNN_OK;
}

int vdnn_event_synchronize(vdnn_ctx* ctx, vdnn_event_t ev) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only) return VDNN_OK;
    VDNN_REQUIRE(ev, "null event");
    VDNN_HIP(hipEventSynchronize((hipEvent_t)ev));
    return VDNN_OK;
}

int vdnn_event_elapsed_ms(vdnn_ctx* ctx, vdnn_event_t start, vdnn_event_t stop, float* ms) {
    VDNN_REQUIRE(ctx && ms, "null argument");
    *ms = 0.0f;
    if (ctx->plan_only) return VDNN_OK;
    VDNN_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return VDNN_OK;
}

int vdnn_host_alloc_pinned(vdnn_ctx* ctx, void** ptr, size_t bytes) {
    VDNN_REQUIRE(ctx && ptr, "null argument");
    *ptr = nullptr;
    if (ctx->plan_only) {
        // a distinct non-null token per request; never dereferenced
        static uintptr_t next = uintptr_t(1) << 45;
        *ptr = (void*)next;
        next += (bytes + 4095) / 4096 * 4096 + 4096;
        return VDNN_OK;
    }
    hipError_t e = hipHostMalloc(ptr, bytes, hipHostMallocDefault);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        set_error("hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
        *ptr = nullptr;
        return VDNN_OOM;
    }
    return VDNN_OK;
}

int vdnn_host_free_pinned(vdnn_ctx* ctx, void* ptr) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only || !ptr) return VDNN_OK;
    VDNN_HIP(hipHostFree(ptr));
    return VDNN_OK;
}

int vdnn_memcpy_d2h_async(vdnn_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only || bytes == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_host && src_dev, "null pointer");
    ProfScope prof(ctx, stream ? (hipStream_t)stream : ctx->d2h, "offload_d2h", 0.0, (double)bytes);
    VDNN_HIP(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, stream ? (hipStream_t)stream : ctx->d2h));
    return VDNN_OK;
}

int vdnn_memcpy_h2d_async(vdnn_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only || bytes == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_dev && src_host, "null pointer");
    ProfScope prof(ctx, stream ? (hipStream_t)stream : ctx->h2d, "prefetch_h2d", 0.0, (double)bytes);
    VDNN_HIP(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, stream ? (hipStream_t)stream : ctx->h2d));
    return VDNN_OK;
}

int vdnn_memcpy_d2h(vdnn_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only || bytes == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_host && src_dev, "null pointer");
    VDNN_HIP(hipDeviceSynchronize());
    VDNN_HIP(hipMemcpy(dst_host, src_dev, bytes, hipMemcpyDeviceToHost));
    return VDNN_OK;
}

int vdnn_memcpy_h2d(vdnn_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only || bytes == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_dev && src_host, "null pointer");
    VDNN_HIP(hipDeviceSynchronize());
    VDNN_HIP(hipMemcpy(dst_dev, src_host, bytes, hipMemcpyHostToDevice));
    VDNN_HIP(hipDeviceSynchronize());
    return VDNN_OK;
}

int vdnn_memcpy_d2d_async(vdnn_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only || bytes == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_dev && src_dev, "null pointer");
    VDNN_HIP(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, stream_of(ctx, stream)));
    return VDNN_OK;
}

int vdnn_profile_enable(vdnn_ctx* ctx, int on) {
    VDNN_REQUIRE(ctx, "null context");
    if (ctx->plan_only) return VDNN_OK;
    VDNN_HIP(hipDeviceSynchronize());
    for (auto& r : ctx->prof_records) { ctx->prof_free_events.push_back(r.start); ctx->prof_free_events.push_back(r.stop); }
    ctx->prof_records.clear();
    ctx->prof_untimed = 0;
    ctx->profiling = on != 0;
    // the events are made here, not in front of the first launches that need them
    while (ctx->profiling && ctx->prof_free_events.size() < 2 * kProfMaxRecords) {
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) { (void)hipGetLastError(); break; }
        ctx->prof_free_events.push_back(e);
    }
    return VDNN_OK;
}

int vdnn_profile_collect(vdnn_ctx* ctx, vdnn_profile_entry* out, int capacity, int* count) {
    VDNN_REQUIRE(ctx && count, "null argument");
    *count = 0;
    if (ctx->plan_only) return VDNN_OK;
    VDNN_HIP(hipDeviceSynchronize());
    std::vector<vdnn_profile_entry> agg;
    for (const auto& r : ctx->prof_records) {
        float ms = 0.0f;
        VDNN_HIP(hipEventElapsedTime(&ms, r.start, r.stop));
        size_t i = 0;
        for (; i < agg.size(); i++) if (strcmp(agg[i].name, r.name) == 0) break;
        if (i == agg.size()) {
            vdnn_profile_entry e;
            memset(&e, 0, sizeof(e));
            strncpy(e.name, r.name, sizeof(e.name) - 1);
            agg.push_back(e);
        }
        agg[i].launches += 1; agg[i].ms += ms; agg[i].flops += r.flops; agg[i].bytes += r.bytes;
    }
    if (ctx->prof_untimed) {
        vdnn_profile_entry e;
        memset(&e, 0, sizeof(e));
        strncpy(e.name, "untimed", sizeof(e.name) - 1);
        e.launches = ctx->prof_untimed;
        agg.push_back(e);
    }
    *count = (int)agg.size();
    for (int i = 0; i < (int)agg.size() && i < capacity; i++) if (out) out[i] = agg[i];
    return VDNN_OK;
}

int vdnn_profile_intervals(vdnn_ctx* ctx, vdnn_profile_interval* out, int capacity, int* count) {
    VDNN_REQUIRE(ctx && count, "null argument");
    *count = 0;
    if (ctx->plan_only || ctx->prof_records.empty()) return VDNN_OK;
    VDNN_HIP(hipDeviceSynchronize());
    // the earliest start is the origin: the first record made need not be the first to run (streams)
    std::vector<float> t0(ctx->prof_records.size()), t1(ctx->prof_records.size());
    const hipEvent_t origin = ctx->prof_records[0].start;
    float lowest = 0.0f;
    for (size_t i = 0; i < ctx->prof_records.size(); i++) {
        const auto& r = ctx->prof_records[i];
        VDNN_HIP(hipEventElapsedTime(&t0[i], origin, r.start));
        VDNN_HIP(hipEventElapsedTime(&t1[i], origin, r.stop));
        if (t0[i] < lowest) lowest = t0[i];
    }
    *count = (int)ctx->prof_records.size();
    for (int i = 0; i < *count && i < capacity && out; i++) {
        const auto& r = ctx->prof_records[i];
        memset(&out[i], 0, sizeof(out[i]));
        strncpy(out[i].name, r.name, sizeof(out[i].name) - 1);
        out[i].stream = r.stream == ctx->compute ? 0 : r.stream == ctx->d2h ? 1 : r.stream == ctx->h2d ? 2 : r.stream == ctx->pack ? 3 : 4;
        out[i].start_ms = (double)(t0[i] - lowest);
        out[i].stop_ms = (double)(t1[i] - lowest);
    }
    return VDNN_OK;
}

int vdnn_out_dim(int in, int pad, int window, int stride) {
    if (stride <= 0 || window <= 0) return 0;
    const int t = in + 2 * pad - window;
    if (t < 0) return 0;
    return t / stride + 1;
}

} // extern "C"
