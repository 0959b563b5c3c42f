// Internals shared by the device back end's translation units.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <vector>

#include "../../include/vdnn_backend.h"
#include "pool.h"

struct vdnn_ctx {
    int device = 0;
    bool plan_only = false;
    hipStream_t compute = nullptr, d2h = nullptr, h2d = nullptr, pack = nullptr;
    vdnn::Pool pool;
    void* pool_base = nullptr;      // hipMalloc'd reservation (null in plan-only mode)
    // Staging for deterministic split reductions (filter gradients, bias gradients, FC split-K).
    // Taken from the pool at vdnn_pool_init so the usage meter sees it; bounded, shape-independent.
    float* reduce_scratch = nullptr;
    size_t reduce_scratch_bytes = 0;
    // The last megabyte of the staging area belongs to the convolution bias gradient alone, so that it can run
    // on another stream beside the kernels that keep their partial sums in the rest.
    float* bias_scratch = nullptr;
    size_t bias_scratch_bytes = 0;
    int num_cu = 256;
    int act_dtype = VDNN_DTYPE_F32;   // element type of activation tensors handed to the kernels
    // per-kernel timing (vdnn_profile_*)
    // At most kProfMaxRecords launches are timed between vdnn_profile_enable and vdnn_profile_collect; the
    // launches after that run untimed. With more than about six thousand events alive, recording one became slow
    // enough to double a step's time.
    struct ProfRecord { const char* name; hipEvent_t start, stop; double flops, bytes; hipStream_t stream; };
    bool profiling = false;
    std::vector<ProfRecord> prof_records;
    std::vector<hipEvent_t> prof_free_events;
    unsigned long long prof_untimed = 0;   // launches since vdnn_profile_enable that ran beyond the limit
    // zero-value compression of offloaded tensors: device words (bytes sent over the link, then the stream
    // cursors of the offloads in flight) and bytes of the tensors that were packed
    unsigned long long* zvc_counters = nullptr;
    unsigned long long zvc_raw_bytes = 0;
    unsigned zvc_next_cursor = 0;
};

namespace vdnn {

static constexpr size_t kReduceScratchBytes = size_t(64) << 20;
static constexpr size_t kBiasScratchBytes = size_t(1) << 20;     // its last part: the convolution bias gradient's partial sums

void set_error(const char* fmt, ...);

inline hipStream_t stream_of(vdnn_ctx* ctx, vdnn_stream_t s) { return s ? (hipStream_t)s : ctx->compute; }

hipEvent_t prof_take_event(vdnn_ctx* ctx);
// looks up the current device's copy of the scratch array of vdnn_conv_bwd_bias_sgd_noalloc (eltwise.hip)
int noalloc_prepare_current_device();
static constexpr size_t kProfMaxRecords = 2048;

// Brackets the launches made during its lifetime with two timing events when profiling is on.
// `name` must be a string literal (it is kept by pointer).
struct ProfScope {
    vdnn_ctx* ctx; hipStream_t stream; size_t index; bool active;
    ProfScope(vdnn_ctx* c, hipStream_t s, const char* name, double flops, double bytes)
        : ctx(c), stream(s), index(0), active(c->profiling && c->prof_records.size() < kProfMaxRecords) {
        if (!active && c->profiling) c->prof_untimed++;
        if (!active) return;
        vdnn_ctx::ProfRecord r{name, prof_take_event(c), prof_take_event(c), flops, bytes, s};
        if (!r.start || !r.stop) { active = false; return; }
        (void)hipEventRecord(r.start, stream);
        index = c->prof_records.size();
        c->prof_records.push_back(r);
    }
    ~ProfScope() { if (active) (void)hipEventRecord(ctx->prof_records[index].stop, stream); }
};

} // namespace vdnn

// activation tensors are float or bfloat16, as the context says; filters, biases and their gradients are float
#define VDNN_BY_ACT(ctx, call_f32, call_bf16) ((ctx) && (ctx)->act_dtype == VDNN_DTYPE_BF16 ? (call_bf16) : (call_f32))

#define VDNN_HIP(call)                                                                        \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess) {                                                               \
            vdnn::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
            return VDNN_EDEVICE;                                                              \
        }                                                                                     \
    } while (0)

#define VDNN_REQUIRE(cond, msg)                                                               \
    do {                                                                                      \
        if (!(cond)) {                                                                        \
            vdnn::set_error("%s: %s (%s:%d)", __func__, msg, __FILE__, __LINE__);             \
            return VDNN_EINVAL;                                                               \
        }                                                                                     \
    } while (0)

// Every kernel entry point starts with this: plan-only contexts launch nothing.
#define VDNN_KERNEL_PROLOGUE(ctx)                                                             \
    do {                                                                                      \
        VDNN_REQUIRE((ctx) != nullptr, "null context");                                       \
        if ((ctx)->plan_only) return VDNN_OK;                                                 \
    } while (0)

#define VDNN_LAUNCH_CHECK()                                                                   \
    do {                                                                                      \
        hipError_t e_ = hipGetLastError();                                                    \
        if (e_ != hipSuccess) {                                                               \
            vdnn::set_error("kernel launch failed: %s (%s:%d)", hipGetErrorString(e_), __FILE__, __LINE__); \
            return VDNN_EDEVICE;                                                              \
        }                                                                                     \
    } while (0)
