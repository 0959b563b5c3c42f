// Internals shared by the device back end's translation units.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/vdnn_backend.h"
#include "pool.h"

struct vdnn_ctx {
    int device = 0;
    bool plan_only = false;
    hipStream_t compute = nullptr, d2h = nullptr, h2d = nullptr;
    vdnn::Pool pool;
    void* pool_base = nullptr;      // hipMalloc'd reservation (null in plan-only mode)
    // Staging for deterministic split reductions (filter gradients, bias gradients, FC split-K).
    // Taken from the pool at vdnn_pool_init so the usage meter sees it; bounded, shape-independent.
    float* reduce_scratch = nullptr;
    size_t reduce_scratch_bytes = 0;
    int num_cu = 256;
};

namespace vdnn {

static constexpr size_t kReduceScratchBytes = size_t(64) << 20;

void set_error(const char* fmt, ...);

inline hipStream_t stream_of(vdnn_ctx* ctx, vdnn_stream_t s) { return s ? (hipStream_t)s : ctx->compute; }

} // namespace vdnn

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
