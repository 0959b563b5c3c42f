/* C ABI of the MI355X (gfx950) device back end of the vDNN engine.
 *
 * This is the lower boundary of the training hot path: everything the reference obtains from
 * cuDNN, cuBLAS, cnmem and the CUDA runtime is reached through these entry points, and the C++
 * host classes (Layer, Network) call nothing else.  Plain pointers and sizes only.
 *
 * Conventions
 *   - every function returns an int status: VDNN_OK (0), VDNN_OOM (-1, the pool cannot serve a
 *     request; mirrors ASSERT_EQ's -1 in layer.h:110-128), or a value < -1 for a hard error;
 *     vdnn_last_error() holds a message for the last failure on the calling thread.
 *   - tensors are fp32, NCHW; filters KCRS; convolution is cross-correlation, dilation 1
 *     (vdnn.h:11-12, 19-20).
 *   - a stream argument of NULL means the context's compute stream.
 *   - kernels are asynchronous on their stream; nothing here synchronises unless it says so.
 *   - a context created with VDNN_CTX_PLAN_ONLY touches no device: the pool hands out addresses of
 *     a virtual range, copies and kernels return VDNN_OK without doing anything.  It exists so the
 *     allocation schedule of a policy can be replayed on a machine without a GPU; it computes
 *     nothing and is not a CPU implementation of the math.
 *   - not thread-safe: one host thread per context, like the reference.
 */
#ifndef VDNN_AMD_BACKEND_H_
#define VDNN_AMD_BACKEND_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VDNN_OK       0
#define VDNN_OOM     (-1)
#define VDNN_EINVAL  (-2)
#define VDNN_EDEVICE (-3)

#define VDNN_CTX_PLAN_ONLY 1

/* Element type of ACTIVATION tensors (layer inputs, outputs and their gradients: every `void*`
 * tensor argument of the kernel entry points below). The reference fixes float (vdnn.h:11-12);
 * bfloat16 storage halves the memory and the offload traffic. Filters, biases, their gradients and
 * loss values are always float (`float*` arguments), and all arithmetic is float with float
 * accumulation; a bfloat16 result is rounded once (to nearest, ties to even) when it is stored. */
#define VDNN_DTYPE_F32  0
#define VDNN_DTYPE_BF16 1

/* passes of a convolution, for vdnn_conv_workspace_bytes */
#define VDNN_PASS_FWD        0
#define VDNN_PASS_BWD_DATA   1
#define VDNN_PASS_BWD_FILTER 2

typedef struct vdnn_ctx vdnn_ctx;
typedef void* vdnn_stream_t; /* a hipStream_t */
typedef void* vdnn_event_t;  /* a hipEvent_t */

/* One layer's geometry: input n,c,h,w; filter k,r,s; padding and stride (the argument list of the
 * reference's Layer constructor, layer.h:133-154). */
typedef struct {
    int n, c, h, w;
    int k, r, s;
    int pad_h, pad_w, stride_h, stride_w;
} vdnn_shape_t;

/* ---- context --------------------------------------------------------------------------------- */
/* Replaces cudnnCreate/cublasCreate/cudaSetDevice (network.cu:16, 39-40; vdnn.cu:59). Creates the
 * compute stream and the two copy streams. */
int vdnn_ctx_create(vdnn_ctx** out, int device, int flags);
int vdnn_ctx_destroy(vdnn_ctx* ctx);
/* Element type of the activation tensors handed to later kernel calls on this context (default
 * VDNN_DTYPE_F32). No counterpart in the reference (CUDNN_DATA_FLOAT is fixed, vdnn.h:12).
 * With VDNN_DTYPE_BF16 the products of forward and backward data (convolution and FC) take the filter
 * rounded to bfloat16, nearest even, so that both factors are bfloat16 and the bfloat16 matrix cores can form
 * them exactly; accumulation, biases, parameter gradients and the parameters in memory stay float, and the
 * update acts on the float values. Backward filter multiplies two activation tensors and rounds nothing. */
int vdnn_ctx_set_activation_dtype(vdnn_ctx* ctx, int dtype);
int vdnn_ctx_activation_dtype(vdnn_ctx* ctx);
const char* vdnn_last_error(void);
/* cudaGetDeviceProperties(...).totalGlobalMem (network.cu:35-36, 48). */
int vdnn_device_mem_info(vdnn_ctx* ctx, size_t* free_bytes, size_t* total_bytes);
int vdnn_device_synchronize(vdnn_ctx* ctx);
/* Streams owned by the context: compute, device-to-host, host-to-device. The reference has
 * stream_compute and one stream_memory (network.cu:41-42); copies get one stream per direction. */
vdnn_stream_t vdnn_ctx_stream_compute(vdnn_ctx* ctx);
vdnn_stream_t vdnn_ctx_stream_d2h(vdnn_ctx* ctx);
vdnn_stream_t vdnn_ctx_stream_h2d(vdnn_ctx* ctx);
/* A fourth stream, for the kernels that pack offloaded tensors (vdnn_zvc_offload_staged_async): the next tensor
 * is packed while the copy engine still moves the one before on the device-to-host stream. */
vdnn_stream_t vdnn_ctx_stream_pack(vdnn_ctx* ctx);

/* ---- pooled device memory (replaces cnmem: network.cu:47-53, layer.cu:989-1011) --------------- */
/* cnmemInit: reserve `bytes` of device memory once; all later requests are carved from it. */
int vdnn_pool_init(vdnn_ctx* ctx, size_t bytes);
/* cnmemFinalize (network.cu:103). Releases the reservation and every block in it. */
int vdnn_pool_finalize(vdnn_ctx* ctx);
/* cnmemMalloc. VDNN_OOM when no free block fits or the cap would be exceeded. */
int vdnn_pool_malloc(vdnn_ctx* ctx, void** ptr, size_t bytes);
/* cnmemFree. */
int vdnn_pool_free(vdnn_ctx* ctx, void* ptr);
/* cnmemMemGetInfo (network.cu:1069, 1098, 1129, 1176): free and total bytes of the pool. */
int vdnn_pool_info(vdnn_ctx* ctx, size_t* free_bytes, size_t* total_bytes);
/* High-water marks since the last reset: bytes in use, and the highest end offset handed out. */
int vdnn_pool_peak(vdnn_ctx* ctx, size_t* peak_in_use, size_t* peak_extent);
int vdnn_pool_reset_peak(vdnn_ctx* ctx);
/* Artificial limit on bytes in use (0 = none); requests beyond it return VDNN_OOM. */
int vdnn_pool_set_cap(vdnn_ctx* ctx, size_t cap_bytes);
/* Number of live blocks (leak checks). */
int vdnn_pool_live_blocks(vdnn_ctx* ctx, size_t* count);

/* ---- streams, events, copies (replaces the CUDA runtime calls of layer.cu:969-987,
 *      network.cu:918-934, 1090-1091, 1168-1169) --------------------------------------------- */
int vdnn_stream_synchronize(vdnn_ctx* ctx, vdnn_stream_t stream);
int vdnn_event_create(vdnn_ctx* ctx, vdnn_event_t* out, int with_timing);
int vdnn_event_destroy(vdnn_ctx* ctx, vdnn_event_t ev);
int vdnn_event_record(vdnn_ctx* ctx, vdnn_event_t ev, vdnn_stream_t stream);
int vdnn_stream_wait_event(vdnn_ctx* ctx, vdnn_stream_t stream, vdnn_event_t ev);
int vdnn_event_synchronize(vdnn_ctx* ctx, vdnn_event_t ev);
int vdnn_event_elapsed_ms(vdnn_ctx* ctx, vdnn_event_t start, vdnn_event_t stop, float* ms);
/* cudaMallocHost / cudaFreeHost: pinned staging buffers for offloaded tensors. */
int vdnn_host_alloc_pinned(vdnn_ctx* ctx, void** ptr, size_t bytes);
int vdnn_host_free_pinned(vdnn_ctx* ctx, void* ptr);
/* cudaMemcpyAsync D2H (offloadSrcData, layer.cu:969-977) and H2D (prefetchPreviousSrcData,
 * layer.cu:979-987). */
int vdnn_memcpy_d2h_async(vdnn_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes, vdnn_stream_t stream);
int vdnn_memcpy_h2d_async(vdnn_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes, vdnn_stream_t stream);
/* The same two copies (layer.cu:969-987) with zero-value compression: the tensor of `count` elements
 * (elem_bytes 4: float, 2: bfloat16) crosses the link without the elements whose bits are all zero, and comes
 * back with every bit it had. The reference copies every tensor whole; a rectified tensor is about half zeros.
 * The host buffer must come from vdnn_host_alloc_pinned and hold vdnn_zvc_buffer_bytes(count, elem_bytes).
 * It receives a packed stream: a table of one 32-bit word per chunk of 4096 elements (padded to 16 bytes), the
 * offset of the chunk's record in units of 16 bytes; a record is a 512-byte map followed by the kept elements in
 * the order of the map's bits, zero filled to 16 bytes. With V = 16 / elem_bytes, bit l of the 64-bit word
 * b V + j of the map says whether element 64 V b + V l + j of the chunk is kept (a lane holds V consecutive
 * elements, 64 lanes a block of 64 V). Records lie without gaps in no particular order, so the stream is as long
 * as its content.
 *   vdnn_zvc_offload_async: a kernel on `stream` packs the tensor straight into the host buffer.
 *   vdnn_zvc_offload_staged_async: the kernel packs into `staging_dev` (device memory, 16-byte aligned,
 *     staging_bytes a multiple of 16) at HBM speed and the copy engine moves staging_bytes to the host buffer;
 *     what the stream has beyond staging_bytes the kernel stores into the host buffer itself, so any size is
 *     correct and the stream's length of the step before is the one to pass. total_host (pinned, may be NULL)
 *     receives the stream's length in bytes when the kernel is done. The kernel runs on pack_stream (NULL: the
 *     context's packing stream) behind what that stream holds, `packed` is recorded there when src_dev has been
 *     read, and the copy runs on copy_stream (NULL: the device-to-host stream) behind `packed`; with `packed`
 *     NULL everything runs on copy_stream. staging_dev must stay until the work on copy_stream is done.
 *     With keep_on_device the copy engine is not used: bytes [0, staging_bytes) of the stream stay in staging_dev
 *     (nothing crosses the link but what did not fit), for vdnn_zvc_prefetch_staged_async to read them there.
 *   vdnn_zvc_prefetch_async: a kernel on `stream` reads the host buffer and expands it into dst_dev.
 *   vdnn_zvc_prefetch_staged_async: the same, reading the stream's first staging_bytes from staging_dev (a block
 *     that vdnn_zvc_offload_staged_async was told to keep) and the rest from the host buffer. */
size_t vdnn_zvc_buffer_bytes(size_t count, int elem_bytes);
int vdnn_zvc_offload_async(vdnn_ctx* ctx, void* dst_host, const void* src_dev, size_t count, int elem_bytes, vdnn_stream_t stream);
int vdnn_zvc_offload_staged_async(vdnn_ctx* ctx, void* dst_host, void* staging_dev, size_t staging_bytes, const void* src_dev, size_t count,
                                  int elem_bytes, unsigned long long* total_host, vdnn_stream_t pack_stream, vdnn_stream_t copy_stream,
                                  vdnn_event_t packed, int keep_on_device);
int vdnn_zvc_prefetch_async(vdnn_ctx* ctx, void* dst_dev, const void* src_host, size_t count, int elem_bytes, vdnn_stream_t stream);
int vdnn_zvc_prefetch_staged_async(vdnn_ctx* ctx, void* dst_dev, const void* staging_dev, size_t staging_bytes, const void* src_host,
                                   size_t count, int elem_bytes, vdnn_stream_t stream);
/* Bytes of the tensors offloaded this way since the context was made, and bytes that crossed the link for
 * them (waits for the device). */
int vdnn_zvc_traffic(vdnn_ctx* ctx, unsigned long long* tensor_bytes, unsigned long long* link_bytes);
/* Blocking copies (cudaMemcpy: layer.cu:940-942, network.cu:827). */
int vdnn_memcpy_d2h(vdnn_ctx* ctx, void* dst_host, const void* src_dev, size_t bytes);
int vdnn_memcpy_h2d(vdnn_ctx* ctx, void* dst_dev, const void* src_host, size_t bytes);
int vdnn_memcpy_d2d_async(vdnn_ctx* ctx, void* dst_dev, const void* src_dev, size_t bytes, vdnn_stream_t stream);

/* ---- convolution (replaces cuDNN: layer.cu:539-665) ------------------------------------------ */
/* Output extent of a convolution or pooling window: (in + 2*pad - window)/stride + 1
 * (cudnnGetConvolution2dForwardOutputDim layer.cu:208-216, cudnnGetPooling2dForwardOutputDim
 * layer.cu:432-439). */
int vdnn_out_dim(int in, int pad, int window, int stride);
/* cudnnGetConvolution*WorkspaceSize (layer.cu:268-294). algo_mode is a vdnnAlgoMode_t value.
 * VDNN_MEMORY_OPT_ALGO always returns 0. VDNN_PERF_OPT_ALGO (the reference asks cuDNN for its fastest algorithm,
 * layer.cu:1013-1089), float activations: forward / backward data on the bfloat16 matrix cores (every float operand
 * as two bfloat16 parts, see vdnn_conv_perf_variant) take the filter bank split that way - the filter's bytes; under
 * the Winograd variant, forward / backward data of 3x3, stride 1, padding 1 layers with at least 128 reduced and more
 * than 64 produced channels take the transformed filter plus the transformed input and output of a chunk of samples
 * (up to 512 MiB), and so does backward filter where the default variant has no kernel; other layers take a
 * re-laid-out copy of the filter; backward filter otherwise takes room for the partial sums of its split reduction
 * where the context's staging area is too small. A pass handed less than this runs the memory-optimal kernels. The _dtype form takes the element type of the activations (VDNN_DTYPE_*); the plain
 * form assumes float. */
size_t vdnn_conv_workspace_bytes(const vdnn_shape_t* shape, int algo_mode, int pass);
size_t vdnn_conv_workspace_bytes_dtype(const vdnn_shape_t* shape, int algo_mode, int pass, int dtype);
/* Tuning (no counterpart in the reference): the bytes that the transformed input and output of one chunk of samples
 * may take in the Winograd variant's workspace; 0 restores the default (512 MiB). Returns the previous value. A
 * process-wide setting: it changes what vdnn_conv_workspace_bytes reports and how the passes split the batch, so set
 * it before networks are built, not between a query and the pass that uses its answer. Results do not depend on it
 * (samples are independent in forward and backward data). */
size_t vdnn_conv_winograd_chunk_bytes(size_t bytes);
/* Tuning (no counterpart in the reference; cuDNN's perf-optimal choice is made by cudnnGet*Algorithm, layer.cu:1012-1090):
 * which kernels VDNN_PERF_OPT_ALGO takes for layers with float activations where both apply. 0 (default): the
 * bfloat16 matrix cores with every float operand as two bfloat16 parts and three matrix instructions per product
 * (about 5e-6 of the largest output from the exact result; workspace = the filter's bytes) - forward and backward
 * data of stride-1 layers (forward: any stride) with at most 32 taps and reduced channels a multiple of 16, backward
 * filter of 3x3 / stride 1 / padding 1 layers with rows of whole groups of four pixels;
 * 1: Winograd F(4x4, 3x3) / F(3x3, 4x4) for wide 3x3 / stride 1 / padding 1 layers (about 2e-5; workspace of a third
 * to three quarters of a gigabyte), which also serves backward filter where variant 0 has no kernel. Returns
 * the previous value; other arguments only query. Process-wide, and it changes what vdnn_conv_workspace_bytes reports:
 * set it before networks are built. */
int vdnn_conv_perf_variant(int variant);
/* cudnnConvolutionForward + cudnnAddTensor (layer.cu:560-582): y = x (*) w + bias[k], the bias is
 * added once after the full reduction. bias may be NULL (no add). */
int vdnn_conv_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                  const void* x, const float* w, const float* bias, void* y,
                  void* workspace, size_t workspace_bytes);
/* cudnnAddTensor alone (layer.cu:576-582): y[n,k,:,:] += bias[k]. */
int vdnn_bias_add(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int k, int hw, const float* bias, void* y);
/* cudnnConvolutionBackwardData (layer.cu:616-625): dx = w^T (*) dy, alpha 1, beta 0. */
int vdnn_conv_bwd_data(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                       const void* dy, const float* w, void* dx,
                       void* workspace, size_t workspace_bytes);
/* cudnnConvolutionBackwardBias with alpha=-lr, beta=1 (layer.cu:631-637):
 * bias[k] += alpha * sum_{n,p,q} dy[n,k,p,q]. Fixed summation order. */
int vdnn_conv_bwd_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape,
                           const void* dy, float* bias, float alpha);
/* vdnn_conv_bwd_bias_sgd for callers that cannot allocate device memory. No counterpart in the reference. It is for
 * code under HIP graph capture, tight serving loops and harnesses that forbid hipMalloc: it takes no context (making
 * one reserves a pool and streams), and the partial sums of its two-stage reduction live in an array of
 * VDNN_NOALLOC_SCRATCH_BYTES that is part of the library's device image (every GPU the library runs on holds one
 * copy until the process ends) instead of a context's staging area. Same kernels, same split of the batch, same
 * bits as vdnn_conv_bwd_bias_sgd on the same device. `stream` is a hipStream_t of the current device (NULL: the
 * null stream); dtype is the element type of dy (VDNN_DTYPE_F32 / VDNN_DTYPE_BF16). A shape whose partial sums
 * (k x batch slices floats; 4 slices of the batch per compute unit divided by k, at least one) exceed the array is
 * rejected with VDNN_EINVAL. Calls no hipMalloc, hipFree or allocating library routine. All calls on one GPU
 * share that GPU's array: two calls that overlap there (different streams, different threads) race; calls on one
 * stream do not.
 * The first call on a device looks up that device's address of the array and its number of compute units (two
 * runtime queries, made once per device, thread-safe). Those queries must not run while a stream is being captured:
 * before capturing on a device, call vdnn_conv_bwd_bias_sgd_noalloc_prepare() with that device current (vdnn_ctx_create
 * on the device does the same). It allocates nothing either and may be called any number of times. */
#define VDNN_NOALLOC_SCRATCH_BYTES (256u << 10)
int vdnn_conv_bwd_bias_sgd_noalloc_prepare(void);
int vdnn_conv_bwd_bias_sgd_noalloc(vdnn_stream_t stream, const vdnn_shape_t* shape, int dtype,
                                   const void* dy, float* bias, float alpha);
/* cudnnConvolutionBackwardFilter with alpha=-lr, beta=1 (layer.cu:651-660):
 * w[k,c,r,s] += alpha * sum_{n,p,q} dy[n,k,p,q] * x[n,c,p*sh-ph+r,q*sw-pw+s]. Fixed summation
 * order (no floating-point atomics). */
int vdnn_conv_bwd_filter_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                             const void* x, const void* dy, float* w, float alpha,
                             void* workspace, size_t workspace_bytes);

/* cudnnConvolutionBackwardBias and cudnnConvolutionBackwardFilter (layer.cu:631-637, 651-660) in one call: both read
 * dy, and for most shapes the filter-gradient kernel adds up the bias gradient from the values it streams (the
 * filter-row kernels of 3x3 / stride 1 / padding 1 layers, the first-layer kernel, the Winograd variant; float
 * activations) instead of a second pass over dy. vdnn_conv_bwd_filter_sums_bias says whether a shape's kernel does;
 * where it does not, the call runs the kernels of vdnn_conv_bwd_bias[_sgd] behind the filter gradient on the same
 * stream (a caller that wants them side by side on another stream issues the two calls itself). The bias gradient's
 * sums take another order than vdnn_conv_bwd_bias_sgd's (same value to float rounding, fixed from run to run).
 *   _bias_sgd:       w += alpha dW,  bias += alpha db
 *   _bias:           dw = dW,        db = sum dy                 (optimizer step left out, see below)
 *   _then_bias_sgd:  dw = dW,        bias += alpha db            (for a caller that applies dW later) */
int vdnn_conv_bwd_filter_sums_bias(const vdnn_shape_t* shape, int algo_mode, int dtype);
int vdnn_conv_bwd_filter_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                                  const void* x, const void* dy, float* w, float* bias, float alpha,
                                  void* workspace, size_t workspace_bytes);
int vdnn_conv_bwd_filter_bias(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                              const void* x, const void* dy, float* dw, float* db, void* workspace, size_t workspace_bytes);
int vdnn_conv_bwd_filter_then_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                                       const void* x, const void* dy, float* dw, float* bias, float alpha,
                                       void* workspace, size_t workspace_bytes);

/* The same two reductions with the optimizer step left out: db[k] = sum dy, dw = sum dy*x (beta = 0).
 * The reference always fuses SGD into these calls (alpha=-lr, beta=1); a training loop that keeps
 * gradients (to average them over devices, or to apply another optimizer) needs them separately.
 * vdnn_sgd_apply then evaluates param += alpha * grad with the arithmetic of the fused calls, so
 * the two routes give the same bits. */
int vdnn_conv_bwd_bias(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* dy, float* db);
int vdnn_conv_bwd_filter(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                         const void* x, const void* dy, float* dw, void* workspace, size_t workspace_bytes);
int vdnn_sgd_apply(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, float alpha, const float* grad, float* param);

/* ---- layers fused with the rectifier next to them ------------------------------------------------
 * The reference runs every ReLU as a layer of its own (cudnnActivationForward / Backward, layer.cu:766-814),
 * which reads and writes the whole tensor once more. These entry points apply it where the tensor is
 * produced instead; each gives the bits of the two separate calls it stands for.
 *   vdnn_conv_fwd_relu / vdnn_fc_fwd_relu:  y = relu(layer(x))            = vdnn_conv_fwd, then vdnn_relu_fwd
 *   vdnn_conv_bwd_data_relu / vdnn_fc_bwd_data_relu / vdnn_maxpool_bwd_relu:
 *       dx = (x > 0) ? layer_backward(dy) : 0, where x is the layer's own input and the output of a ReLU
 *                                                                         = the layer's backward, then vdnn_relu_bwd */
int vdnn_conv_fwd_relu(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                       const void* x, const float* w, const float* bias, void* y,
                       void* workspace, size_t workspace_bytes);
int vdnn_conv_bwd_data_relu(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                            const void* dy, const float* w, const void* x, void* dx,
                            void* workspace, size_t workspace_bytes);
int vdnn_fc_fwd_relu(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                     const void* x, const float* w, const float* bias, void* y);
int vdnn_fc_bwd_data_relu(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                          const void* dy, const float* w, const void* x, void* dx);
int vdnn_maxpool_bwd_relu(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape,
                          const void* x, const void* y, const void* dy, void* dx);
/* Whether dx may be the very tensor x in vdnn_conv_bwd_data[_relu] / vdnn_maxpool_bwd[_relu] (no counterpart in the
 * reference, which allocates gradData beside srcData, layer.cu:599, 897): 1 for stride-1 convolutions with more than
 * four input channels that are not one dense product, and for 2x2 / stride 2 / unpadded pooling over planes of even
 * height and a width that is a multiple of four. There every lane reads the elements it overwrites before it does, and
 * nothing else reads x. (The filter gradient reads x: the caller computes it first.) Other shapes return an error
 * when handed dx == x as the gate. */
int vdnn_conv_bwd_data_in_place_ok(const vdnn_shape_t* shape);
int vdnn_maxpool_bwd_in_place_ok(const vdnn_shape_t* shape);

/* ---- fully connected (replaces cuBLAS: layer.cu:667-764) ------------------------------------- */
/* Sgemm(T,N) + rank-1 bias broadcast (layer.cu:677-706): y[n,o] = sum_i w[o,i] x[n,i] + bias[o].
 * w is [c_out][c_in] row-major. */
int vdnn_fc_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                const void* x, const float* w, const float* bias, void* y);
/* Sgemm(N,N) (layer.cu:725-733): dx[n,i] = sum_o w[o,i] dy[n,o]. */
int vdnn_fc_bwd_data(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                     const void* dy, const float* w, void* dx);
/* Sgemm(N,T) alpha=-lr beta=1 (layer.cu:736-744): w[o,i] += alpha * sum_n x[n,i] dy[n,o]. */
int vdnn_fc_bwd_weight_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                           const void* x, const void* dy, float* w, float alpha);
/* Sgemm with a ones vector, alpha=-lr beta=1 (layer.cu:747-761): bias[o] += alpha * sum_n dy[n,o]. */
int vdnn_fc_bwd_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_out,
                         const void* dy, float* bias, float alpha);
/* The two FC reductions without the optimizer step (see vdnn_conv_bwd_filter). */
int vdnn_fc_bwd_weight(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                       const void* x, const void* dy, float* dw);
int vdnn_fc_bwd_bias(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_out, const void* dy, float* db);

/* ---- bandwidth-bound layers (replaces cuDNN: layer.cu:766-915) -------------------------------- */
/* cudnnActivationForward, ReLU, NaN propagates (layer.cu:774-781, 380-385): y = x > 0 ? x : (x!=x ? x : 0). */
int vdnn_relu_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, void* y);
/* cudnnActivationBackward (layer.cu:802-811): dx = x > 0 ? dy : 0. x may be NULL, then the test is
 * y > 0, which selects the same elements. */
int vdnn_relu_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, const void* y,
                  const void* dy, void* dx);
/* cudnnActivationForward/Backward with CUDNN_ACTIVATION_TANH / CUDNN_ACTIVATION_SIGMOID (mode chosen from
 * the layer type at layer.cu:362-369; same call sites as ReLU, layer.cu:774-781, 802-811):
 * y = tanh(x), dx = dy (1 - y^2); y = 1 / (1 + exp(-x)), dx = dy y (1 - y). Backward reads y, not x. */
int vdnn_tanh_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, void* y);
int vdnn_tanh_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* y, const void* dy, void* dx);
int vdnn_sigmoid_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, void* y);
int vdnn_sigmoid_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* y, const void* dy, void* dx);
/* cudnnPoolingForward, max, NaN not propagated (layer.cu:875-882, 416-428). Window r x s. */
int vdnn_maxpool_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* x, void* y);
/* cudnnPoolingBackward (layer.cu:903-912): each window's dy goes to its first maximum in row-major
 * window order; overlapping windows accumulate in row-major order of the windows. */
int vdnn_maxpool_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape,
                     const void* x, const void* y, const void* dy, void* dx);
/* Cross-channel LRN, window 5, alpha 1e-4, beta 0.75, k 2 (no counterpart in the reference; the
 * AlexNet configuration names it): scale = k + alpha/5 * sum_{|c'-c|<=2} x_c'^2, y = x * scale^-beta. */
int vdnn_lrn_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c, int hw, const void* x, void* y);
int vdnn_lrn_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c, int hw,
                 const void* x, const void* y, const void* dy, void* dx);
/* cudnnSoftmaxForward ACCURATE / INSTANCE (layer.cu:824-832): per sample over `classes`. */
int vdnn_softmax_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* x, void* y);
/* cudnnSoftmaxBackward (layer.cu:853-862): dx_i = y_i * (dy_i - sum_j dy_j y_j). */
int vdnn_softmax_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes,
                     const void* y, const void* dy, void* dx);
/* calculateDiffTensor (network.cu:3-8): r = a - b. */
int vdnn_sub(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* a, const void* b, void* r);
/* fillVectorWithOnes generalised (layer.cu:33-38): p[i] = value. */
int vdnn_fill(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, float value, void* p);
/* Fused softmax + cross-entropy on integer labels (no counterpart in the reference, which never
 * forms a loss): prob = softmax(logits); loss[0] = -(1/n) sum_n log prob[n,label_n], summed in
 * sample order by one workgroup. loss may be NULL. */
int vdnn_softmax_ce_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* logits,
                        const int32_t* labels, void* prob, float* loss);
/* dlogits = (prob - onehot(label)) / n. */
int vdnn_softmax_ce_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* prob,
                        const int32_t* labels, void* dlogits);
/* Mean cross-entropy of a probability tensor against a dense target (one-hot or soft):
 * loss[0] = -(1/n) sum_n sum_c target[n,c] * log(max(prob[n,c], FLT_MIN)). Monitoring only. */
int vdnn_cross_entropy_dense(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes,
                             const void* prob, const void* target, float* loss);

/* ---- per-kernel timing (no counterpart in the reference, whose _PROFILE_* macros are unused:
 *      layer.h:34-38) ---------------------------------------------------------------------------
 * While enabled, every kernel launch of this library is bracketed by two events on its own stream - the
 * first 2048 launches after vdnn_profile_enable, that is; the ones after them run untimed (thousands of live
 * events slow every further one down; an entry named "untimed" counts them). vdnn_profile_collect synchronises
 * the device and returns one entry per kernel class: launches,
 * summed duration, and the algorithmic work of those launches (floating-point operations for the
 * MFMA kernels, bytes that must cross HBM for the bandwidth-bound ones). */
typedef struct {
    char   name[48];
    unsigned long long launches;
    double ms;
    double flops;
    double bytes;
} vdnn_profile_entry;
int vdnn_profile_enable(vdnn_ctx* ctx, int on);
int vdnn_profile_collect(vdnn_ctx* ctx, vdnn_profile_entry* out, int capacity, int* count);
/* The same launches one by one, in the order they were made: when each began and ended, in milliseconds since the
 * first of them began, and the stream it ran on (0 compute, 1 device-to-host, 2 host-to-device, 3 packing, 4 any
 * other). From these a caller works out how much of the copies' time ran beside kernels of the compute stream.
 * *count receives the number of timed launches, of which the first `capacity` are written. */
typedef struct {
    char   name[48];
    int    stream;
    double start_ms, stop_ms;
} vdnn_profile_interval;
int vdnn_profile_intervals(vdnn_ctx* ctx, vdnn_profile_interval* out, int capacity, int* count);

#ifdef __cplusplus
}
#endif
#endif
