// Bandwidth-bound layers: ReLU, max-pool, LRN, softmax, bias add / bias gradient, the first-diff
// subtraction, fills and the ordered reduction of split partial sums.
// Replaces cudnnActivation*/cudnnPooling*/cudnnSoftmax*/cudnnAddTensor/cudnnConvolutionBackwardBias
// (layer.cu:576-582, 631-637, 766-915) and the reference's two own kernels (layer.cu:33-38,
// network.cu:3-8). All reductions have a fixed order: results do not depend on timing.
#include "backend_internal.h"
#include "mfma_gemm.h"

#include <atomic>
#include <cfloat>
#include <mutex>

namespace vdnn {
int launch_bias_grad_final(vdnn_ctx* ctx, hipStream_t st, const float* partial, float* bias, int K, int splits, float alpha, int accumulate);

constexpr int EB = 256; // threads per workgroup

static inline unsigned grid_for(size_t items, int per_block, int max_blocks) {
    size_t b = (items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > (size_t)max_blocks) b = max_blocks;
    return (unsigned)b;
}

// ---- wavefront / workgroup reductions (fixed tree order) -----------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// every thread returns the workgroup-wide result; EB == 256 -> 4 wavefronts
__device__ __forceinline__ float block_sum(float v, float* sh) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    return (sh[0] + sh[1]) + (sh[2] + sh[3]);
}
__device__ __forceinline__ float block_max(float v, float* sh) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) sh[wave] = v;
    __syncthreads();
    return fmaxf(fmaxf(sh[0], sh[1]), fmaxf(sh[2], sh[3]));
}

// ---- four / two consecutive activation elements as floats ----------------------------------------------
// float: one 128-bit (64-bit) access; bfloat16: one 64-bit (32-bit) access. p must be aligned to the access.
__device__ __forceinline__ float4 ld4(const float* p) { return *(const float4*)p; }
__device__ __forceinline__ float4 ld4(const bf16_t* p) {
    const uint2 w = *(const uint2*)p;
    return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xFFFF0000u), __uint_as_float(w.y << 16), __uint_as_float(w.y & 0xFFFF0000u));
}
__device__ __forceinline__ void st4(float* p, float4 v) { *(float4*)p = v; }
__device__ __forceinline__ void st4(bf16_t* p, float4 v) {
    uint2 w;
    w.x = pack2_bf16(v.x, v.y);
    w.y = pack2_bf16(v.z, v.w);
    *(uint2*)p = w;
}
__device__ __forceinline__ float2 ld2(const float* p) { return *(const float2*)p; }
__device__ __forceinline__ float2 ld2(const bf16_t* p) {
    const unsigned w = *(const unsigned*)p;
    return make_float2(__uint_as_float(w << 16), __uint_as_float(w & 0xFFFF0000u));
}
__device__ __forceinline__ void st2(float* p, float2 v) { *(float2*)p = v; }
__device__ __forceinline__ void st2(bf16_t* p, float2 v) {
    *(unsigned*)p = pack2_bf16(v.x, v.y);
}

// ---- ReLU ---------------------------------------------------------------------------------------

template <class E>
__global__ void __launch_bounds__(EB) relu_fwd_kernel(const E* __restrict__ x, E* __restrict__ y, size_t n4, size_t n) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < n4; i += stride) {
        float4 v = ld4(x + 4 * i);
        v.x = relu_value(v.x); v.y = relu_value(v.y); v.z = relu_value(v.z); v.w = relu_value(v.w);
        st4(y + 4 * i, v);
    }
    for (size_t i = n4 * 4 + (size_t)blockIdx.x * EB + threadIdx.x; i < n; i += stride) store_elem(y + i, relu_value(load_elem(x + i)));
}

template <class E>
__global__ void __launch_bounds__(EB) relu_bwd_kernel(const E* __restrict__ t, const E* __restrict__ dy,
                                                      E* __restrict__ dx, size_t n4, size_t n) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < n4; i += stride) {
        const float4 a = ld4(t + 4 * i), d = ld4(dy + 4 * i);
        float4 o;
        o.x = a.x > 0.0f ? d.x : 0.0f; o.y = a.y > 0.0f ? d.y : 0.0f;
        o.z = a.z > 0.0f ? d.z : 0.0f; o.w = a.w > 0.0f ? d.w : 0.0f;
        st4(dx + 4 * i, o);
    }
    for (size_t i = n4 * 4 + (size_t)blockIdx.x * EB + threadIdx.x; i < n; i += stride)
        store_elem(dx + i, load_elem(t + i) > 0.0f ? load_elem(dy + i) : 0.0f);
}

// ---- tanh / sigmoid: the other two activation modes of the layer (four elements per thread) -----------
// backward needs the output only: tanh' = 1 - y^2, sigmoid' = y (1 - y)
template <int MODE> __device__ __forceinline__ float act1(float v) {
    return MODE == 0 ? tanhf(v) : 1.0f / (1.0f + expf(-v));
}
template <int MODE> __device__ __forceinline__ float dact1(float y, float d) {
    return MODE == 0 ? d * (1.0f - y * y) : d * (y * (1.0f - y));
}

template <int MODE, class E>
__global__ void __launch_bounds__(EB) act_fwd_kernel(const E* __restrict__ x, E* __restrict__ y, size_t n4, size_t n) {
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x;
    if (i < n4) {
        float4 v = ld4(x + 4 * i);
        v.x = act1<MODE>(v.x); v.y = act1<MODE>(v.y); v.z = act1<MODE>(v.z); v.w = act1<MODE>(v.w);
        st4(y + 4 * i, v);
    }
    const size_t t = n4 * 4 + i;
    if (t < n) store_elem(y + t, act1<MODE>(load_elem(x + t)));
}

template <int MODE, class E>
__global__ void __launch_bounds__(EB) act_bwd_kernel(const E* __restrict__ y, const E* __restrict__ dy, E* __restrict__ dx,
                                                     size_t n4, size_t n) {
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x;
    if (i < n4) {
        const float4 a = ld4(y + 4 * i), d = ld4(dy + 4 * i);
        float4 o;
        o.x = dact1<MODE>(a.x, d.x); o.y = dact1<MODE>(a.y, d.y); o.z = dact1<MODE>(a.z, d.z); o.w = dact1<MODE>(a.w, d.w);
        st4(dx + 4 * i, o);
    }
    const size_t t = n4 * 4 + i;
    if (t < n) store_elem(dx + t, dact1<MODE>(load_elem(y + t), load_elem(dy + t)));
}

// ---- elementwise helpers ------------------------------------------------------------------------
template <class E>
__global__ void __launch_bounds__(EB) sub_kernel(const E* __restrict__ a, const E* __restrict__ b, E* __restrict__ r, size_t n) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < n; i += stride) store_elem(r + i, load_elem(a + i) - load_elem(b + i));
}
template <class E>
__global__ void __launch_bounds__(EB) fill_kernel(E* __restrict__ p, float v, size_t n) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < n; i += stride) store_elem(p + i, v);
}
// y[n,k,:] += bias[k]; one workgroup row per (n,k) plane chunk
template <class E>
__global__ void __launch_bounds__(EB) bias_add_kernel(E* __restrict__ y, const float* __restrict__ bias, int K, int hw, size_t total) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < total; i += stride) {
        const int k = (int)((i / hw) % K);
        store_elem(y + i, load_elem(y + i) + bias[k]);
    }
}

// p[0] + p[stride] + p[2 stride] + ... (`splits` terms), added in that order. The adds wait for one another; the loads
// need not: eight splits are fetched at a time (a thread that fetches, adds, fetches pays a trip to memory per split).
__device__ __forceinline__ float ordered_sum(const float* __restrict__ p, size_t stride, int splits) {
    float s = p[0];
    int k = 1;
    for (; k + 8 <= splits; k += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = p[(size_t)(k + j) * stride];
#pragma unroll
        for (int j = 0; j < 8; j++) s += v[j];
    }
    if (k + 4 <= splits) {
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = p[(size_t)(k + j) * stride];
#pragma unroll
        for (int j = 0; j < 4; j++) s += v[j];
        k += 4;
    }
    for (; k < splits; k++) s += p[(size_t)k * stride];
    return s;
}

// out[i] = (accumulate ? out[i] : 0) + alpha * (p[0][i] + p[1][i] + ...) (+ bias[i % ncols]); split order fixed.
// out and gate may be one tensor (a gradient written over the input that gates it): an element is read before it is written.
template <class E>
__global__ void __launch_bounds__(EB) reduce_splits_kernel(E* out, const float* __restrict__ partial, size_t count,
                                                           int splits, float alpha, int accumulate, const float* __restrict__ bias_j, int ncols,
                                                           int relu, const E* gate) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < count; i += stride) {
        const float s = ordered_sum(partial + i, count, splits);
        float r = accumulate ? __fmaf_rn(alpha, s, load_elem(out + i)) : alpha * s; // one fused multiply-add on every route
        if (bias_j) r += bias_j[i % ncols];
        if (relu) r = relu_value(r);
        if (gate) r = load_elem(gate + i) > 0.0f ? r : 0.0f;
        store_elem(out + i, r);
    }
}

// The same sums when the splits are many (a reduction split over the whole chip for a small filter bank): a thread per
// output would walk hundreds of partial sums one after the other on a handful of workgroups. Here a workgroup owns 32
// outputs and eight groups of consecutive splits; a thread adds its group's splits in order, the eight group sums are
// added in group order through LDS. TAP: the partial sums are in tap-major column order (see reduce_splits_tap_kernel);
// the workgroup's 32 outputs are then 32 neighbours in that order (one 128-byte run per split), written to their places
// in the filter's order - the reads are `splits` times the writes.
template <bool TAP>
__global__ void __launch_bounds__(256) reduce_splits_wide_kernel(float* __restrict__ out, const float* __restrict__ partial, size_t count,
                                                                 int splits, float alpha, int accumulate, int C, int RS) {
    __shared__ float sums[8][33];
    const int o = threadIdx.x & 31, grp = threadIdx.x >> 5;
    const size_t i = (size_t)blockIdx.x * 32 + o;
    const int per = (splits + 7) / 8;
    const int k0 = grp * per, k1 = k0 + per < splits ? k0 + per : splits;
    float s = 0.0f;
    if (i < count && k0 < k1) s = ordered_sum(partial + (size_t)k0 * count + i, count, k1 - k0);
    sums[grp][o] = s;
    __syncthreads();
    if (grp == 0 && i < count) {
        float t = sums[0][o];
#pragma unroll
        for (int g = 1; g < 8; g++) t += (g * per < splits) ? sums[g][o] : 0.0f;
        size_t dst = i;
        if (TAP) {
            const int ncols = C * RS;
            const size_t m = i / ncols;
            const int rem = (int)(i - m * ncols);
            const int tap = rem / C, c = rem - tap * C;
            dst = m * ncols + (size_t)c * RS + tap;
        }
        out[dst] = accumulate ? __fmaf_rn(alpha, t, out[dst]) : alpha * t;
    }
}
constexpr int kWideReduceSplits = 32;        // from this many splits on,
constexpr size_t kWideReduceCount = 131072; // up to this many outputs (beyond, a thread per output fills the chip)

template <class E>
static int launch_reduce_splits_t(vdnn_ctx* ctx, hipStream_t stream, E* out, const float* partial, size_t count,
                                  int splits, float alpha, int accumulate, const float* bias_j, int ncols, int relu, const E* gate) {
    ProfScope prof(ctx, stream, "reduce_splits", 0.0, 4.0 * (double)count * (splits + 2));
    if constexpr (sizeof(E) == 4) {
        if (splits >= kWideReduceSplits && count <= kWideReduceCount && !bias_j && !relu && !gate) {
            hipLaunchKernelGGL(reduce_splits_wide_kernel<false>, dim3((unsigned)((count + 31) / 32)), dim3(256), 0, stream,
                               (float*)out, partial, count, splits, alpha, accumulate, 0, 0);
            VDNN_LAUNCH_CHECK();
            return VDNN_OK;
        }
    }
    hipLaunchKernelGGL(reduce_splits_kernel<E>, dim3(grid_for(count, EB, 0x7FFFFFFF)), dim3(EB), 0, stream,
                       out, partial, count, splits, alpha, accumulate, bias_j, ncols, relu, gate);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}
int launch_reduce_splits(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count,
                         int splits, float alpha, int accumulate, const float* bias_j, int ncols, int relu, const float* gate) {
    return launch_reduce_splits_t(ctx, stream, out, partial, count, splits, alpha, accumulate, bias_j, ncols, relu, gate);
}
int launch_reduce_splits(vdnn_ctx* ctx, hipStream_t stream, bf16_t* out, const float* partial, size_t count,
                         int splits, float alpha, int accumulate, const float* bias_j, int ncols, int relu, const bf16_t* gate) {
    return launch_reduce_splits_t(ctx, stream, out, partial, count, splits, alpha, accumulate, bias_j, ncols, relu, gate);
}

// tiles of a convolution result that were split (tail mode): out[n][m][pix] = sum over the tile's splits (+ bias[m]);
// partial[(t*splits + ks)*TM*TN + row*TN + col] for the t-th split tile, tiles numbered m-tile fastest
template <class E>
__global__ void __launch_bounds__(EB) reduce_tail_nchw_kernel(E* out, const float* __restrict__ partial, int splits, int TM, int TN,
                                                              int M, int N, int mtiles, int full_tiles, const float* __restrict__ bias, int opix, size_t total,
                                                              int relu, const E* gate) { // (out and gate may be one tensor)
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x;
    if (i >= total) return;
    const int per = TM * TN;
    const int t = (int)(i / per), local = (int)(i - (size_t)t * per);
    const int row = local / TN, col = local - row * TN;
    const int tile = full_tiles + t;
    const int m = (tile % mtiles) * TM + row, j = (tile / mtiles) * TN + col;
    if (m >= M || j >= N) return;
    float s = ordered_sum(partial + (size_t)t * splits * per + local, (size_t)per, splits);
    if (bias) s += bias[m];
    if (relu) s = relu_value(s);
    const int n = j / opix, pix = j - n * opix;
    const size_t o = ((size_t)n * M + m) * opix + pix;
    if (gate) s = load_elem(gate + o) > 0.0f ? s : 0.0f;
    store_elem(out + o, s);
}

template <class E>
static int launch_reduce_tail_nchw_t(vdnn_ctx* ctx, hipStream_t stream, E* out, const float* partial, int tail_tiles, int splits, int TM, int TN,
                                     int M, int N, int mtiles, int full_tiles, const float* bias, int opix, int relu, const E* gate) {
    const size_t total = (size_t)tail_tiles * TM * TN;
    ProfScope prof(ctx, stream, "reduce_splits", 0.0, 4.0 * (double)total * (splits + 1));
    hipLaunchKernelGGL(reduce_tail_nchw_kernel<E>, dim3(grid_for(total, EB, 0x7FFFFFFF)), dim3(EB), 0, stream,
                       out, partial, splits, TM, TN, M, N, mtiles, full_tiles, bias, opix, total, relu, gate);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}
int launch_reduce_tail_nchw(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, int tail_tiles, int splits, int TM, int TN,
                            int M, int N, int mtiles, int full_tiles, const float* bias, int opix, int relu, const float* gate) {
    return launch_reduce_tail_nchw_t(ctx, stream, out, partial, tail_tiles, splits, TM, TN, M, N, mtiles, full_tiles, bias, opix, relu, gate);
}
int launch_reduce_tail_nchw(vdnn_ctx* ctx, hipStream_t stream, bf16_t* out, const float* partial, int tail_tiles, int splits, int TM, int TN,
                            int M, int N, int mtiles, int full_tiles, const float* bias, int opix, int relu, const bf16_t* gate) {
    return launch_reduce_tail_nchw_t(ctx, stream, out, partial, tail_tiles, splits, TM, TN, M, N, mtiles, full_tiles, bias, opix, relu, gate);
}

// filter gradient whose partial sums are in tap-major column order: out[m][c][tap] gets partial[.][m][tap*C + c]
__global__ void __launch_bounds__(EB) reduce_splits_tap_kernel(float* __restrict__ out, const float* __restrict__ partial, size_t count,
                                                               int splits, float alpha, int accumulate, int C, int RS) {
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x;
    if (i >= count) return;
    const int ncols = C * RS;
    const size_t m = i / ncols;
    const int rem = (int)(i - m * ncols);
    const int c = rem / RS, tap = rem - c * RS;
    const size_t src = m * ncols + (size_t)tap * C + c;
    const float s = ordered_sum(partial + src, count, splits);
    out[i] = accumulate ? __fmaf_rn(alpha, s, out[i]) : alpha * s;
}

// The same for filters of up to 16 taps, a workgroup per output channel and 64 input channels: the partial sums are read
// in their own order (for a tap, 64 consecutive channels: whole lines), the sums pass through LDS and leave in the
// filter's order (64 channels x taps: one run). A thread per output reads its partial sums C elements apart from its
// neighbour's of the next tap - a line fetched for 28 bytes of it. Same sums in the same order: the same bits.
constexpr int kTapTileC = 64, kTapTileMaxRS = 16;
__global__ void __launch_bounds__(256) reduce_splits_tap_tile_kernel(float* __restrict__ out, const float* __restrict__ partial, size_t count,
                                                                     int splits, float alpha, int accumulate, int C, int RS, int cblocks) {
    __shared__ float tile[kTapTileMaxRS][kTapTileC + 1];
    const int m = blockIdx.x / cblocks, c0 = (blockIdx.x - m * cblocks) * kTapTileC;
    const size_t row = (size_t)m * C * RS;
    for (int idx = threadIdx.x; idx < RS * kTapTileC; idx += 256) {
        const int tap = idx / kTapTileC, cc = idx - tap * kTapTileC;
        if (c0 + cc < C) {
            const size_t src = row + (size_t)tap * C + c0 + cc;
            tile[tap][cc] = ordered_sum(partial + src, count, splits);
        }
    }
    __syncthreads();
    const int here = C - c0 < kTapTileC ? C - c0 : kTapTileC;
    float* o = out + row + (size_t)c0 * RS;
    for (int idx = threadIdx.x; idx < here * RS; idx += 256) {
        const int cc = idx / RS, tap = idx - cc * RS;
        const float s = tile[tap][cc];
        o[idx] = accumulate ? __fmaf_rn(alpha, s, o[idx]) : alpha * s;
    }
}

int launch_reduce_splits_tap(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count, int splits,
                             float alpha, int accumulate, int C, int RS) {
    ProfScope prof(ctx, stream, "reduce_splits", 0.0, 4.0 * (double)count * (splits + 2));
    const size_t rows = count / ((size_t)C * RS);
    const int cblocks = (C + kTapTileC - 1) / kTapTileC;
    if (splits >= kWideReduceSplits && count <= kWideReduceCount)
        hipLaunchKernelGGL(reduce_splits_wide_kernel<true>, dim3((unsigned)((count + 31) / 32)), dim3(256), 0, stream,
                           out, partial, count, splits, alpha, accumulate, C, RS);
    else if (RS <= kTapTileMaxRS && rows * (size_t)C * RS == count && rows * cblocks < (1ul << 31))
        hipLaunchKernelGGL(reduce_splits_tap_tile_kernel, dim3((unsigned)(rows * cblocks)), dim3(256), 0, stream,
                           out, partial, count, splits, alpha, accumulate, C, RS, cblocks);
    else
    hipLaunchKernelGGL(reduce_splits_tap_kernel, dim3(grid_for(count, EB, 0x7FFFFFFF)), dim3(EB), 0, stream,
                       out, partial, count, splits, alpha, accumulate, C, RS);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

// NCHW result of a split convolution: out[i] = p[0][i] + p[1][i] + ... (+ bias[channel of i]); split order fixed
template <class E>
__global__ void __launch_bounds__(EB) reduce_splits_nchw_kernel(E* out, const float* __restrict__ partial, size_t count,
                                                                int splits, const float* __restrict__ bias, int opix, int channels,
                                                                int relu, const E* gate) { // (out and gate may be one tensor)
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x;
    if (i >= count) return;
    float s = partial[i];
    for (int k = 1; k < splits; k++) s += partial[(size_t)k * count + i];
    if (bias) s += bias[(i / opix) % channels];
    if (relu) s = relu_value(s);
    if (gate) s = load_elem(gate + i) > 0.0f ? s : 0.0f;
    store_elem(out + i, s);
}

template <class E>
static int launch_reduce_splits_nchw_t(vdnn_ctx* ctx, hipStream_t stream, E* out, const float* partial, size_t count, int splits,
                                       const float* bias, int opix, int channels, int relu, const E* gate) {
    ProfScope prof(ctx, stream, "reduce_splits", 0.0, 4.0 * (double)count * (splits + 1));
    hipLaunchKernelGGL(reduce_splits_nchw_kernel<E>, dim3(grid_for(count, EB, 0x7FFFFFFF)), dim3(EB), 0, stream,
                       out, partial, count, splits, bias, opix, channels, relu, gate);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}
int launch_reduce_splits_nchw(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count, int splits,
                              const float* bias, int opix, int channels, int relu, const float* gate) {
    return launch_reduce_splits_nchw_t(ctx, stream, out, partial, count, splits, bias, opix, channels, relu, gate);
}
int launch_reduce_splits_nchw(vdnn_ctx* ctx, hipStream_t stream, bf16_t* out, const float* partial, size_t count, int splits,
                              const float* bias, int opix, int channels, int relu, const bf16_t* gate) {
    return launch_reduce_splits_nchw_t(ctx, stream, out, partial, count, splits, bias, opix, channels, relu, gate);
}

// param[i] = fma(alpha, grad[i], param[i]), the expression the fused updates evaluate
__global__ void __launch_bounds__(EB) sgd_apply_kernel(const float* __restrict__ grad, float* __restrict__ param, float alpha, size_t count) {
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x;
    if (i < count) {
        param[i] = __fmaf_rn(alpha, grad[i], param[i]);
    }
}

// ---- bias gradient of a convolution: bias[k] += alpha * sum_{n,pq} dy[n,k,pq] -------------------
// Sum of V consecutive elements (one access), in a fixed order.
template <int V, class E> __device__ __forceinline__ float sum_of_run(const E* p);
template <> __device__ __forceinline__ float sum_of_run<1, float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float sum_of_run<1, bf16_t>(const bf16_t* p) { return load_elem(p); }
template <> __device__ __forceinline__ float sum_of_run<4, float>(const float* p) { const float4 v = ld4(p); return (v.x + v.y) + (v.z + v.w); }
template <> __device__ __forceinline__ float sum_of_run<4, bf16_t>(const bf16_t* p) { const float4 v = ld4(p); return (v.x + v.y) + (v.z + v.w); }
template <> __device__ __forceinline__ float sum_of_run<8, bf16_t>(const bf16_t* p) {
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = *(const u32x4*)p;
    return ((__builtin_bit_cast(float, v.x << 16) + __builtin_bit_cast(float, v.x & 0xFFFF0000u)) +
            (__builtin_bit_cast(float, v.y << 16) + __builtin_bit_cast(float, v.y & 0xFFFF0000u))) +
           ((__builtin_bit_cast(float, v.z << 16) + __builtin_bit_cast(float, v.z & 0xFFFF0000u)) +
            (__builtin_bit_cast(float, v.w << 16) + __builtin_bit_cast(float, v.w & 0xFFFF0000u)));
}
// Planes with fewer accesses than the workgroup has threads (13 x 13, 14 x 14 ...): walking them sample by sample
// leaves most threads idle and a thread's loads one behind the other (83 GB/s on AlexNet's layers). Here the
// workgroup's samples are one index space (sample, access), a thread takes every EB-th of it, four in flight.
template <int V, class E>
__device__ __forceinline__ float bias_grad_small_planes(const E* __restrict__ dy, int n0, int n1, int K, int k, int PQ) {
    const int pqv = PQ / V, total = (n1 - n0) * pqv;
    float s[4] = {0.f, 0.f, 0.f, 0.f};
    for (int j = threadIdx.x; j < total; j += 4 * EB) {
        float t[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int jj = j + u * EB;
            const int n = jj / pqv, i = jj - n * pqv;
            t[u] = jj < total ? sum_of_run<V>(dy + ((size_t)(n0 + n) * K + k) * PQ + (size_t)i * V) : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 4; u++) s[u] += t[u];
    }
    return (s[0] + s[1]) + (s[2] + s[3]);
}

// stage 1: workgroup (k, split) sums samples [n0, n1) of channel k into partial[k*splits + split]
template <class E>
__global__ void __launch_bounds__(EB) bias_grad_partial_kernel(const E* __restrict__ dy, float* __restrict__ partial,
                                                               int N, int K, int PQ, int splits, int n_per_split) {
    __shared__ float sh[4];
    const int k = blockIdx.x / splits, sp = blockIdx.x % splits;
    const int n0 = sp * n_per_split, n1 = min(N, n0 + n_per_split);
    float acc = 0.0f;
    const bool aligned = (((uintptr_t)dy & 15) == 0);
    if (sizeof(E) == 2 && (PQ & 7) == 0 && aligned && (PQ >> 3) < EB) {
        if constexpr (sizeof(E) == 2) acc = bias_grad_small_planes<8>(dy, n0, n1, K, k, PQ);
    } else if ((PQ & 3) == 0 && aligned && (PQ >> 2) < EB && !(sizeof(E) == 2 && (PQ & 7) == 0)) {
        acc = bias_grad_small_planes<4>(dy, n0, n1, K, k, PQ);
    } else if (!((PQ & 3) == 0 && aligned) && PQ < EB) {
        acc = bias_grad_small_planes<1>(dy, n0, n1, K, k, PQ);
    } else if (sizeof(E) == 2 && (PQ & 7) == 0 && (((uintptr_t)dy & 15) == 0)) {
        // bfloat16: eight elements (16 bytes) per access, eight independent partial sums per thread
        typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
        float s[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const int pq8 = PQ >> 3;
        for (int n = n0; n < n1; n++) {
            const u32x4* p = (const u32x4*)(dy + ((size_t)n * K + k) * PQ);
            for (int i = threadIdx.x; i < pq8; i += EB) {
                const u32x4 v = p[i];
                s[0] += __builtin_bit_cast(float, v.x << 16); s[1] += __builtin_bit_cast(float, v.x & 0xFFFF0000u);
                s[2] += __builtin_bit_cast(float, v.y << 16); s[3] += __builtin_bit_cast(float, v.y & 0xFFFF0000u);
                s[4] += __builtin_bit_cast(float, v.z << 16); s[5] += __builtin_bit_cast(float, v.z & 0xFFFF0000u);
                s[6] += __builtin_bit_cast(float, v.w << 16); s[7] += __builtin_bit_cast(float, v.w & 0xFFFF0000u);
            }
        }
        acc = ((s[0] + s[1]) + (s[2] + s[3])) + ((s[4] + s[5]) + (s[6] + s[7]));
    } else if ((PQ & 3) == 0 && (((uintptr_t)dy & 15) == 0)) {
        // four elements per access, four independent partial sums per thread (a fixed order, combined below)
        float4 a4 = make_float4(0.f, 0.f, 0.f, 0.f);
        const int pq4 = PQ >> 2;
        for (int n = n0; n < n1; n++) {
            const E* p = dy + ((size_t)n * K + k) * PQ;
            for (int i = threadIdx.x; i < pq4; i += EB) {
                const float4 v = ld4(p + 4 * i);
                a4.x += v.x; a4.y += v.y; a4.z += v.z; a4.w += v.w;
            }
        }
        acc = (a4.x + a4.y) + (a4.z + a4.w);
    } else {
        for (int n = n0; n < n1; n++) {
            const E* p = dy + ((size_t)n * K + k) * PQ;
            for (int i = threadIdx.x; i < PQ; i += EB) acc += load_elem(p + i);
        }
    }
    acc = block_sum(acc, sh);
    if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}
// stage 2: one wavefront per channel; lane l adds partials l, l + 64, ... in that order, the 64 lane sums are added by
// halving (a fixed order: the same bits every time). A channel's partials can be a few hundred (one per reduction split
// of the filter-gradient kernel that left them): one thread walking them took longer than the kernel before it.
__global__ void __launch_bounds__(EB) bias_grad_final_kernel(const float* __restrict__ partial, float* __restrict__ bias, int K, int splits, float alpha, int accumulate) {
    const int k = blockIdx.x * (EB / 64) + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (k >= K) return;
    float s = 0.0f;
    for (int i = lane; i < splits; i += 64) s += partial[(size_t)k * splits + i];
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off);
    if (lane == 0) bias[k] = accumulate ? __fmaf_rn(alpha, s, bias[k]) : alpha * s;
}

// bias[o] += alpha * sum_n dy[n,o]
template <class E>
__global__ void __launch_bounds__(EB) fc_bias_grad_kernel(const E* __restrict__ dy, float* __restrict__ bias, int N, int Cout, float alpha, int accumulate) {
    const int o = blockIdx.x * EB + threadIdx.x;
    if (o >= Cout) return;
    float s = 0.0f;
    for (int n = 0; n < N; n++) s += load_elem(dy + (size_t)n * Cout + o);
    bias[o] = accumulate ? __fmaf_rn(alpha, s, bias[o]) : alpha * s;
}

// ---- max pooling --------------------------------------------------------------------------------
struct PoolGeo { int N, C, H, W, R, S, P, Q, ph, pw, sh, sw; };

template <class E>
__global__ void __launch_bounds__(EB) maxpool_fwd_kernel(const E* __restrict__ x, E* __restrict__ y, PoolGeo g, size_t total) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < total; i += stride) {
        const int q = (int)(i % g.Q);
        const size_t t = i / g.Q;
        const int p = (int)(t % g.P);
        const size_t nc = t / g.P;
        const E* xp = x + nc * g.H * g.W;
        float m = -FLT_MAX;
        for (int r = 0; r < g.R; r++) {
            const int ih = p * g.sh - g.ph + r;
            if (ih < 0 || ih >= g.H) continue;
            for (int s = 0; s < g.S; s++) {
                const int iw = q * g.sw - g.pw + s;
                if (iw < 0 || iw >= g.W) continue;
                const float v = load_elem(xp + (size_t)ih * g.W + iw);
                if (v > m) m = v;
            }
        }
        store_elem(y + i, m);
    }
}

// 2x2 stride 2, no padding, even extents, W % 4 == 0: one thread makes two outputs from two four-element rows
template <class E>
__global__ void __launch_bounds__(EB) maxpool2x2_fwd_kernel(const E* __restrict__ x, E* __restrict__ y, int H, int W, size_t total_pairs) {
    const int Q2 = W / 4, P = H / 2;
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < total_pairs; i += stride) {
        const int q2 = (int)(i % Q2);
        const size_t t = i / Q2;
        const int p = (int)(t % P);
        const size_t nc = t / P;
        const E* r0 = x + (nc * H + 2 * (size_t)p) * W + 4 * (size_t)q2;
        const float4 a = ld4(r0), b = ld4(r0 + W);
        float m0 = -FLT_MAX, m1 = -FLT_MAX;
        if (a.x > m0) m0 = a.x; if (a.y > m0) m0 = a.y; if (b.x > m0) m0 = b.x; if (b.y > m0) m0 = b.y;
        if (a.z > m1) m1 = a.z; if (a.w > m1) m1 = a.w; if (b.z > m1) m1 = b.z; if (b.w > m1) m1 = b.w;
        float2 o; o.x = m0; o.y = m1;
        st2(y + (nc * P + p) * (size_t)(W / 2) + 2 * (size_t)q2, o);
    }
}

// argmax of window (p,q) with the forward's comparison: first strict maximum in row-major order;
// the first valid position if nothing exceeds -FLT_MAX
template <class E>
__device__ __forceinline__ int window_argmax(const E* __restrict__ xp, const PoolGeo& g, int p, int q) {
    float m = -FLT_MAX;
    int arg = -1;
    for (int r = 0; r < g.R; r++) {
        const int ih = p * g.sh - g.ph + r;
        if (ih < 0 || ih >= g.H) continue;
        for (int s = 0; s < g.S; s++) {
            const int iw = q * g.sw - g.pw + s;
            if (iw < 0 || iw >= g.W) continue;
            const float v = load_elem(xp + (size_t)ih * g.W + iw);
            if (arg < 0) arg = ih * g.W + iw;
            if (v > m) { m = v; arg = ih * g.W + iw; }
        }
    }
    return arg;
}

// gather form: one thread per input element, windows visited in row-major order
template <class E>
__global__ void __launch_bounds__(EB) maxpool_bwd_kernel(const E* __restrict__ x, const E* __restrict__ dy, E* __restrict__ dx,
                                                         PoolGeo g, size_t total, int gate) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < total; i += stride) {
        const int w = (int)(i % g.W);
        const size_t t = i / g.W;
        const int h = (int)(t % g.H);
        const size_t nc = t / g.H;
        const E* xp = x + nc * g.H * g.W;
        const E* dyp = dy + nc * g.P * g.Q;
        // windows containing (h,w): p*sh - ph <= h <= p*sh - ph + R - 1
        int p_lo = h + g.ph - g.R + 1; p_lo = p_lo <= 0 ? 0 : (p_lo + g.sh - 1) / g.sh;
        int p_hi = (h + g.ph) / g.sh; if (p_hi > g.P - 1) p_hi = g.P - 1;
        int q_lo = w + g.pw - g.S + 1; q_lo = q_lo <= 0 ? 0 : (q_lo + g.sw - 1) / g.sw;
        int q_hi = (w + g.pw) / g.sw; if (q_hi > g.Q - 1) q_hi = g.Q - 1;
        const int self = h * g.W + w;
        float acc = 0.0f;
        for (int p = p_lo; p <= p_hi; p++)
            for (int q = q_lo; q <= q_hi; q++)
                if (window_argmax(xp, g, p, q) == self) acc += load_elem(dyp + (size_t)p * g.Q + q);
        if (gate && !(load_elem(x + i) > 0.0f)) acc = 0.0f; // x is a rectifier's output: its gradient passes only where x > 0
        store_elem(dx + i, acc);
    }
}

// Unpadded pooling with a compile-time window and stride (AlexNet's 3x3 / stride 2) on planes that fit LDS: a
// workgroup stages `group` consecutive (n,c) planes - one contiguous run of memory - and writes their outputs, another
// contiguous run. The general kernels address every element with 64-bit divisions by run-time extents and run-time
// loop bounds, which cost more than the memory accesses; here every division is by a constant or a 32-bit multiply-high.
// Same comparison, same order: the same bits.
template <class E, int R, int S, int SH, int SW>
__global__ void __launch_bounds__(EB) maxpool_fwd_planes_kernel(const E* __restrict__ x, E* __restrict__ y, int H, int W, int P, int Q,
                                                                long planes, int group, FastDiv dPQ, FastDiv dQ) {
    extern __shared__ float pool_lds[];
    const int HW = H * W, PQ = P * Q;
    const long plane0 = (long)blockIdx.x * group;
    const int here = (int)(planes - plane0 < group ? planes - plane0 : group);
    const E* xp = x + plane0 * HW;
    for (int i = threadIdx.x; i < here * HW; i += EB) pool_lds[i] = load_elem(xp + i);
    __syncthreads();
    E* yp = y + plane0 * PQ;
    for (int o = threadIdx.x; o < here * PQ; o += EB) {
        const int pl = dPQ.div(o), pq = o - pl * PQ;
        const int p = dQ.div(pq), q = pq - p * Q;
        const float* b = pool_lds + pl * HW + p * SH * W + q * SW;
        float m = -FLT_MAX;
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int s_ = 0; s_ < S; s_++) {
                const float v = b[r * W + s_];
                if (v > m) m = v;
            }
        store_elem(yp + o, m);
    }
}

// The backward counterpart: x and dy of `group` planes in LDS, every window's winner found once (first strict maximum
// in row-major order, the window's first element if nothing exceeds -FLT_MAX), then every input element adds up the dy
// of the windows that contain it and chose it, windows in row-major order - the general kernels' rule and order.
template <class E, int R, int S, int SH, int SW>
__global__ void __launch_bounds__(EB) maxpool_bwd_planes_fixed_kernel(const E* __restrict__ x, const E* __restrict__ dy, E* __restrict__ dx,
                                                                      int H, int W, int P, int Q, long planes, int group, int gate,
                                                                      FastDiv dPQ, FastDiv dQ, FastDiv dHW, FastDiv dW) {
    extern __shared__ float pool_lds[];
    const int HW = H * W, PQ = P * Q;
    float* xs = pool_lds;                      // [group][HW]
    float* dys = xs + group * HW;              // [group][PQ]
    int* arg = (int*)(dys + group * PQ);       // [group][PQ] winner's index in its plane
    const long plane0 = (long)blockIdx.x * group;
    const int here = (int)(planes - plane0 < group ? planes - plane0 : group);
    const E* xp = x + plane0 * HW;
    const E* dyp = dy + plane0 * PQ;
    for (int i = threadIdx.x; i < here * HW; i += EB) xs[i] = load_elem(xp + i);
    for (int i = threadIdx.x; i < here * PQ; i += EB) dys[i] = load_elem(dyp + i);
    __syncthreads();
    for (int o = threadIdx.x; o < here * PQ; o += EB) {
        const int pl = dPQ.div(o), pq = o - pl * PQ;
        const int p = dQ.div(pq), q = pq - p * Q;
        const int first = p * SH * W + q * SW;
        const float* b = xs + pl * HW + first;
        float m = -FLT_MAX;
        int a = first;
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
            for (int s_ = 0; s_ < S; s_++) {
                const float v = b[r * W + s_];
                if (v > m) { m = v; a = first + r * W + s_; }
            }
        arg[o] = a;
    }
    __syncthreads();
    E* dxp = dx + plane0 * HW;
    for (int i = threadIdx.x; i < here * HW; i += EB) {
        const int pl = dHW.div(i), self = i - pl * HW;
        const int h = dW.div(self), w = self - h * W;
        // windows containing (h, w): p * SH <= h <= p * SH + R - 1
        int p_lo = h - R + 1; p_lo = p_lo <= 0 ? 0 : (p_lo + SH - 1) / SH;
        int p_hi = h / SH; if (p_hi > P - 1) p_hi = P - 1;
        int q_lo = w - S + 1; q_lo = q_lo <= 0 ? 0 : (q_lo + SW - 1) / SW;
        int q_hi = w / SW; if (q_hi > Q - 1) q_hi = Q - 1;
        const int* ap = arg + pl * PQ;
        const float* dp = dys + pl * PQ;
        float acc = 0.0f;
        for (int p = p_lo; p <= p_hi; p++)
            for (int q = q_lo; q <= q_hi; q++)
                if (ap[p * Q + q] == self) acc += dp[p * Q + q];
        if (gate && !(xs[i] > 0.0f)) acc = 0.0f;
        store_elem(dxp + i, acc);
    }
}

// Overlapping windows on planes that fit LDS (AlexNet's 3x3 stride 2): a workgroup stages `group` whole
// (n,c) planes and their dy, finds every window's winner once, and each input element then asks the few
// windows that contain it. Same winner rule and the same summation order as the gather kernel above, so the
// same bits; x, dy and dx cross HBM once.
template <class E>
__global__ void __launch_bounds__(EB) maxpool_bwd_planes_kernel(const E* __restrict__ x, const E* __restrict__ dy, E* __restrict__ dx,
                                                                PoolGeo g, long planes, int group, int gate) {
    extern __shared__ float pool_lds[];
    const int HW = g.H * g.W, PQ = g.P * g.Q;
    float* xs = pool_lds;                      // [group][HW]
    float* dys = xs + group * HW;              // [group][PQ]
    int* arg = (int*)(dys + group * PQ);       // [group][PQ] winner's index in its plane
    const long plane0 = (long)blockIdx.x * group;
    const int here = (int)(planes - plane0 < group ? planes - plane0 : group);
    const E* xp = x + plane0 * HW;
    const E* dyp = dy + plane0 * PQ;
    for (int i = threadIdx.x; i < here * HW; i += EB) xs[i] = load_elem(xp + i);
    for (int i = threadIdx.x; i < here * PQ; i += EB) dys[i] = load_elem(dyp + i);
    __syncthreads();
    for (int o = threadIdx.x; o < here * PQ; o += EB) {
        const int pl = o / PQ, pq = o - pl * PQ;
        const int p = pq / g.Q, q = pq - p * g.Q;
        const float* xpl = xs + pl * HW;
        float m = -FLT_MAX;
        int a = -1;
        for (int r = 0; r < g.R; r++) {
            const int ih = p * g.sh - g.ph + r;
            if (ih < 0 || ih >= g.H) continue;
            for (int s_ = 0; s_ < g.S; s_++) {
                const int iw = q * g.sw - g.pw + s_;
                if (iw < 0 || iw >= g.W) continue;
                const float v = xpl[ih * g.W + iw];
                if (a < 0) a = ih * g.W + iw;
                if (v > m) { m = v; a = ih * g.W + iw; }
            }
        }
        arg[o] = a;
    }
    __syncthreads();
    E* dxp = dx + plane0 * HW;
    for (int i = threadIdx.x; i < here * HW; i += EB) {
        const int pl = i / HW, self = i - pl * HW;
        const int h = self / g.W, w = self - h * g.W;
        int p_lo = h + g.ph - g.R + 1; p_lo = p_lo <= 0 ? 0 : (p_lo + g.sh - 1) / g.sh;
        int p_hi = (h + g.ph) / g.sh; if (p_hi > g.P - 1) p_hi = g.P - 1;
        int q_lo = w + g.pw - g.S + 1; q_lo = q_lo <= 0 ? 0 : (q_lo + g.sw - 1) / g.sw;
        int q_hi = (w + g.pw) / g.sw; if (q_hi > g.Q - 1) q_hi = g.Q - 1;
        float acc = 0.0f;
        for (int p = p_lo; p <= p_hi; p++)
            for (int q = q_lo; q <= q_hi; q++)
                if (arg[pl * PQ + p * g.Q + q] == self) acc += dys[pl * PQ + p * g.Q + q];
        if (gate && !(xs[i] > 0.0f)) acc = 0.0f;
        store_elem(dxp + i, acc);
    }
}

// 2x2 stride 2 exact cover: one thread per pair of windows, writes all eight inputs. dx may be x itself: a thread has
// read its eight inputs before it writes the eight gradients, and no other thread touches them.
template <class E>
__global__ void __launch_bounds__(EB) maxpool2x2_bwd_kernel(const E* x, const E* __restrict__ dy, E* dx,
                                                            int H, int W, size_t total_pairs, int gate) {
    const int Q2 = W / 4, P = H / 2;
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < total_pairs; i += stride) {
        const int q2 = (int)(i % Q2);
        const size_t t = i / Q2;
        const int p = (int)(t % P);
        const size_t nc = t / P;
        const size_t off = (nc * H + 2 * (size_t)p) * W + 4 * (size_t)q2;
        const float4 a = ld4(x + off), b = ld4(x + off + W);
        float2 d = ld2(dy + (nc * P + p) * (size_t)(W / 2) + 2 * (size_t)q2);
        // window 0: a.x a.y / b.x b.y ; window 1: a.z a.w / b.z b.w ; first strict maximum wins
        int s0 = 0; float m0 = -FLT_MAX;
        if (a.x > m0) { m0 = a.x; s0 = 0; } if (a.y > m0) { m0 = a.y; s0 = 1; }
        if (b.x > m0) { m0 = b.x; s0 = 2; } if (b.y > m0) { m0 = b.y; s0 = 3; }
        int s1 = 0; float m1 = -FLT_MAX;
        if (a.z > m1) { m1 = a.z; s1 = 0; } if (a.w > m1) { m1 = a.w; s1 = 1; }
        if (b.z > m1) { m1 = b.z; s1 = 2; } if (b.w > m1) { m1 = b.w; s1 = 3; }
        // gated: the winner receives the gradient only where it is positive (the rectifier that produced x)
        if (gate) { d.x = m0 > 0.0f ? d.x : 0.0f; d.y = m1 > 0.0f ? d.y : 0.0f; }
        float4 oa, ob;
        oa.x = s0 == 0 ? d.x : 0.0f; oa.y = s0 == 1 ? d.x : 0.0f; ob.x = s0 == 2 ? d.x : 0.0f; ob.y = s0 == 3 ? d.x : 0.0f;
        oa.z = s1 == 0 ? d.y : 0.0f; oa.w = s1 == 1 ? d.y : 0.0f; ob.z = s1 == 2 ? d.y : 0.0f; ob.w = s1 == 3 ? d.y : 0.0f;
        st4(dx + off, oa);
        st4(dx + off + W, ob);
    }
}

// ---- LRN across channels: window 5, alpha 1e-4, beta 0.75, k 2 -------------------------------------
#define LRN_A5 (1e-4f / 5.0f)
#define LRN_BETA 0.75f
#define LRN_KC 2.0f

// One thread = LRN_CH consecutive channels of one (sample, pixel), lanes along pixels: the channels it needs
// (its own and the halo of the windows) are fetched up front, each window sum is taken in ascending channel
// order, and a value crosses HBM once apart from the halo.
constexpr int LRN_CH = 16;

// scale^-3/4 = r * sqrt(r) with r = scale^-1/2: two hardware approximations of one unit in the last place each and a
// multiply, instead of the general powf (dozens of instructions, which made the kernels wait for the vector ALU, not
// for memory). scale >= 2 always (k = 2, the rest a sum of squares).
__device__ __forceinline__ float lrn_pow_m075(float scale) {
    const float r = __builtin_amdgcn_rsqf(scale);
    return r * __builtin_amdgcn_sqrtf(r);
}

template <class E>
__global__ void __launch_bounds__(EB) lrn_fwd_kernel(const E* __restrict__ x, E* __restrict__ y, int C, int hw, int chunks, size_t total) {
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x; // (sample, chunk, pixel), pixel fastest
    if (i >= total) return;
    const int pix = (int)(i % hw);
    const size_t t = i / hw;
    const int chunk = (int)(t % chunks);
    const size_t n = t / chunks;
    const int c0 = chunk * LRN_CH;
    const E* xp = x + (n * C) * hw + pix;
    E* yp = y + (n * C) * hw + pix;
    float v[LRN_CH + 4]; // channels c0-2 .. c0+LRN_CH+1, zero outside the tensor
#pragma unroll
    for (int k = 0; k < LRN_CH + 4; k++) {
        const int c = c0 - 2 + k;
        v[k] = (c >= 0 && c < C) ? load_elem(xp + (size_t)c * hw) : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < LRN_CH; k++) {
        if (c0 + k >= C) break;
        float ss = 0.0f;
#pragma unroll
        for (int d = 0; d < 5; d++) ss += v[k + d] * v[k + d];
        const float scale = LRN_KC + LRN_A5 * ss;
        store_elem(yp + (size_t)(c0 + k) * hw, v[k + 2] * lrn_pow_m075(scale));
    }
}

template <class E>
__global__ void __launch_bounds__(EB) lrn_bwd_kernel(const E* __restrict__ x, const E* __restrict__ y, const E* __restrict__ dy,
                                                     E* __restrict__ dx, int C, int hw, int chunks, size_t total) {
    const size_t i = (size_t)blockIdx.x * EB + threadIdx.x;
    if (i >= total) return;
    const int pix = (int)(i % hw);
    const size_t t_ = i / hw;
    const int chunk = (int)(t_ % chunks);
    const size_t n = t_ / chunks;
    const int c0 = chunk * LRN_CH;
    const size_t base = (n * C) * hw + pix;
    float xv[LRN_CH + 8];  // channels c0-4 .. c0+LRN_CH+3
    float term[LRN_CH + 4]; // dy*y/scale of channels c0-2 .. c0+LRN_CH+1
    float dyv[LRN_CH + 4];  // dy of the same channels: the thread's own sixteen are among them
    float yv[LRN_CH + 4];
    float scale_own[LRN_CH];
#pragma unroll
    for (int k = 0; k < LRN_CH + 8; k++) {
        const int c = c0 - 4 + k;
        xv[k] = (c >= 0 && c < C) ? load_elem(x + base + (size_t)c * hw) : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < LRN_CH + 4; k++) { // every fetch is issued before the first value is used
        const int c = c0 - 2 + k;
        const bool in = c >= 0 && c < C;
        dyv[k] = in ? load_elem(dy + base + (size_t)c * hw) : 0.0f;
        yv[k] = in ? load_elem(y + base + (size_t)c * hw) : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < LRN_CH + 4; k++) {
        float ss = 0.0f; // the window of channel c0 - 2 + k, ascending
#pragma unroll
        for (int e = 0; e < 5; e++) ss += xv[k + e] * xv[k + e];
        const float scale = LRN_KC + LRN_A5 * ss;
        if (k >= 2 && k < LRN_CH + 2) scale_own[k - 2] = scale;
        term[k] = dyv[k] * yv[k] * __builtin_amdgcn_rcpf(scale); // (zero outside the tensor: dy and y read as zero there)
    }
#pragma unroll
    for (int k = 0; k < LRN_CH; k++) {
        const int c = c0 + k;
        if (c >= C) break;
        float tsum = 0.0f;
#pragma unroll
        for (int d = 0; d < 5; d++) tsum += term[k + d];
        const float dyc = dyv[k + 2];
        store_elem(dx + base + (size_t)c * hw, dyc * lrn_pow_m075(scale_own[k]) - (2.0f * 1e-4f * LRN_BETA / 5.0f) * xv[k + 4] * tsum);
    }
}

// ---- softmax (one workgroup per sample) -------------------------------------------------------------
template <class E>
__global__ void __launch_bounds__(EB) softmax_fwd_kernel(const E* __restrict__ x, E* __restrict__ y, int classes) {
    __shared__ float sh[4];
    const E* xr = x + (size_t)blockIdx.x * classes;
    E* yr = y + (size_t)blockIdx.x * classes;
    float m = -FLT_MAX;
    for (int j = threadIdx.x; j < classes; j += EB) m = fmaxf(m, load_elem(xr + j));
    m = block_max(m, sh);
    float s = 0.0f;
    for (int j = threadIdx.x; j < classes; j += EB) s += expf(load_elem(xr + j) - m);
    s = block_sum(s, sh);
    const float inv = 1.0f / s;
    // the exponentials are evaluated again rather than parked in y: a bfloat16 y is rounded once
    for (int j = threadIdx.x; j < classes; j += EB) store_elem(yr + j, expf(load_elem(xr + j) - m) * inv);
}

template <class E>
__global__ void __launch_bounds__(EB) softmax_bwd_kernel(const E* __restrict__ y, const E* __restrict__ dy, E* __restrict__ dx, int classes) {
    __shared__ float sh[4];
    const size_t base = (size_t)blockIdx.x * classes;
    float dot = 0.0f;
    for (int j = threadIdx.x; j < classes; j += EB) dot += load_elem(dy + base + j) * load_elem(y + base + j);
    dot = block_sum(dot, sh);
    for (int j = threadIdx.x; j < classes; j += EB) store_elem(dx + base + j, load_elem(y + base + j) * (load_elem(dy + base + j) - dot));
}

// per-sample -log p[label] into sample_loss[n]
template <class E>
__global__ void __launch_bounds__(EB) nll_label_kernel(const E* __restrict__ prob, const int32_t* __restrict__ labels, float* __restrict__ sample_loss, int n, int classes) {
    const int i = blockIdx.x * EB + threadIdx.x;
    if (i >= n) return;
    const int lab = labels[i];
    float p = (lab >= 0 && lab < classes) ? load_elem(prob + (size_t)i * classes + lab) : 1.0f;
    sample_loss[i] = -logf(fmaxf(p, FLT_MIN));
}
// per-sample -sum_c target*log p
template <class E>
__global__ void __launch_bounds__(EB) ce_dense_kernel(const E* __restrict__ prob, const E* __restrict__ target, float* __restrict__ sample_loss, int classes) {
    __shared__ float sh[4];
    const size_t base = (size_t)blockIdx.x * classes;
    float s = 0.0f;
    for (int j = threadIdx.x; j < classes; j += EB) {
        const float t = load_elem(target + base + j);
        if (t != 0.0f) s -= t * logf(fmaxf(load_elem(prob + base + j), FLT_MIN));
    }
    s = block_sum(s, sh);
    if (threadIdx.x == 0) sample_loss[blockIdx.x] = s;
}
// loss[0] = mean of sample_loss, summed in sample order by one workgroup
__global__ void __launch_bounds__(EB) mean_kernel(const float* __restrict__ v, float* __restrict__ out, int n) {
    __shared__ float sh[4];
    float s = 0.0f;
    for (int i = threadIdx.x; i < n; i += EB) s += v[i];
    s = block_sum(s, sh);
    if (threadIdx.x == 0) out[0] = s / (float)n;
}
template <class E>
__global__ void __launch_bounds__(EB) softmax_ce_bwd_kernel(const E* __restrict__ prob, const int32_t* __restrict__ labels, E* __restrict__ d, int classes, float inv_n, size_t total) {
    const size_t stride = (size_t)gridDim.x * EB;
    for (size_t i = (size_t)blockIdx.x * EB + threadIdx.x; i < total; i += stride) {
        const int n = (int)(i / classes), j = (int)(i % classes);
        store_elem(d + i, (load_elem(prob + i) - (labels[n] == j ? 1.0f : 0.0f)) * inv_n);
    }
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

} // namespace vdnn

using namespace vdnn;

// ---- launchers, one instance per activation element type ----------------------------------------------
template <class E>
static int relu_fwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* xv, void* yv) {
    VDNN_KERNEL_PROLOGUE(ctx);
    const E* x = (const E*)xv; E* y = (E*)yv;
    VDNN_REQUIRE(x && y, "null tensor");
    if (count == 0) return VDNN_OK;
    const size_t n4 = (aligned16(x) && aligned16(y)) ? count / 4 : 0;
    ProfScope prof(ctx, stream_of(ctx, stream), "relu_fwd", 0.0, 2.0 * sizeof(E) * (double)count);
    hipLaunchKernelGGL(relu_fwd_kernel<E>, dim3(grid_for(n4 ? n4 : count, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), x, y, n4, count);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int relu_bwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* xv, const void* yv, const void* dyv, void* dxv) {
    VDNN_KERNEL_PROLOGUE(ctx);
    const E* t = (const E*)(xv ? xv : yv); const E* dy = (const E*)dyv; E* dx = (E*)dxv;
    VDNN_REQUIRE(t && dy && dx, "null tensor");
    if (count == 0) return VDNN_OK;
    const size_t n4 = (aligned16(t) && aligned16(dy) && aligned16(dx)) ? count / 4 : 0;
    ProfScope prof(ctx, stream_of(ctx, stream), "relu_bwd", 0.0, 3.0 * sizeof(E) * (double)count);
    hipLaunchKernelGGL(relu_bwd_kernel<E>, dim3(grid_for(n4 ? n4 : count, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), t, dy, dx, n4, count);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <int MODE, class E>
static int act_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, const char* name, size_t count, const void* xv, void* yv) {
    VDNN_KERNEL_PROLOGUE(ctx);
    const E* x = (const E*)xv; E* y = (E*)yv;
    VDNN_REQUIRE(x && y, "null tensor");
    if (count == 0) return VDNN_OK;
    const size_t n4 = (aligned16(x) && aligned16(y)) ? count / 4 : 0;
    const size_t threads = n4 > count - n4 * 4 ? n4 : count - n4 * 4;
    ProfScope prof(ctx, stream_of(ctx, stream), name, 0.0, 2.0 * sizeof(E) * (double)count);
    hipLaunchKernelGGL((act_fwd_kernel<MODE, E>), dim3(grid_for(threads, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), x, y, n4, count);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <int MODE, class E>
static int act_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, const char* name, size_t count, const void* yv, const void* dyv, void* dxv) {
    VDNN_KERNEL_PROLOGUE(ctx);
    const E* y = (const E*)yv; const E* dy = (const E*)dyv; E* dx = (E*)dxv;
    VDNN_REQUIRE(y && dy && dx, "null tensor");
    if (count == 0) return VDNN_OK;
    const size_t n4 = (aligned16(y) && aligned16(dy) && aligned16(dx)) ? count / 4 : 0;
    const size_t threads = n4 > count - n4 * 4 ? n4 : count - n4 * 4;
    ProfScope prof(ctx, stream_of(ctx, stream), name, 0.0, 3.0 * sizeof(E) * (double)count);
    hipLaunchKernelGGL((act_bwd_kernel<MODE, E>), dim3(grid_for(threads, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), y, dy, dx, n4, count);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int sub_t(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* a, const void* b, void* r) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(a && b && r, "null tensor");
    if (count == 0) return VDNN_OK;
    hipLaunchKernelGGL(sub_kernel<E>, dim3(grid_for(count, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), (const E*)a, (const E*)b, (E*)r, count);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int fill_t(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, float value, void* p) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(p, "null tensor");
    if (count == 0) return VDNN_OK;
    hipLaunchKernelGGL(fill_kernel<E>, dim3(grid_for(count, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), (E*)p, value, count);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int bias_add_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int k, int hw, const float* bias, void* y) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(bias && y && n > 0 && k > 0 && hw > 0, "bad argument");
    const size_t total = (size_t)n * k * hw;
    hipLaunchKernelGGL(bias_add_kernel<E>, dim3(grid_for(total, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), (E*)y, bias, k, hw, total);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

// The two launches of the convolution bias gradient, shared by the entry points below: stage 1 leaves one partial
// sum per (channel, batch slice) in `partials`, stage 2 adds a channel's partials in slice order. The split of the
// batch depends on the shape and the number of compute units only, so every caller computes the same bits.
static int bias_grad_splits(int N, int K, int num_cu, int* per_out) {
    int splits = (4 * num_cu + K - 1) / K;
    if (splits > N) splits = N;
    if (splits < 1) splits = 1;
    const int per = (N + splits - 1) / splits;
    *per_out = per;
    return (N + per - 1) / per;
}

// stage 2 alone, for kernels that leave the bias gradient's partial sums themselves (partial[k * splits + i])
int vdnn::launch_bias_grad_final(vdnn_ctx* ctx, hipStream_t st, const float* partial, float* bias, int K, int splits, float alpha, int accumulate) {
    ProfScope prof(ctx, st, "conv_bwd_bias_final", 0.0, 4.0 * (double)K * (splits + 2));
    hipLaunchKernelGGL(bias_grad_final_kernel, dim3((K + EB / 64 - 1) / (EB / 64)), dim3(EB), 0, st, partial, bias, K, splits, alpha, accumulate);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int bias_grad_launch(hipStream_t st, const E* dy, float* bias, float* partials, int N, int K, int PQ, int splits, int per,
                            float alpha, int accumulate) {
    hipLaunchKernelGGL(bias_grad_partial_kernel<E>, dim3(K * splits), dim3(EB), 0, st, dy, partials, N, K, PQ, splits, per);
    VDNN_LAUNCH_CHECK();
    hipLaunchKernelGGL(bias_grad_final_kernel, dim3((K + EB / 64 - 1) / (EB / 64)), dim3(EB), 0, st, partials, bias, K, splits, alpha, accumulate);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int conv_bwd_bias_impl(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* dy, float* bias, float alpha, int accumulate) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(shape && dy && bias, "null argument");
    const int N = shape->n, K = shape->k;
    const int P = vdnn_out_dim(shape->h, shape->pad_h, shape->r, shape->stride_h);
    const int Q = vdnn_out_dim(shape->w, shape->pad_w, shape->s, shape->stride_w);
    VDNN_REQUIRE(N > 0 && K > 0 && P > 0 && Q > 0, "bad geometry");
    // split the batch so that K*splits workgroups fill the chip; geometry depends on the shape only
    int per = 0;
    const int splits = bias_grad_splits(N, K, ctx->num_cu, &per);
    // (partial sums in a part of the staging area that no other kernel uses: the call may run on a stream of its own)
    VDNN_REQUIRE(ctx->bias_scratch && (size_t)K * splits * sizeof(float) <= ctx->bias_scratch_bytes, "staging area too small");
    hipStream_t st = stream_of(ctx, stream);
    ProfScope prof(ctx, st, "conv_bwd_bias", 0.0, (double)sizeof(E) * (double)N * K * P * Q);
    return bias_grad_launch<E>(st, (const E*)dy, bias, ctx->bias_scratch, N, K, P * Q, splits, per, alpha, accumulate);
}

// ---- the convolution bias gradient for callers that cannot allocate ---------------------------------------------
// Partial sums of vdnn_conv_bwd_bias_sgd_noalloc live in this array instead of a context's staging area. Every
// device that loads the library holds its own copy at its own address until the process ends. The name below is a
// host-side handle of the symbol, not a device address: host code only ever uses the address that
// hipGetSymbolAddress returned for the device at hand.
static constexpr size_t kNoAllocScratchBytes = VDNN_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) float g_noalloc_scratch[kNoAllocScratchBytes / sizeof(float)];

namespace {
// `ready` is published with release order after `scratch` and `num_cu` are written, and read with acquire order:
// a thread that sees it set sees the two fields. The look-up itself is serialised by a mutex, so two threads that make
// their first call on a device together query once.
struct NoAllocDevice { float* scratch = nullptr; int num_cu = 0; std::atomic<bool> ready{false}; };
constexpr int kMaxDevices = 64;
NoAllocDevice g_noalloc_devices[kMaxDevices];
std::mutex g_noalloc_lookup;
} // namespace

// Address of the current device's copy of the array and that device's number of compute units, looked up once per
// device with that device current. Allocates nothing. The look-up makes two runtime queries (hipGetSymbolAddress,
// hipDeviceGetAttribute): it must not happen while a stream of the calling thread is being captured, so a caller that
// captures runs vdnn_conv_bwd_bias_sgd_noalloc_prepare (or creates a context) on the device beforehand.
static int noalloc_device(NoAllocDevice** out) {
    int dev = -1;
    VDNN_HIP(hipGetDevice(&dev));
    VDNN_REQUIRE(dev >= 0 && dev < kMaxDevices, "device index out of range");
    NoAllocDevice& d = g_noalloc_devices[dev];
    if (!d.ready.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_noalloc_lookup);
        if (!d.ready.load(std::memory_order_relaxed)) {
            float* ptr = nullptr;
            VDNN_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(g_noalloc_scratch)));
            VDNN_REQUIRE(ptr != nullptr, "no address for the scratch array on this device");
            int cus = 0;
            VDNN_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
            VDNN_REQUIRE(cus > 0, "device reports no compute units");
            d.scratch = ptr;
            d.num_cu = cus;
            d.ready.store(true, std::memory_order_release);
        }
    }
    *out = &d;
    return VDNN_OK;
}

namespace vdnn {
// Called by vdnn_ctx_create with the context's device current, so that a later vdnn_conv_bwd_bias_sgd_noalloc on
// that device finds the address already there (a first call under stream capture then makes no query at all).
int noalloc_prepare_current_device() {
    NoAllocDevice* d = nullptr;
    return noalloc_device(&d);
}
} // namespace vdnn

template <class E>
static int fc_bwd_bias_impl(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_out, const void* dy, float* bias, float alpha, int accumulate) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(dy && bias && n > 0 && c_out > 0, "bad argument");
    hipLaunchKernelGGL(fc_bias_grad_kernel<E>, dim3((c_out + EB - 1) / EB), dim3(EB), 0, stream_of(ctx, stream), (const E*)dy, bias, n, c_out, alpha, accumulate);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

static bool pool_geo(const vdnn_shape_t* s, PoolGeo& g) {
    g.N = s->n; g.C = s->c; g.H = s->h; g.W = s->w; g.R = s->r; g.S = s->s;
    g.ph = s->pad_h; g.pw = s->pad_w; g.sh = s->stride_h; g.sw = s->stride_w;
    if (g.N <= 0 || g.C <= 0 || g.H <= 0 || g.W <= 0 || g.R <= 0 || g.S <= 0 || g.sh <= 0 || g.sw <= 0 || g.ph < 0 || g.pw < 0) return false;
    g.P = vdnn_out_dim(g.H, g.ph, g.R, g.sh);
    g.Q = vdnn_out_dim(g.W, g.pw, g.S, g.sw);
    return g.P > 0 && g.Q > 0 && (long)g.H * g.W < (1l << 31);
}

// 3x3 / stride 2 without padding, every window inside the plane (what (H - 3) / 2 + 1 outputs per axis give)
static bool pool_is_3x3_s2(const PoolGeo& g) {
    return g.R == 3 && g.S == 3 && g.sh == 2 && g.sw == 2 && g.ph == 0 && g.pw == 0 && g.H >= 3 && g.W >= 3 &&
           2 * (g.P - 1) + 3 <= g.H && 2 * (g.Q - 1) + 3 <= g.W;
}

static bool pool_is_2x2_exact(const PoolGeo& g, const void* a, const void* b, const void* c) {
    return g.R == 2 && g.S == 2 && g.sh == 2 && g.sw == 2 && g.ph == 0 && g.pw == 0 && g.H % 2 == 0 && g.W % 4 == 0 &&
           aligned16(a) && aligned16(b) && (!c || aligned16(c));
}

template <class E>
static int maxpool_fwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* xv, void* yv) {
    VDNN_KERNEL_PROLOGUE(ctx);
    const E* x = (const E*)xv; E* y = (E*)yv;
    PoolGeo g;
    VDNN_REQUIRE(shape && pool_geo(shape, g), "unsupported pooling geometry");
    VDNN_REQUIRE(x && y, "null tensor");
    hipStream_t st = stream_of(ctx, stream);
    ProfScope prof(ctx, st, "maxpool_fwd", 0.0, (double)sizeof(E) * ((double)g.N * g.C * g.H * g.W + (double)g.N * g.C * g.P * g.Q));
    if (pool_is_2x2_exact(g, x, y, nullptr)) {
        const size_t pairs = (size_t)g.N * g.C * (g.H / 2) * (g.W / 4);
        hipLaunchKernelGGL(maxpool2x2_fwd_kernel<E>, dim3(grid_for(pairs, EB, 0x7FFFFFFF)), dim3(EB), 0, st, x, y, g.H, g.W, pairs);
    } else if (pool_is_3x3_s2(g) && (size_t)g.H * g.W * 4 <= 48 * 1024) {
        // whole planes in LDS: as many per workgroup as give every thread a few elements
        const size_t per_plane = (size_t)g.H * g.W * 4;
        int group = (int)((8 * EB + g.H * g.W - 1) / (g.H * g.W));
        if ((size_t)group * per_plane > 48 * 1024) group = (int)(48 * 1024 / per_plane);
        if (group < 1) group = 1;
        const long planes = (long)g.N * g.C;
        const long blocks = (planes + group - 1) / group;
        VDNN_REQUIRE(blocks < (1l << 31), "grid too large");
        hipLaunchKernelGGL((maxpool_fwd_planes_kernel<E, 3, 3, 2, 2>), dim3((unsigned)blocks), dim3(EB), group * per_plane, st, x, y, g.H, g.W, g.P, g.Q,
                           planes, group, FastDiv::make(g.P * g.Q), FastDiv::make(g.Q));
    } else {
        const size_t total = (size_t)g.N * g.C * g.P * g.Q;
        hipLaunchKernelGGL(maxpool_fwd_kernel<E>, dim3(grid_for(total, EB, 0x7FFFFFFF)), dim3(EB), 0, st, x, y, g, total);
    }
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int maxpool_bwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape,
                         const void* xv, const void* yv, const void* dyv, void* dxv, int gate) {
    VDNN_KERNEL_PROLOGUE(ctx);
    (void)yv; // the winner of each window is recomputed from x with the forward's comparison
    const E* x = (const E*)xv; const E* dy = (const E*)dyv; E* dx = (E*)dxv;
    PoolGeo g;
    VDNN_REQUIRE(shape && pool_geo(shape, g), "unsupported pooling geometry");
    VDNN_REQUIRE(x && dy && dx, "null tensor");
    hipStream_t st = stream_of(ctx, stream);
    ProfScope prof(ctx, st, "maxpool_bwd", 0.0, (double)sizeof(E) * (2.0 * g.N * g.C * g.H * g.W + (double)g.N * g.C * g.P * g.Q));
    VDNN_REQUIRE((const void*)x != (const void*)dx || (pool_is_2x2_exact(g, x, dx, dy) && (g.W / 2) % 2 == 0),
                 "the gradient may be written over the input only by the 2x2 / stride 2 kernel (vdnn_maxpool_bwd_in_place_ok)");
    if (pool_is_2x2_exact(g, x, dx, dy) && (g.W / 2) % 2 == 0) {
        const size_t pairs = (size_t)g.N * g.C * (g.H / 2) * (g.W / 4);
        hipLaunchKernelGGL(maxpool2x2_bwd_kernel<E>, dim3(grid_for(pairs, EB, 0x7FFFFFFF)), dim3(EB), 0, st, x, dy, dx, g.H, g.W, pairs, gate);
    } else if ((size_t)g.H * g.W * 4 + (size_t)g.P * g.Q * 8 <= 48 * 1024) {
        // whole planes in LDS: as many per workgroup as give every thread a few elements
        const size_t per_plane = (size_t)g.H * g.W * 4 + (size_t)g.P * g.Q * 8;
        int group = (int)((4 * EB + g.H * g.W - 1) / (g.H * g.W));
        if ((size_t)group * per_plane > 48 * 1024) group = (int)(48 * 1024 / per_plane);
        if (group < 1) group = 1;
        const long planes = (long)g.N * g.C;
        const long blocks = (planes + group - 1) / group;
        VDNN_REQUIRE(blocks < (1l << 31), "grid too large");
        if (pool_is_3x3_s2(g))
            hipLaunchKernelGGL((maxpool_bwd_planes_fixed_kernel<E, 3, 3, 2, 2>), dim3((unsigned)blocks), dim3(EB), group * per_plane, st, x, dy, dx,
                               g.H, g.W, g.P, g.Q, planes, group, gate, FastDiv::make(g.P * g.Q), FastDiv::make(g.Q), FastDiv::make(g.H * g.W), FastDiv::make(g.W));
        else
            hipLaunchKernelGGL(maxpool_bwd_planes_kernel<E>, dim3((unsigned)blocks), dim3(EB), group * per_plane, st, x, dy, dx, g, planes, group, gate);
    } else {
        const size_t total = (size_t)g.N * g.C * g.H * g.W;
        hipLaunchKernelGGL(maxpool_bwd_kernel<E>, dim3(grid_for(total, EB, 0x7FFFFFFF)), dim3(EB), 0, st, x, dy, dx, g, total, gate);
    }
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int lrn_fwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c, int hw, const void* x, void* y) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(x && y && n > 0 && c > 0 && hw > 0, "bad argument");
    const size_t total = (size_t)n * c * hw;
    const int chunks = (c + LRN_CH - 1) / LRN_CH;
    const size_t threads = (size_t)n * chunks * hw;
    VDNN_REQUIRE((threads + EB - 1) / EB < (1ul << 31), "grid too large");
    ProfScope prof(ctx, stream_of(ctx, stream), "lrn_fwd", 0.0, 2.0 * sizeof(E) * (double)total);
    hipLaunchKernelGGL(lrn_fwd_kernel<E>, dim3(grid_for(threads, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream), (const E*)x, (E*)y, c, hw, chunks, threads);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int lrn_bwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c, int hw, const void* x, const void* y, const void* dy, void* dx) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(x && y && dy && dx && n > 0 && c > 0 && hw > 0, "bad argument");
    const size_t total = (size_t)n * c * hw;
    const int chunks = (c + LRN_CH - 1) / LRN_CH;
    const size_t threads = (size_t)n * chunks * hw;
    VDNN_REQUIRE((threads + EB - 1) / EB < (1ul << 31), "grid too large");
    ProfScope prof(ctx, stream_of(ctx, stream), "lrn_bwd", 0.0, 4.0 * sizeof(E) * (double)total);
    hipLaunchKernelGGL(lrn_bwd_kernel<E>, dim3(grid_for(threads, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream),
                       (const E*)x, (const E*)y, (const E*)dy, (E*)dx, c, hw, chunks, threads);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int softmax_fwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* x, void* y) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(x && y && n > 0 && classes > 0, "bad argument");
    hipLaunchKernelGGL(softmax_fwd_kernel<E>, dim3(n), dim3(EB), 0, stream_of(ctx, stream), (const E*)x, (E*)y, classes);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int softmax_bwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* y, const void* dy, void* dx) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(y && dy && dx && n > 0 && classes > 0, "bad argument");
    hipLaunchKernelGGL(softmax_bwd_kernel<E>, dim3(n), dim3(EB), 0, stream_of(ctx, stream), (const E*)y, (const E*)dy, (E*)dx, classes);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int softmax_ce_fwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* logits,
                            const int32_t* labels, void* prob, float* loss) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(logits && labels && prob && n > 0 && classes > 0, "bad argument");
    hipStream_t st = stream_of(ctx, stream);
    hipLaunchKernelGGL(softmax_fwd_kernel<E>, dim3(n), dim3(EB), 0, st, (const E*)logits, (E*)prob, classes);
    VDNN_LAUNCH_CHECK();
    if (loss) {
        VDNN_REQUIRE((size_t)n * sizeof(float) <= ctx->reduce_scratch_bytes, "staging area too small");
        hipLaunchKernelGGL(nll_label_kernel<E>, dim3((n + EB - 1) / EB), dim3(EB), 0, st, (const E*)prob, labels, ctx->reduce_scratch, n, classes);
        VDNN_LAUNCH_CHECK();
        hipLaunchKernelGGL(mean_kernel, dim3(1), dim3(EB), 0, st, ctx->reduce_scratch, loss, n);
        VDNN_LAUNCH_CHECK();
    }
    return VDNN_OK;
}

template <class E>
static int softmax_ce_bwd_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* prob,
                            const int32_t* labels, void* dlogits) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(prob && labels && dlogits && n > 0 && classes > 0, "bad argument");
    const size_t total = (size_t)n * classes;
    hipLaunchKernelGGL(softmax_ce_bwd_kernel<E>, dim3(grid_for(total, EB, 0x7FFFFFFF)), dim3(EB), 0, stream_of(ctx, stream),
                       (const E*)prob, labels, (E*)dlogits, classes, 1.0f / (float)n, total);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

template <class E>
static int cross_entropy_dense_t(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes,
                                 const void* prob, const void* target, float* loss) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(prob && target && loss && n > 0 && classes > 0, "bad argument");
    VDNN_REQUIRE((size_t)n * sizeof(float) <= ctx->reduce_scratch_bytes, "staging area too small");
    hipStream_t st = stream_of(ctx, stream);
    hipLaunchKernelGGL(ce_dense_kernel<E>, dim3(n), dim3(EB), 0, st, (const E*)prob, (const E*)target, ctx->reduce_scratch, classes);
    VDNN_LAUNCH_CHECK();
    hipLaunchKernelGGL(mean_kernel, dim3(1), dim3(EB), 0, st, ctx->reduce_scratch, loss, n);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

// the same call for either activation element type
#define ACT_CALL(fn, ...) VDNN_BY_ACT(ctx, fn<float>(__VA_ARGS__), fn<bf16_t>(__VA_ARGS__))

extern "C" {

int vdnn_relu_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, void* y) { return ACT_CALL(relu_fwd_t, ctx, stream, count, x, y); }
int vdnn_relu_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, const void* y, const void* dy, void* dx) {
    return ACT_CALL(relu_bwd_t, ctx, stream, count, x, y, dy, dx);
}

int vdnn_tanh_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, void* y) {
    return VDNN_BY_ACT(ctx, (act_fwd<0, float>(ctx, stream, "tanh_fwd", count, x, y)), (act_fwd<0, bf16_t>(ctx, stream, "tanh_fwd", count, x, y)));
}
int vdnn_tanh_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* y, const void* dy, void* dx) {
    return VDNN_BY_ACT(ctx, (act_bwd<0, float>(ctx, stream, "tanh_bwd", count, y, dy, dx)), (act_bwd<0, bf16_t>(ctx, stream, "tanh_bwd", count, y, dy, dx)));
}
int vdnn_sigmoid_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* x, void* y) {
    return VDNN_BY_ACT(ctx, (act_fwd<1, float>(ctx, stream, "sigmoid_fwd", count, x, y)), (act_fwd<1, bf16_t>(ctx, stream, "sigmoid_fwd", count, x, y)));
}
int vdnn_sigmoid_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* y, const void* dy, void* dx) {
    return VDNN_BY_ACT(ctx, (act_bwd<1, float>(ctx, stream, "sigmoid_bwd", count, y, dy, dx)), (act_bwd<1, bf16_t>(ctx, stream, "sigmoid_bwd", count, y, dy, dx)));
}

int vdnn_sub(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, const void* a, const void* b, void* r) { return ACT_CALL(sub_t, ctx, stream, count, a, b, r); }
int vdnn_fill(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, float value, void* p) { return ACT_CALL(fill_t, ctx, stream, count, value, p); }
int vdnn_bias_add(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int k, int hw, const float* bias, void* y) { return ACT_CALL(bias_add_t, ctx, stream, n, k, hw, bias, y); }

int vdnn_conv_bwd_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* dy, float* bias, float alpha) {
    return ACT_CALL(conv_bwd_bias_impl, ctx, stream, shape, dy, bias, alpha, 1);
}
int vdnn_conv_bwd_bias_sgd_noalloc_prepare(void) { return vdnn::noalloc_prepare_current_device(); }
int vdnn_conv_bwd_bias_sgd_noalloc(vdnn_stream_t stream, const vdnn_shape_t* shape, int dtype, const void* dy, float* bias, float alpha) {
    VDNN_REQUIRE(shape && dy && bias, "null argument");
    VDNN_REQUIRE(dtype == VDNN_DTYPE_F32 || dtype == VDNN_DTYPE_BF16, "unknown element type");
    const int N = shape->n, K = shape->k;
    const int P = vdnn_out_dim(shape->h, shape->pad_h, shape->r, shape->stride_h);
    const int Q = vdnn_out_dim(shape->w, shape->pad_w, shape->s, shape->stride_w);
    VDNN_REQUIRE(N > 0 && K > 0 && P > 0 && Q > 0, "bad geometry");
    NoAllocDevice* d = nullptr;
    const int rc = noalloc_device(&d);
    if (rc != VDNN_OK) return rc;
    int per = 0;
    const int splits = bias_grad_splits(N, K, d->num_cu, &per);
    if ((size_t)K * splits * sizeof(float) > kNoAllocScratchBytes) {
        set_error("vdnn_conv_bwd_bias_sgd_noalloc: %d channels x %d batch slices need %zu bytes of partial sums, the built-in scratch "
                  "array holds %zu; use vdnn_conv_bwd_bias_sgd with a context", K, splits, (size_t)K * splits * sizeof(float),
                  kNoAllocScratchBytes);
        return VDNN_EINVAL;
    }
    // stage 1 writes every partial that stage 2 reads: nothing of the last call's contents has to be cleared
    if (dtype == VDNN_DTYPE_BF16)
        return bias_grad_launch<bf16_t>((hipStream_t)stream, (const bf16_t*)dy, bias, d->scratch, N, K, P * Q, splits, per, alpha, 1);
    return bias_grad_launch<float>((hipStream_t)stream, (const float*)dy, bias, d->scratch, N, K, P * Q, splits, per, alpha, 1);
}
int vdnn_conv_bwd_bias(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* dy, float* db) {
    return ACT_CALL(conv_bwd_bias_impl, ctx, stream, shape, dy, db, 1.0f, 0);
}
int vdnn_fc_bwd_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_out, const void* dy, float* bias, float alpha) {
    return ACT_CALL(fc_bwd_bias_impl, ctx, stream, n, c_out, dy, bias, alpha, 1);
}
int vdnn_fc_bwd_bias(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_out, const void* dy, float* db) {
    return ACT_CALL(fc_bwd_bias_impl, ctx, stream, n, c_out, dy, db, 1.0f, 0);
}

// param[i] += alpha * grad[i]: the optimizer step when gradients are kept instead of fused into backward
int vdnn_sgd_apply(vdnn_ctx* ctx, vdnn_stream_t stream, size_t count, float alpha, const float* grad, float* param) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(grad && param, "null tensor");
    if (count == 0) return VDNN_OK;
    hipStream_t st = stream_of(ctx, stream);
    ProfScope prof(ctx, st, "sgd_apply", 0.0, 12.0 * (double)count);
    hipLaunchKernelGGL(sgd_apply_kernel, dim3(grid_for(count, EB, 0x7FFFFFFF)), dim3(EB), 0, st, grad, param, alpha, count);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

int vdnn_maxpool_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* x, void* y) { return ACT_CALL(maxpool_fwd_t, ctx, stream, shape, x, y); }
int vdnn_maxpool_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* x, const void* y, const void* dy, void* dx) {
    return ACT_CALL(maxpool_bwd_t, ctx, stream, shape, x, y, dy, dx, 0);
}
int vdnn_maxpool_bwd_relu(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, const void* x, const void* y, const void* dy, void* dx) {
    return ACT_CALL(maxpool_bwd_t, ctx, stream, shape, x, y, dy, dx, 1);
}
int vdnn_maxpool_bwd_in_place_ok(const vdnn_shape_t* shape) {
    PoolGeo g;
    if (!shape || !pool_geo(shape, g)) return 0;
    return g.R == 2 && g.S == 2 && g.sh == 2 && g.sw == 2 && g.ph == 0 && g.pw == 0 && g.H % 2 == 0 && g.W % 4 == 0;
}
int vdnn_lrn_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c, int hw, const void* x, void* y) { return ACT_CALL(lrn_fwd_t, ctx, stream, n, c, hw, x, y); }
int vdnn_lrn_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c, int hw, const void* x, const void* y, const void* dy, void* dx) {
    return ACT_CALL(lrn_bwd_t, ctx, stream, n, c, hw, x, y, dy, dx);
}
int vdnn_softmax_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* x, void* y) { return ACT_CALL(softmax_fwd_t, ctx, stream, n, classes, x, y); }
int vdnn_softmax_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* y, const void* dy, void* dx) {
    return ACT_CALL(softmax_bwd_t, ctx, stream, n, classes, y, dy, dx);
}
int vdnn_softmax_ce_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* logits, const int32_t* labels, void* prob, float* loss) {
    return ACT_CALL(softmax_ce_fwd_t, ctx, stream, n, classes, logits, labels, prob, loss);
}
int vdnn_softmax_ce_bwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* prob, const int32_t* labels, void* dlogits) {
    return ACT_CALL(softmax_ce_bwd_t, ctx, stream, n, classes, prob, labels, dlogits);
}
int vdnn_cross_entropy_dense(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int classes, const void* prob, const void* target, float* loss) {
    return ACT_CALL(cross_entropy_dense_t, ctx, stream, n, classes, prob, target, loss);
}

} // extern "C"
