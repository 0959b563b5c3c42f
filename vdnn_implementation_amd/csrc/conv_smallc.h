// Backward data for layers with at most four input channels (the first layer of each network),
// on the vector ALU: the implicit GEMM would have only C <= 4 output rows.
#pragma once
#include <hip/hip_runtime.h>

#include "conv_loaders.h"

namespace vdnn {

// ---- backward data for layers with at most four input channels (the first layer of each network) --
// The implicit GEMM has only C <= 4 output rows, which would fill 3/64 of an MFMA tile; instead one
// thread produces all channels of one input pixel with vector FMAs, summing over (k, r, s) in that
// order. Filters are staged through LDS eight output channels at a time as [k][tap] -> float4 of the
// (zero padded) input channels, so every lane reads the same address (broadcast).
constexpr int SMALLC_KC = 8;
constexpr int SMALLC_MAXTAPS = 128;

// stride 1, any window
template <class E>
__global__ void __launch_bounds__(256) conv_bwd_data_smallc_kernel(const E* __restrict__ dy, const float* __restrict__ w,
                                                                   E* __restrict__ dx, const ConvGeo g) {
    __shared__ float4 ws[SMALLC_KC][SMALLC_MAXTAPS];
    const int tid = threadIdx.x;
    const int RS = g.R * g.S;
    const long pix = (long)blockIdx.x * 256 + tid;
    const long total = (long)g.N * g.H * g.W;
    const bool live = pix < total;
    const long pc = live ? pix : 0;
    const int n = (int)(pc / (g.H * g.W));
    const int hw = (int)(pc - (long)n * g.H * g.W);
    const int h = hw / g.W, x = hw - h * g.W;
    const int th = h + g.ph, tw = x + g.pw;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k0 = 0; k0 < g.K; k0 += SMALLC_KC) {
        __syncthreads();
        for (int i = tid; i < SMALLC_KC * RS; i += 256) {
            const int kk = i / RS, tap = i - kk * RS;
            float v[4] = {0.f, 0.f, 0.f, 0.f};
            if (k0 + kk < g.K)
                for (int c = 0; c < g.C; c++) v[c] = w[((long)(k0 + kk) * g.C + c) * RS + tap];
            ws[kk][tap] = make_float4(v[0], v[1], v[2], v[3]);
        }
        __syncthreads();
        if (!live) continue;
        const int kmax = min(SMALLC_KC, g.K - k0);
        for (int kk = 0; kk < kmax; kk++) {
            const E* dyp = dy + ((long)n * g.K + k0 + kk) * g.P * g.Q;
            for (int r = 0; r < g.R; r++) {
                const int p = th - r;
                if ((unsigned)p >= (unsigned)g.P) continue;
                const E* row = dyp + (long)p * g.Q;
                for (int s = 0; s < g.S; s++) {
                    const int q = tw - s;
                    if ((unsigned)q >= (unsigned)g.Q) continue;
                    const float d = load_elem(row + q);
                    const float4 f = ws[kk][r * g.S + s];
                    acc.x += d * f.x; acc.y += d * f.y; acc.z += d * f.z; acc.w += d * f.w;
                }
            }
        }
    }
    if (!live) return;
    E* o = dx + (long)n * g.C * g.H * g.W + hw;
    const long plane = (long)g.H * g.W;
    store_elem(o, acc.x);
    if (g.C > 1) store_elem(o + plane, acc.y);
    if (g.C > 2) store_elem(o + 2 * plane, acc.z);
    if (g.C > 3) store_elem(o + 3 * plane, acc.w);
}

// Strided layers (AlexNet / OverFeat conv1: 11x11, stride 4). An input pixel only receives the taps
// congruent to its position modulo the stride, so pixels are grouped by residue class (th mod sh,
// tw mod sw): within a class every pixel uses the same taps, the filter reads are wavefront-uniform
// and consecutive lanes read consecutive dy columns. One workgroup = 256 pixels of one class of one
// sample; summation order per pixel is (k, r, s) ascending as in the kernels above.
template <class E>
__global__ void __launch_bounds__(256) conv_bwd_data_smallc_strided_kernel(const E* __restrict__ dy, const float* __restrict__ w,
                                                                           E* __restrict__ dx, const ConvGeo g, int Ht, int Wt, int blocks_per_class) {
    __shared__ float4 ws[SMALLC_KC][SMALLC_MAXTAPS];
    const int tid = threadIdx.x;
    const int RS = g.R * g.S;
    const int classes = g.sh * g.sw;
    const int blk = blockIdx.x % blocks_per_class;
    const int rest = blockIdx.x / blocks_per_class;
    const int cls = rest % classes, n = rest / classes;
    const int rh = cls / g.sw, rw = cls - rh * g.sw;
    const int idx = blk * 256 + tid;
    const int i = idx / Wt, j = idx - i * Wt;
    const int th = i * g.sh + rh, tw = j * g.sw + rw;
    const int h = th - g.ph, x = tw - g.pw;
    const bool live = i < Ht && h >= 0 && h < g.H && x >= 0 && x < g.W;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int k0 = 0; k0 < g.K; k0 += SMALLC_KC) {
        __syncthreads();
        for (int t = tid; t < SMALLC_KC * RS; t += 256) {
            const int kk = t / RS, tap = t - kk * RS;
            float v[4] = {0.f, 0.f, 0.f, 0.f};
            if (k0 + kk < g.K)
                for (int c = 0; c < g.C; c++) v[c] = w[((long)(k0 + kk) * g.C + c) * RS + tap];
            ws[kk][tap] = make_float4(v[0], v[1], v[2], v[3]);
        }
        __syncthreads();
        if (!live) continue;
        const int kmax = min(SMALLC_KC, g.K - k0);
        for (int kk = 0; kk < kmax; kk++) {
            const E* dyp = dy + ((long)n * g.K + k0 + kk) * g.P * g.Q;
            for (int r = rh, p = i; r < g.R && p >= 0; r += g.sh, p--) {
                if (p >= g.P) continue;
                const E* row = dyp + (long)p * g.Q;
                for (int s = rw, q = j; s < g.S && q >= 0; s += g.sw, q--) {
                    if (q >= g.Q) continue;
                    const float d = load_elem(row + q);
                    const float4 f = ws[kk][r * g.S + s];
                    acc.x += d * f.x; acc.y += d * f.y; acc.z += d * f.z; acc.w += d * f.w;
                }
            }
        }
    }
    if (!live) return;
    E* o = dx + ((long)n * g.C * g.H + h) * g.W + x;
    const long plane = (long)g.H * g.W;
    store_elem(o, acc.x);
    if (g.C > 1) store_elem(o + plane, acc.y);
    if (g.C > 2) store_elem(o + 2 * plane, acc.z);
    if (g.C > 3) store_elem(o + 3 * plane, acc.w);
}

// Second stage of the strided few-channel backward data on the matrix cores. The first stage is a 1x1
// convolution T[n][(c,r,s)][p][q] = sum_k w[k,c,r,s] * dy[n,k,p,q] (every product the layer needs, once);
// here an input pixel adds up the entries whose tap lands on it: dx[n,c,h,x] = sum over taps (r,s) with
// (h+ph-r) = p*sh and (x+pw-s) = q*sw of T[n][(c,r,s)][p][q], taps in ascending (r,s) order.
template <class E>
__global__ void __launch_bounds__(256) conv_bwd_data_gather_taps_kernel(const float* __restrict__ T, E* __restrict__ dx, const ConvGeo g, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int x = (int)(i % g.W);
    long t = i / g.W;
    const int h = (int)(t % g.H); t /= g.H;
    const int c = (int)(t % g.C);
    const long n = t / g.C;
    const int PQ = g.P * g.Q;
    const float* Tc = T + (n * g.C + c) * (long)g.R * g.S * PQ;
    float acc = 0.0f;
    for (int r = (h + g.ph) % g.sh; r < g.R; r += g.sh) {
        const int p = (h + g.ph - r) / g.sh;
        if (h + g.ph - r < 0) break;
        if (p >= g.P) continue;
        for (int s = (x + g.pw) % g.sw; s < g.S; s += g.sw) {
            const int q = (x + g.pw - s) / g.sw;
            if (x + g.pw - s < 0) break;
            if (q >= g.Q) continue;
            acc += Tc[(long)(r * g.S + s) * PQ + p * g.Q + q];
        }
    }
    store_elem(dx + i, acc);
}

// The same, for a compile-time window at stride 1 (VGG's 3x3): fully unrolled and branch-free. Taps
// outside dy are read from a clamped position and replaced by zero. The filter values of one output
// channel are wave-uniform, so they are fetched with scalar loads straight from global memory.
template <int RC, int SC, int CC, class E>
__global__ void __launch_bounds__(256) conv_bwd_data_smallc_s1_kernel(const E* __restrict__ dy, const float* __restrict__ w,
                                                                      E* __restrict__ dx, const ConvGeo g) {
    constexpr int RS = RC * SC;
    const int tid = threadIdx.x;
    const long pix = (long)blockIdx.x * 256 + tid;
    const long total = (long)g.N * g.H * g.W;
    const bool live = pix < total;
    const long pc = live ? pix : 0;
    const int n = (int)(pc / (g.H * g.W));
    const int hw = (int)(pc - (long)n * g.H * g.W);
    const int h = hw / g.W, x = hw - h * g.W;
    int rowoff[RC], col[SC];
    bool rowok[RC], colok[SC];
#pragma unroll
    for (int r = 0; r < RC; r++) {
        const int p = h + g.ph - r;
        rowok[r] = (unsigned)p < (unsigned)g.P;
        rowoff[r] = rowok[r] ? p * g.Q : 0;
    }
#pragma unroll
    for (int s = 0; s < SC; s++) {
        const int q = x + g.pw - s;
        colok[s] = (unsigned)q < (unsigned)g.Q;
        col[s] = colok[s] ? q : 0;
    }
    float acc[CC];
#pragma unroll
    for (int c = 0; c < CC; c++) acc[c] = 0.f;
    const long kstride = (long)g.P * g.Q;
    const E* dyp = dy + (long)n * g.K * kstride;
    for (int k = 0; k < g.K; k++, dyp += kstride) {
        const float* wk = w + (long)k * CC * RS; // uniform: scalar loads
#pragma unroll
        for (int r = 0; r < RC; r++) {
            const E* row = dyp + rowoff[r];
#pragma unroll
            for (int s = 0; s < SC; s++) {
                const float v = load_elem(row + col[s]);
                const float d = (rowok[r] & colok[s]) ? v : 0.0f;
#pragma unroll
                for (int c = 0; c < CC; c++) acc[c] += d * wk[c * RS + r * SC + s];
            }
        }
    }
    if (!live) return;
    E* o = dx + (long)n * CC * g.H * g.W + hw;
    const long plane = (long)g.H * g.W;
#pragma unroll
    for (int c = 0; c < CC; c++) store_elem(o + c * plane, acc[c]);
}

// ---- backward filter for 3x3 layers with at most four input channels ------------------------------
// The implicit GEMM has only C*9 <= 36 columns, which would fill a tenth of a 256-wide MFMA tile, and
// the pass is bound by reading dy once. Lanes run along output pixels (coalesced dy and x reads); one
// thread keeps the C*9 products of KG output channels in registers, walks its share of one chunk of
// pixels, and the workgroup's sums go to partial[chunk][k][c][tap] in a fixed order (wavefront
// shuffle tree, then the four wavefronts in order). The chunks are added in order by the split
// reduction that also applies the SGD step.
struct PixelStep { int dn, dp, dq; }; // 256 pixels = dn samples + dp rows + dq columns

template <int CC, int KG, class E>
__global__ void __launch_bounds__(256) conv_bwd_filter_smallc3x3_kernel(const E* __restrict__ dy, const E* __restrict__ x,
                                                                        float* __restrict__ partial, const ConvGeo g,
                                                                        long pix_per_chunk, PixelStep step) {
    constexpr int TAPS = CC * 9;
    __shared__ float red[4][KG * TAPS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kgroups = g.K / KG;
    const int kg = blockIdx.x % kgroups;
    const long chunk = blockIdx.x / kgroups;
    const long total = (long)g.N * g.P * g.Q;
    const long pix0 = chunk * pix_per_chunk;
    const long pix1 = pix0 + pix_per_chunk < total ? pix0 + pix_per_chunk : total;
    const int PQ = g.P * g.Q;
    long pix = pix0 + tid;
    int n = (int)(pix / PQ);
    int rem = (int)(pix - (long)n * PQ);
    int p = rem / g.Q, q = rem - p * g.Q;

    float acc[KG][TAPS];
#pragma unroll
    for (int j = 0; j < KG; j++)
#pragma unroll
        for (int t = 0; t < TAPS; t++) acc[j][t] = 0.0f;

    const long plane = (long)g.H * g.W;
    for (; pix < pix1; pix += 256) {
        const int ih0 = p * g.sh - g.ph, iw0 = q * g.sw - g.pw;
        const E* xs = x + (long)n * CC * plane;
        float xv[TAPS];
#pragma unroll
        for (int r = 0; r < 3; r++) {
            const int ih = ih0 + r;
            const bool vr = (unsigned)ih < (unsigned)g.H;
            const int ihc = vr ? ih : 0;
#pragma unroll
            for (int t = 0; t < 3; t++) {
                const int iw = iw0 + t;
                const bool v = vr & ((unsigned)iw < (unsigned)g.W);
                const int iwc = ((unsigned)iw < (unsigned)g.W) ? iw : 0;
#pragma unroll
                for (int c = 0; c < CC; c++) {
                    const float val = load_elem(xs + c * plane + (long)ihc * g.W + iwc);
                    xv[c * 9 + r * 3 + t] = v ? val : 0.0f;
                }
            }
        }
        const E* dyp = dy + ((long)n * g.K + kg * KG) * PQ + p * g.Q + q;
#pragma unroll
        for (int j = 0; j < KG; j++) {
            const float d = load_elem(dyp + (long)j * PQ);
#pragma unroll
            for (int t = 0; t < TAPS; t++) acc[j][t] += d * xv[t];
        }
        // advance 256 pixels
        q += step.dq;
        const int cq = q >= g.Q;
        q -= cq ? g.Q : 0;
        p += step.dp + cq;
        const int cp = p >= g.P;
        p -= cp ? g.P : 0;
        n += step.dn + cp;
    }

#pragma unroll
    for (int j = 0; j < KG; j++)
#pragma unroll
        for (int t = 0; t < TAPS; t++) {
            float v = acc[j][t];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
            if (lane == 0) red[wave][j * TAPS + t] = v;
        }
    __syncthreads();
    if (tid < KG * TAPS) {
        const float v = ((red[0][tid] + red[1][tid]) + red[2][tid]) + red[3][tid];
        partial[chunk * ((long)g.K * TAPS) + (long)kg * KG * TAPS + tid] = v;
    }
}

} // namespace vdnn
