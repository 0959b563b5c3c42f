// Blocked tap-major reduction order for convolutions whose reduced channel count is a multiple of the
// slice depth: reduction index kk = (channel block * RS + tap) * 16 + channel in block, so one 16-deep
// slice is one filter tap (r, s) and 16 consecutive channels, and the RS slices of a channel block
// follow each other (the same filter lines and the same rows of the activation tensor stay hot in
// L1/L2 across the taps). Everything that depends on the tap - its offset, the lane's "this tap is
// outside the image" bit - is then computed once per slice instead of once per load: the im2col side
// needs two vector instructions per slice, the filter side none. (The sum over (c, r, s) is merely
// taken in a different order than channel-major.)
#pragma once
#include "conv_loaders.h"

namespace vdnn {

// ---- filter operand: element (row, channel l, tap) at w[row*row_stride + l*red_stride + tap] --------
//   forward:        rows = output channels k, l = input channel c : row_stride = C*RS, red_stride = RS
//   backward data:  rows = input channels c,  l = output channel k: row_stride = RS,   red_stride = C*RS
// The slice's (tap, first channel) goes into the scalar offset; per-lane offsets are constants.
// Lanes of a 16-lane group run along whichever index is close in memory: the channel l in forward
// (thread t: l = t%16, rows t/16 + 16*i), the row in backward data (thread t: rows t%16 + 16*i, l = t/16).
template <bool LANES_ALONG_ROWS>
struct LoadFilterTap {
    static constexpr bool RED_MAJOR = true;
    const float* w;
    int row_stride, red_stride, rows, RS;
    unsigned bytes;
    FastDiv divRS;
    template <int T> struct Regs { float s[T / 16]; };
    template <int T> struct State { int vrow[T / 16]; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(w, bytes);
#pragma unroll
        for (int i = 0; i < T / 16; i++) {
            const int row = row0 + (LANES_ALONG_ROWS ? (tid & 15) : (tid >> 4)) + 16 * i;
            const int l = LANES_ALONG_ROWS ? (tid >> 4) : (tid & 15);
            st.vrow[i] = row < rows ? (row * row_stride + l * red_stride) * 4 : OOB;
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int, int, Regs<T>& r) const {
        const int slice = kk0 / KB;
        const int cb = divRS.div(slice), tap = slice - cb * RS;
        const int soff = (cb * KB * red_stride + tap) * 4;
#pragma unroll
        for (int i = 0; i < T / 16; i++) r.s[i] = buf_load(st.rsrc, st.vrow[i], soff);
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 16; i++) {
            if (LANES_ALONG_ROWS) lds[((tid & 15) + 16 * i) * RED_STRIDE + (tid >> 4)] = r.s[i];
            else lds[((tid >> 4) + 16 * i) * RED_STRIDE + (tid & 15)] = r.s[i];
        }
    }
};

// ---- im2col operand, columns = output pixels, tap-major reduction ------------------------------------
// MODE 0: forward gather from x; MODE 1: backward data at stride 1 (src = dy). At most 32 taps.
template <int MODE, class E = float>
struct LoadIm2colPixTap {
    static constexpr bool RED_MAJOR = false;
    static constexpr int ES = ElemBytes<E>::V;
    LoadIm2colPix<MODE, false, E> base; // geometry and per-pixel state are those of the channel-major loader
    template <int T> using Regs = typename LoadIm2colPix<MODE, false, E>::template Regs<T>;
    template <int T> using State = typename LoadIm2colPix<MODE, false, E>::template State<T>;
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int ncols, int k_begin) const {
        base.template init<T>(st, j0, tid, ncols, k_begin);
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int, int tid, Regs<T>& r) const {
        const int plane = base.Hs * base.Ws;
        const int slice = kk0 / KB;
        const int cb = base.divRS.div(slice), tap = slice - cb * (base.R * base.S), ch0 = cb * KB;
        const int tr = base.divS.div(tap), ts = tap - tr * base.S;
        const int tapoff = MODE == 0 ? tr * base.Ws + ts : (base.R - 1 - tr) * base.Ws + (base.S - 1 - ts);
        const int voff = st.vbase | bit_to_all_ones(st.inv, tap);
        const int chb = ch0 + __builtin_amdgcn_readfirstlane(tid / T);
        const int soff0 = (chb * plane + tapoff) * ES, step = (NT / T) * plane * ES;
#pragma unroll
        for (int i = 0; i < T * KB / NT; i++) r.s[i] = buf_load_e<E>(st.rsrc, voff, soff0 + i * step);
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
        LoadIm2colPix<MODE, false, E>::template store<T>(lds, tid, r);
    }
};

} // namespace vdnn

namespace vdnn {

// ---- im2col operand of backward filter, columns in tap-major order: B[(n,p,q)][tap*C + c] -------------
// The filter gradient's columns are taken as (tap, channel) instead of (channel, tap), so that the T
// columns of a tile share one tap (C a multiple of T) or fall into NTAP groups of T/NTAP channels with
// one tap each (C = T/NTAP). A thread owns pixel t%16 of the slice and columns t/16 + 16*i, as in the
// channel-major loader, but the tap - its offset and whether it falls outside the image for the
// thread's pixel - is then a per-slice quantity per group instead of per load: a load costs one vector
// add. The epilogue StoreFilterTap puts the result back into the filter's (k, c, r, s) layout.
template <int NTAP, class E = float>
struct LoadIm2colRedTap {
    static constexpr bool RED_MAJOR = true;
    static constexpr int ES = ElemBytes<E>::V;
    const E* x;
    int N, C, H, W, R, S, P, Q, ph, pw, sh, sw;
    int ncols; // C*R*S
    int kchunk, Ktot;
    FastDiv divC, divS;
    template <int T> struct Regs { float s[T / 16]; };
    // The vector unit is shared with the MFMAs, so the per-slice address work is kept to adds, compares
    // and selects on three carried quantities: the input row and column the thread's pixel reads through
    // the first group's tap, and the byte offset of that element in the thread's first channel plane.
    // A slice moves the pixel KB places along (n, p, q); up to two row wraps (Q >= KB/2) and one sample
    // wrap (P*Q >= KB) are applied without branches. Pixels past the end of the reduction lie in the
    // sample after the descriptor's range and read as zero, as do the matching values of the other
    // operand, so no liveness test is needed; the columns of a group are whole channel planes apart
    // (scalar offsets of the load instructions).
    template <int T> struct State {
        int ih, iw;          // p*sh - ph + r0, q*sw - pw + s0 for the first group's tap (r0, s0)
        int off;             // byte offset of (n, c_thread, ih, iw) from the descriptor base
        int dih[NTAP], diw[NTAP], doff[NTAP]; // further groups relative to the first (wave-uniform)
        int iw_wrap, ih_wrap; // values of iw / ih at which the row / the sample ends
        __amdgpu_buffer_rsrc_t rsrc;
    };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int, int k_begin) const {
        const int PQ = P * Q;
        const int n_first = k_begin / PQ;
        const long chw = (long)C * H * W;
        const long shift = -((long)ph * W + pw);
        int k_last = k_begin + kchunk; if (k_last > Ktot) k_last = Ktot;
        const int n_last = k_last > k_begin ? (k_last - 1) / PQ : n_first;
        st.rsrc = make_rsrc(x + (long)n_first * chw + shift, clamp_range(((long)(n_last - n_first + 1) * chw - shift) * ES));
        const int kk = k_begin + (tid & 15);
        const int n = kk / PQ, pq = kk - n * PQ;
        const int p = pq / Q, q = pq - p * Q;
        int r0 = 0, s0 = 0, c0 = 0;
#pragma unroll
        for (int g = 0; g < NTAP; g++) {
            const int jg = j0 + g * (T / NTAP);           // one tap per group of T/NTAP columns
            const int tap = divC.div(jg);
            const int r = divS.div(tap), s_ = tap - r * S;
            const int c = jg - tap * C;
            if (g == 0) { r0 = r; s0 = s_; c0 = c; st.dih[0] = 0; st.diw[0] = 0; st.doff[0] = 0; }
            else {
                st.dih[g] = jg < ncols ? r - r0 : 0x20000000; // a group past the last tap never passes the row test
                st.diw[g] = s_ - s0;
                st.doff[g] = (((r - r0) * W + (s_ - s0)) + (c - c0) * H * W) * ES;
            }
        }
        st.ih = p * sh - ph + r0; st.iw = q * sw - pw + s0;
        st.iw_wrap = Q * sw - pw + s0; st.ih_wrap = P * sh - ph + r0;
        st.off = (int)(((long)(n - n_first) * chw + (long)(c0 + (tid >> 4)) * H * W + (long)(p * sh + r0) * W + q * sw + s0) * ES);
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int, int, Regs<T>& r) const {
        int base[NTAP];
#pragma unroll
        for (int g = 0; g < NTAP; g++) {
            const bool ok = g == 0 ? ((unsigned)st.ih < (unsigned)H) & ((unsigned)st.iw < (unsigned)W)
                                   : ((unsigned)(st.ih + st.dih[g]) < (unsigned)H) & ((unsigned)(st.iw + st.diw[g]) < (unsigned)W);
            base[g] = (g == 0 ? st.off : st.off + st.doff[g]) | (ok ? 0 : SENT);
        }
        constexpr int PERG = T / 16 / NTAP;
        const int plane16 = 16 * H * W * ES;
#pragma unroll
        for (int i = 0; i < T / 16; i++) r.s[i] = buf_load_e<E>(st.rsrc, base[i / PERG], (i % PERG) * plane16);
        // next slice: KB pixels further
        st.iw += KB * sw; st.off += KB * sw * ES;
        const int qsw = Q * sw;
        const int wraps = (st.iw >= st.iw_wrap ? 1 : 0) + (st.iw >= st.iw_wrap + qsw ? 1 : 0);
        st.iw -= __mul24(wraps, qsw);
        st.ih += __mul24(wraps, sh);
        st.off += __mul24(wraps, (sh * W - qsw) * ES);
        const bool next = st.ih >= st.ih_wrap;                // into the next sample
        st.ih -= next ? P * sh : 0;
        st.off += next ? (C * H * W - P * sh * W) * ES : 0;
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 16; i++) lds[((tid >> 4) + 16 * i) * RED_STRIDE + (tid & 15)] = r.s[i];
    }
};

// Result of the tap-major backward filter: GEMM column j = tap*C + c is filter element (m, c, tap) at
// out[m*ncols + c*RS + tap]. A split's partial sums stay in GEMM order (coalesced stores); the ordered
// sum over the splits puts them into the filter's layout.
struct StoreFilterTap {
    float* out;
    float* partial;
    int C, RS;
    long partial_stride;
    float alpha;
    int accumulate;
    FastDiv divC;
    static constexpr bool TAIL = false;
    __device__ __forceinline__ void store_tail(const floatx16 (&)[2][2], int, int, int, long, int, int) const {}
    __device__ __forceinline__ void store(const floatx16 (&acc)[2][2], int m0, int j0, int lane, int ks, const GemmDims& d, bool to_partial) const {
        const int l32 = lane & 31, lk = lane >> 5;
#pragma unroll
        for (int jt = 0; jt < 2; jt++) {
            const int j = j0 + jt * 32 + l32;
            if (j >= d.N) continue;
            const int tap = divC.div(j), c = j - tap * C;
            const long col = (long)c * RS + tap;
#pragma unroll
            for (int it = 0; it < 2; it++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                    if (m >= d.M) continue;
                    const long idx = (long)m * d.N + col;
                    const float a = acc[it][jt][v];
                    if (to_partial) partial[(long)ks * partial_stride + (long)m * d.N + j] = a;
                    else out[idx] = accumulate ? __fmaf_rn(alpha, a, out[idx]) : alpha * a;
                }
        }
    }
};

// Filter bank re-laid-out for the blocked tap-major order (the workspace of the perf-optimal mode):
// packed[row][(cb*RS + tap)*16 + l] = w[row*row_stride + (cb*16 + l)*red_stride + tap], so that the A
// operand becomes a dense reduction-major matrix read with 128-bit loads.
__global__ void __launch_bounds__(256) pack_filter_tap_kernel(const float* __restrict__ w, float* __restrict__ packed,
                                                              int rows, int Cred, int RS, int row_stride, int red_stride, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int per_row = Cred * RS;
    const int row = (int)(i / per_row), kk = (int)(i - (long)row * per_row);
    const int l = kk & 15, slice = kk >> 4;
    const int cb = slice / RS, tap = slice - cb * RS;
    packed[i] = w[(long)row * row_stride + (long)(cb * 16 + l) * red_stride + tap];
}

} // namespace vdnn
