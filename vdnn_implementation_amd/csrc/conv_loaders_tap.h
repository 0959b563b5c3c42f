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
