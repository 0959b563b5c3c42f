// Operand loaders of the convolution kernels: filter banks and im2col views of NCHW tensors for the
// MFMA tile engine. Every loader fetches through a buffer descriptor so that padding taps, tile
// edges and the end of a reduction range read as zero without branches or selects.
#pragma once
#include "mfma_gemm.h"

namespace vdnn {

struct ConvGeo {
    int N, C, H, W, K, R, S, P, Q, ph, pw, sh, sw;
};

// bit `pos` of `mask` as 0 / -1 (one v_bfe_i32)
__device__ __forceinline__ int bit_to_all_ones(unsigned mask, int pos) { return __builtin_amdgcn_sbfe((int)mask, (unsigned)pos, 1u); }

// valid positions t in [0, window) with 0 <= origin + t < extent, as a bit mask
__device__ __forceinline__ unsigned valid_window_bits(int origin, int window, int extent) {
    int lo = -origin; if (lo < 0) lo = 0;
    int hi = extent - origin; if (hi > window) hi = window;
    if (hi <= lo) return 0u;
    return ((1u << hi) - 1u) & ~((1u << lo) - 1u);
}

// ---- im2col operand, columns = output pixels (row-major in LDS: lanes run along pixels) ---------
// MODE 0: forward gather from x.          src[n, ch, oh*sh-ph+r, ow*sw-pw+s]
// MODE 1: backward data, stride 1.        src[n, ch, oh+ph-r,    ow+pw-s]          (src = dy)
// MODE 2: backward data, any stride.      src[n, ch, (oh+ph-r)/sh, (ow+pw-s)/sw] where divisible
// A lane owns one pixel for the whole kernel: its byte offset goes into the per-lane offset, the tap
// (ch, r, s) is wave-uniform and goes into the scalar offset, and the pixel's out-of-image taps are a
// bit mask that is OR-ed into the offset as all-ones. BIGWIN: windows of more than 32 taps keep
// separate row and column masks.
template <int MODE, bool BIGWIN, class E = float>
struct LoadIm2colPix {
    static constexpr bool RED_MAJOR = false;
    static constexpr int ES = ElemBytes<E>::V;
    const E* src;
    int Hs, Ws;      // extent of one source plane
    int OH, OW;      // extent of the output pixel grid
    int R, S, ph, pw, sh, sw;
    long sample_elems; // channels_of_src * Hs * Ws
    int nsamples;
    FastDiv divRS, divS;
    template <int T> struct Regs { float s[T * KB / NT]; };
    template <int T> struct State {
        int vbase;                 // byte offset of the pixel (MODE 2: of its sample) from the descriptor base
        unsigned inv, invrow, invcol; // bit set = tap reads as zero
        int ih0, iw0;              // MODE 2
        __amdgpu_buffer_rsrc_t rsrc;
    };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int ncols, int) const {
        const int opix = OH * OW;
        const int j = j0 + tid % T;
        const bool valid = j < ncols;
        const int jj = valid ? j : j0;
        const int n_first = j0 / opix;
        const int n = jj / opix, pix = jj - n * opix;
        const int oh = pix / OW, ow = pix - oh * OW;
        const long first = (long)n_first * sample_elems;
        long shift; // descriptor base relative to the first sample, in elements (<= 0)
        int ih0, iw0;
        if (MODE == 0) {
            shift = -((long)ph * Ws + pw);
            ih0 = oh * sh - ph; iw0 = ow * sw - pw;
            st.vbase = (int)(((long)(n - n_first) * sample_elems + (long)oh * sh * Ws + ow * sw) * ES);
        } else if (MODE == 1) {
            shift = (long)(ph - R + 1) * Ws + (pw - S + 1);
            ih0 = oh + ph; iw0 = ow + pw;
            st.vbase = (int)(((long)(n - n_first) * sample_elems + (long)oh * Ws + ow) * ES);
        } else {
            shift = 0;
            ih0 = oh + ph; iw0 = ow + pw;
            st.vbase = (int)((long)(n - n_first) * sample_elems * ES);
        }
        st.ih0 = ih0; st.iw0 = iw0;
        // the descriptor covers only the samples this tile touches (the host checks that this is
        // below 2 GiB, so the scalar offset 0x7FFFFFF0 of an exhausted reduction range is out of range)
        int n_last = (j0 + T - 1) / opix;
        if (n_last > nsamples - 1) n_last = nsamples - 1;
        st.rsrc = make_rsrc(src + first + shift, clamp_range(((long)(n_last - n_first + 1) * sample_elems - shift) * ES));
        unsigned vrow = 0, vcol = 0; // valid taps
        for (int r = 0; r < R; r++) {
            bool ok;
            if (MODE == 0) ok = (unsigned)(ih0 + r) < (unsigned)Hs;
            else if (MODE == 1) ok = (unsigned)(ih0 - r) < (unsigned)Hs;
            else { const int t = ih0 - r; ok = t >= 0 && t % sh == 0 && t / sh < Hs; }
            if (ok) vrow |= 1u << r;
        }
        for (int s = 0; s < S; s++) {
            bool ok;
            if (MODE == 0) ok = (unsigned)(iw0 + s) < (unsigned)Ws;
            else if (MODE == 1) ok = (unsigned)(iw0 - s) < (unsigned)Ws;
            else { const int t = iw0 - s; ok = t >= 0 && t % sw == 0 && t / sw < Ws; }
            if (ok) vcol |= 1u << s;
        }
        if (!valid) { vrow = 0; vcol = 0; }
        st.invrow = ~vrow; st.invcol = ~vcol;
        unsigned v = 0;
        if (!BIGWIN)
            for (int r = 0; r < R; r++) if ((vrow >> r) & 1u) v |= vcol << (r * S);
        st.inv = ~v;
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int kend, int tid, Regs<T>& r) const {
        const int RS = R * S, plane = Hs * Ws;
        // every lane of a wavefront shares kk: the tap arithmetic stays on the scalar unit
        const int kbase = __builtin_amdgcn_readfirstlane(kk0 + tid / T);
#pragma unroll
        for (int i = 0; i < T * KB / NT; i++) {
            const int kk = kbase + (NT / T) * i;
            const int ch = divRS.div(kk), rs = kk - ch * RS;
            const int tr = divS.div(rs), ts = rs - tr * S;
            int soff, voff;
            if (MODE == 0) soff = (ch * plane + tr * Ws + ts) * ES;
            else if (MODE == 1) soff = (ch * plane + (R - 1 - tr) * Ws + (S - 1 - ts)) * ES;
            else soff = ch * plane * ES;
            if (kk >= kend) soff = 0x7FFFFFF0;
            const int dead = BIGWIN || MODE == 2 ? (bit_to_all_ones(st.invrow, tr) | bit_to_all_ones(st.invcol, ts)) : bit_to_all_ones(st.inv, rs);
            if (MODE == 2) voff = (st.vbase + (((st.ih0 - tr) / sh) * Ws + (st.iw0 - ts) / sw) * ES) | dead;
            else voff = st.vbase | dead;
            r.s[i] = buf_load_e<E>(st.rsrc, voff, soff);
        }
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T * KB / NT; i++) lds[(tid / T + (NT / T) * i) * T + tid % T] = r.s[i];
    }
};

// ---- filter bank as the A operand of backward data: A[c][(k,r,s)] = w[k,c,r,s] ------------------
// a gather (runs of R*S contiguous values): 32-bit loads, thread t: kk t%16 of rows t/16 + 16*i
struct LoadFilterT {
    static constexpr bool RED_MAJOR = true;
    const float* w;
    int C, RS;
    unsigned bytes; // below MAX_SUM_RANGE
    FastDiv divRS;
    template <int T> struct Regs { float s[T / 16]; };
    template <int T> struct State { int crow[T / 16]; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(w, bytes);
#pragma unroll
        for (int i = 0; i < T / 16; i++) {
            const int c = row0 + (tid >> 4) + 16 * i;
            st.crow[i] = c < C ? c * RS * 4 : SENT;
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int kend, int tid, Regs<T>& r) const {
        const int kk = kk0 + (tid & 15);
        const int k = divRS.div(kk), rs = kk - k * RS;
        const int kpart = kk < kend ? (k * C * RS + rs) * 4 : SENT;
#pragma unroll
        for (int i = 0; i < T / 16; i++) r.s[i] = buf_load(st.rsrc, st.crow[i] + kpart, 0);
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 16; i++) lds[((tid >> 4) + 16 * i) * RED_STRIDE + (tid & 15)] = r.s[i];
    }
};

// (n, pq) of a reduction index that advances by KB per slice. Branch-free for any plane size (a plane may
// be smaller than a slice): the quotient comes from a multiply-high, so the tile loop stays one basic block.
struct PixelCursor {
    int n, pq;
    __device__ __forceinline__ void init(int kk, int PQ, int n_first) { n = kk / PQ; pq = kk - n * PQ; n -= n_first; }
    __device__ __forceinline__ void advance(int PQ, FastDiv divPQ) {
        pq += KB;
        const int q = divPQ.div(pq);
        n += q;
        pq -= q * PQ;
    }
};

// ---- dy as the A operand of backward filter: A[k][(n,p,q)] = dy[n,k,p,q] -------------------------
// The descriptor starts at the first sample of the workgroup's reduction range. VEC4 (plane size a
// multiple of four): 128-bit chunks, thread t: chunk t%4 of rows t/4 + 64*i; else 32-bit elements.
template <bool VEC4, class E = float>
struct LoadDyRed {
    static constexpr bool RED_MAJOR = true;
    static constexpr int ES = ElemBytes<E>::V;
    const E* dy;
    int N, K, PQ;
    int kchunk, Ktot; // reduction indices per split and in total
    FastDiv divPQ;
    template <int T> struct Regs { floatx4 v[T / 64]; float s[VEC4 ? 1 : T / 16]; };
    template <int T> struct State { int mrow[VEC4 ? T / 64 : T / 16]; PixelCursor cur; int kk; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int k_begin) const {
        // the descriptor covers the samples of this split's range only (below MAX_SUM_RANGE, host-checked)
        const int n_first = k_begin / PQ;
        int k_last = k_begin + kchunk; if (k_last > Ktot) k_last = Ktot;
        const int n_last = k_last > k_begin ? (k_last - 1) / PQ : n_first;
        st.rsrc = make_rsrc(dy + (long)n_first * K * PQ, clamp_range((long)(n_last - n_first + 1) * K * PQ * ES));
        st.kk = k_begin + (VEC4 ? 4 * (tid & 3) : (tid & 15));
        st.cur.init(st.kk, PQ, n_first);
        if (VEC4) {
#pragma unroll
            for (int i = 0; i < T / 64; i++) { const int m = row0 + (tid >> 2) + 64 * i; st.mrow[i] = m < K ? m * PQ * ES : SENT; }
        } else {
#pragma unroll
            for (int i = 0; i < T / 16; i++) { const int m = row0 + (tid >> 4) + 16 * i; st.mrow[i] = m < K ? m * PQ * ES : SENT; }
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int kend, int, Regs<T>& r) const {
        // the marker is OR-ed in (offsets stay below SENT) so that nothing here tempts the compiler into a branch
        const int npart = ((st.cur.n * K * PQ + st.cur.pq) * ES) | (st.kk < kend ? 0 : SENT);
        if (VEC4) {
#pragma unroll
            for (int i = 0; i < T / 64; i++) r.v[i] = buf_load4_e<E>(st.rsrc, st.mrow[i] + npart, 0);
        } else {
#pragma unroll
            for (int i = 0; i < T / 16; i++) r.s[i] = buf_load_e<E>(st.rsrc, st.mrow[i] + npart, 0);
        }
        st.kk += KB;
        st.cur.advance(PQ, divPQ);
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
        if (VEC4) {
#pragma unroll
            for (int i = 0; i < T / 64; i++) *(floatx4*)(lds + ((tid >> 2) + 64 * i) * RED_STRIDE + 4 * (tid & 3)) = r.v[i];
        } else {
#pragma unroll
            for (int i = 0; i < T / 16; i++) lds[((tid >> 4) + 16 * i) * RED_STRIDE + (tid & 15)] = r.s[i];
        }
    }
};

// The same operand with 128-bit chunks and a byte offset that is carried from slice to slice with adds and
// selects (no integer multiply in the loop). Needs P*Q >= KB (at most one sample wrap per step), P*Q a
// multiple of four and 16-byte aligned planes.
template <class E = float>
struct LoadDyRedInc {
    static constexpr bool RED_MAJOR = true;
    static constexpr int ES = ElemBytes<E>::V;
    const E* dy;
    int N, K, PQ;
    int kchunk, Ktot;
    template <int T> struct Regs { floatx4 v[T / 64]; };
    // Pixels past the end of the reduction lie in the sample after the descriptor's range and read as zero.
    template <int T> struct State { int mrow[T / 64]; int pq, off; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int k_begin) const {
        const int n_first = k_begin / PQ;
        int k_last = k_begin + kchunk; if (k_last > Ktot) k_last = Ktot;
        const int n_last = k_last > k_begin ? (k_last - 1) / PQ : n_first;
        st.rsrc = make_rsrc(dy + (long)n_first * K * PQ, clamp_range((long)(n_last - n_first + 1) * K * PQ * ES));
        const int kk = k_begin + 4 * (tid & 3);
        const int n = kk / PQ;
        st.pq = kk - n * PQ;
        st.off = (int)(((long)(n - n_first) * K * PQ + st.pq) * ES);
#pragma unroll
        for (int i = 0; i < T / 64; i++) { const int m = row0 + (tid >> 2) + 64 * i; st.mrow[i] = m < K ? m * PQ * ES : SENT; }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int, int, Regs<T>& r) const {
#pragma unroll
        for (int i = 0; i < T / 64; i++) r.v[i] = buf_load4_e<E>(st.rsrc, st.mrow[i] + st.off, 0);
        st.pq += KB;
        const bool wrap = st.pq >= PQ;
        st.pq -= wrap ? PQ : 0;
        st.off += wrap ? (KB + (K - 1) * PQ) * ES : KB * ES;
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 64; i++) *(floatx4*)(lds + ((tid >> 2) + 64 * i) * RED_STRIDE + 4 * (tid & 3)) = r.v[i];
    }
};

// ---- im2col operand of backward filter: B[(n,p,q)][(c,r,s)] = x[n,c,p*sh-ph+r,q*sw-pw+s] ---------
// reduction-major: thread t owns pixel t%16 of the slice and columns t/16 + 16*i. Per slice it
// derives the pixel's offset and its mask of out-of-image taps once; each column adds a constant.
template <bool BIGWIN, class E = float>
struct LoadIm2colRed {
    static constexpr bool RED_MAJOR = true;
    static constexpr int ES = ElemBytes<E>::V;
    const E* x;
    int N, C, H, W, R, S, P, Q, ph, pw, sh, sw;
    int ncols; // C*R*S
    int kchunk, Ktot; // reduction indices per split and in total
    FastDiv divRS, divS, divQ, divPQ;
    template <int T> struct Regs { float s[T / 16]; };
    template <int T> struct State {
        int jconst[T / 16]; // byte offset of (c*H*W + r*W + s), or SENT for a column outside the matrix
        int tap[T / 16];    // r*S + s (BIGWIN: r << 8 | s)
        PixelCursor cur; int kk;
        __amdgpu_buffer_rsrc_t rsrc;
    };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int, int k_begin) const {
        const int PQ = P * Q, RS = R * S;
        const int n_first = k_begin / PQ;
        const long chw = (long)C * H * W;
        const long shift = -((long)ph * W + pw);
        int k_last = k_begin + kchunk; if (k_last > Ktot) k_last = Ktot;
        const int n_last = k_last > k_begin ? (k_last - 1) / PQ : n_first;
        st.rsrc = make_rsrc(x + (long)n_first * chw + shift, clamp_range(((long)(n_last - n_first + 1) * chw - shift) * ES));
        st.kk = k_begin + (tid & 15);
        st.cur.init(st.kk, PQ, n_first);
#pragma unroll
        for (int i = 0; i < T / 16; i++) {
            const int j = j0 + (tid >> 4) + 16 * i;
            if (j < ncols) {
                const int c = divRS.div(j), rs = j - c * RS;
                const int r = divS.div(rs), s = rs - r * S;
                st.jconst[i] = (c * H * W + r * W + s) * ES;
                st.tap[i] = BIGWIN ? ((r << 8) | s) : rs;
            } else {
                st.jconst[i] = SENT;
                st.tap[i] = 0;
            }
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int kend, int, Regs<T>& r) const {
        const int PQ = P * Q;
        const int p = divQ.div(st.cur.pq), q = st.cur.pq - p * Q;
        const int ih0 = p * sh - ph, iw0 = q * sw - pw;
        const int pixbase = ((st.cur.n * C * H * W + p * sh * W + q * sw) * ES) | (st.kk < kend ? 0 : SENT);
        const unsigned vrow = valid_window_bits(ih0, R, H), vcol = valid_window_bits(iw0, S, W);
        if (BIGWIN) {
            const unsigned invrow = ~vrow, invcol = ~vcol;
#pragma unroll
            for (int i = 0; i < T / 16; i++) {
                const int dead = bit_to_all_ones(invrow, st.tap[i] >> 8) | bit_to_all_ones(invcol, st.tap[i] & 255);
                r.s[i] = buf_load_e<E>(st.rsrc, (pixbase + st.jconst[i]) | dead, 0);
            }
        } else {
            unsigned v = 0;
            for (int tr = 0; tr < R; tr++) v |= ((vrow >> tr) & 1u) ? (vcol << (tr * S)) : 0u;
            const unsigned inv = ~v;
#pragma unroll
            for (int i = 0; i < T / 16; i++)
                r.s[i] = buf_load_e<E>(st.rsrc, (pixbase + st.jconst[i]) | bit_to_all_ones(inv, st.tap[i]), 0);
        }
        st.kk += KB;
        st.cur.advance(PQ, divPQ);
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 16; i++) lds[((tid >> 4) + 16 * i) * RED_STRIDE + (tid & 15)] = r.s[i];
    }
};

// ---- result of forward / backward data: out[n][m][pix] = acc (+ bias[m]) --------------------------
template <class E = float>
struct StoreNCHW {
    E* out;
    const float* bias; // optional, per output channel
    int opix;          // pixels of one output plane
    float* partial;    // split reductions: split ks writes its sums to partial[ks][same index], bias added by the reduction
    int relu;          // rectify the result (after the bias)
    const E* gate;     // optional, same layout as out: the result is kept where gate > 0 and zero elsewhere
    static constexpr bool TAIL = true;
    // tail mode: a split tile's sums go to partial[slot][row in tile][column in tile], slot = (tile, split)
    __device__ __forceinline__ void store_tail(const floatx16 (&acc)[2][2], int wm0, int wn0, int lane, long slot, int TM, int TN) const {
        const int l32 = lane & 31, lk = lane >> 5;
        float* po = partial + slot * TM * TN;
#pragma unroll
        for (int jt = 0; jt < 2; jt++)
#pragma unroll
            for (int it = 0; it < 2; it++)
#pragma unroll
                for (int v = 0; v < 16; v++)
                    po[(wm0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4)) * TN + wn0 + jt * 32 + l32] = acc[it][jt][v];
    }
    __device__ __forceinline__ void store(const floatx16 (&acc)[2][2], int m0, int j0, int lane, int ks, const GemmDims& d, bool to_partial) const {
        const int l32 = lane & 31, lk = lane >> 5;
        // Bias and gate values are read before the stores they feed, eight at a time: a load that follows a store
        // through a pointer it might share has to be issued behind it, and with the load's result needed for the next
        // store that is one round trip to memory per element. Eight, not the whole tile: the registers they wait in
        // count against the three workgroups a compute unit holds. (A gate that *is* the output tensor - the gradient
        // written over the layer's own input - is read by the lane that overwrites it, before it does.)
#pragma unroll
        for (int jt = 0; jt < 2; jt++) {
            const int j = j0 + jt * 32 + l32;
            if (j >= d.N) continue;
            const int n = j / opix, pix = j - n * opix;
            const size_t base = (size_t)n * d.M * opix + pix;
            E* o = out + base;
            float* po = partial + (size_t)ks * d.M * d.N + base;
#pragma unroll
            for (int it = 0; it < 2; it++)
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    float bv[8], gt[8];
                    if (!to_partial && bias) {
#pragma unroll
                        for (int u = 0; u < 8; u++) {
                            const int v = 8 * h + u, m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                            bv[u] = m < d.M ? bias[m] : 0.0f;
                        }
                    }
                    if (!to_partial && gate) {
#pragma unroll
                        for (int u = 0; u < 8; u++) {
                            const int v = 8 * h + u, m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                            gt[u] = m < d.M ? load_elem(gate + base + (size_t)m * opix) : 1.0f;
                        }
                    }
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        const int v = 8 * h + u, m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                        if (m >= d.M) continue;
                        float r = acc[it][jt][v];
                        if (to_partial) {
                            po[(size_t)m * opix] = r;
                        } else {
                            if (bias) r += bv[u];
                            if (relu) r = relu_value(r);
                            if (gate) r = gt[u] > 0.0f ? r : 0.0f;
                            store_elem(o + (size_t)m * opix, r);
                        }
                    }
                }
        }
    }
};

} // namespace vdnn
