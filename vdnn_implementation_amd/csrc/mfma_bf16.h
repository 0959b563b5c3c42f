// Tile engine on the bfloat16 matrix cores (v_mfma_f32_32x32x16_bf16: 16x the multiply rate of the float
// instruction). Used when activations are stored as bfloat16: products of two bfloat16 values are exact in
// float and the accumulators are float, so against the float engine on the same (bfloat16-valued) operands
// only the order of summation differs. The filter operand is the float master copy rounded to bfloat16
// (nearest even) by the packing kernel below.
//
// Same tiling as the float engine (256 threads, four 64x64 wave tiles, two LDS buffers) with 32-deep slices.
// Both operands sit in LDS reduction-major, 32 values (64 bytes) + 16 bytes of padding per row, so that the
// 128-bit store of eight consecutive reduction values by eight consecutive lanes and the 128-bit fragment
// read of a 32-row block are both free of bank conflicts. The instruction takes eight reduction values per
// lane for both operands, so any order of the reduction inside a slice works as long as both sides agree.
#pragma once
#include "conv_loaders.h"

namespace vdnn {

constexpr int KH = 32;      // reduction depth of one slice
constexpr int HSTRIDE = 40; // LDS row stride in 16-bit units
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

// Filter bank of a float layer split into bfloat16 parts, for the kernels that multiply float layers on the bfloat16
// matrix cores (conv3x3_bf16.h, LoadIm2colPixTapS below): 16-channel blocks, tap-major,
// packed[row][((cb*RS + tap)*2 + part)*16 + l] = part of w[row*row_stride + (cb*16 + l)*red_stride + tap], part 0 = hi, 1 = lo
// (row_stride / red_stride as in pack_filter_tap_bf16_kernel). One thread per filter element.
static __global__ void __launch_bounds__(256) pack_filter_split_kernel(const float* __restrict__ w, unsigned short* __restrict__ packed,
                                                                int rows, int Cred, int RS, int row_stride, int red_stride, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int per_row = Cred * RS;
    const int row = (int)(i / per_row), kk = (int)(i - (long)row * per_row);
    const int l = kk & 15, slice = kk >> 4;
    const int cb = slice / RS, tap = slice - cb * RS;
    const float v = w[(long)row * row_stride + (long)(cb * 16 + l) * red_stride + tap];
    const unsigned short hi = float_to_bf16_bits(v);
    const unsigned short lo = float_to_bf16_bits(v - __builtin_bit_cast(float, (unsigned)hi << 16));
    unsigned short* at = packed + (long)row * per_row * 2 + (long)slice * 32 + l;
    at[0] = hi; at[16] = lo;
}

typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
// (hi, lo) parts of two floats, each pair packed into one word (first value in the low half)
__device__ __forceinline__ void split_pair(float a, float b, unsigned& hi, unsigned& lo) {
    hi = __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{a, b}, bf16x2));
    const float ha = __builtin_bit_cast(float, hi << 16), hb = __builtin_bit_cast(float, hi & 0xFFFF0000u);
    lo = __builtin_bit_cast(unsigned, __builtin_convertvector(floatx2{a - ha, b - hb}, bf16x2));
}

// LDS takes a 128-bit store eight lanes at a time, on 32 banks of four bytes (measured: 8 cycles per store when the
// eight lanes' 32 words fall on 32 different banks, 16 otherwise). With rows of HSTRIDE = 40 halfwords (20 words)
// four lanes per 64-byte row and two consecutive rows per eight lanes meet on four banks (20 + 12 = 32 = 0); rows
// r and r + 4 (80 words = 16 mod 32) tile the banks. So the four lanes t%4 of a row take the rows in the order
// 0 4 1 5 2 6 3 7 of every eight: which thread fetches which row is free.
__device__ __forceinline__ int rows_by_four_lanes(int tid) {
    const int b = tid >> 2;
    return (b & ~7) | ((b & 1) << 2) | ((b >> 1) & 3);
}
// The same for two lanes per row (a 16-byte piece each, rows of 20 words): rows 0 2 4 6 1 3 5 7 of every eight.
__device__ __forceinline__ int rows_by_two_lanes(int tid) {
    const int b = tid >> 1;
    return (b & ~7) | ((b & 3) << 1) | ((b >> 2) & 1);
}

// ---- dense bfloat16 reduction-major operand: element (row, kk) at base[row*ld + kk] --------------------
// thread t: values 8*(t%4) .. +7 of rows rows_by_four_lanes(t) + 64*i, one 128-bit load each
struct LoadPackedH {
    const unsigned short* base;
    long ld;        // elements between rows (a multiple of 8)
    int rows;
    unsigned bytes; // below 2 GiB
    template <int T> struct Regs { uintx4 v[T / 64]; };
    template <int T> struct State { int vrow[T / 64]; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(base, bytes);
#pragma unroll
        for (int i = 0; i < T / 64; i++) {
            const int row = row0 + rows_by_four_lanes(tid) + 64 * i;
            st.vrow[i] = row < rows ? (int)(((long)row * ld + 8 * (tid & 3)) * 2) : OOB;
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int, int, Regs<T>& r) const {
        const int soff = kk0 * 2;
#pragma unroll
        for (int i = 0; i < T / 64; i++) r.v[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(st.rsrc, st.vrow[i], soff, 0));
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 64; i++) *(uintx4*)(lds + (rows_by_four_lanes(tid) + 64 * i) * HSTRIDE + 8 * (tid & 3)) = r.v[i];
    }
};

// ---- im2col operand, columns = output pixels, blocked tap-major reduction (32 channels per tap) ------
// MODE 0: forward gather from x; MODE 1: backward data at stride 1 (src = dy). A lane owns one pixel
// (consecutive lanes, consecutive pixels: every 16-bit load of a wavefront covers one run of a plane) and
// fetches eight consecutive channels of it per item, packed into one 128-bit LDS store.
template <int MODE>
struct LoadIm2colPixTapH {
    LoadIm2colPix<MODE, false, bf16_t> base; // geometry and per-pixel state of the float engine's loader
    template <int T> struct Regs { uintx4 v[T / 64]; };
    template <int T> using State = typename LoadIm2colPix<MODE, false, bf16_t>::template State<T>;
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int ncols, int k_begin) const {
        base.template init<T>(st, j0, tid, ncols, k_begin);
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int, int tid, Regs<T>& r) const {
        const int plane = base.Hs * base.Ws;
        const int slice = kk0 / KH;
        const int cb = base.divRS.div(slice), tap = slice - cb * (base.R * base.S);
        const int tr = base.divS.div(tap), ts = tap - tr * base.S;
        const int tapoff = MODE == 0 ? tr * base.Ws + ts : (base.R - 1 - tr) * base.Ws + (base.S - 1 - ts);
        const int voff = st.vbase | bit_to_all_ones(st.inv, tap);
        const int g0 = __builtin_amdgcn_readfirstlane(tid / T);
#pragma unroll
        for (int i = 0; i < T / 64; i++) {
            const int ch = cb * KH + 8 * (g0 + (NT / T) * i);
            const int soff = (ch * plane + tapoff) * 2, step = plane * 2;
            unsigned h[8];
#pragma unroll
            for (int e = 0; e < 8; e++) h[e] = (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(st.rsrc, voff, soff + e * step, 0);
            r.v[i].x = h[0] | (h[1] << 16); r.v[i].y = h[2] | (h[3] << 16);
            r.v[i].z = h[4] | (h[5] << 16); r.v[i].w = h[6] | (h[7] << 16);
        }
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 64; i++) *(uintx4*)(lds + (tid % T) * HSTRIDE + 8 * (tid / T + (NT / T) * i)) = r.v[i];
    }
};

// The same operand of a float layer for the perf-optimal mode's products of bfloat16 parts (conv3x3_bf16.h): a slice is
// one tap x 16 channels, an LDS row holds [hi of the 16 channels | lo of the 16 channels]. A lane owns one pixel and
// fetches eight consecutive channels of it per item as floats, splits them (hi = bf16(v), lo = bf16(v - hi)) and
// writes two 128-bit LDS pieces. kk0 counts the 16-bit values of a row of the filter operand (32 per slice).
template <int MODE>
struct LoadIm2colPixTapS {
    LoadIm2colPix<MODE, false, float> base; // geometry and per-pixel state of the float engine's loader
    static constexpr int ITEMS(int T) { return 2 * T / NT > 0 ? 2 * T / NT : 1; } // two channel groups per pixel
    template <int T> struct Regs { float v[2 * T / NT > 0 ? 2 * T / NT : 1][8]; };
    template <int T> using State = typename LoadIm2colPix<MODE, false, float>::template State<T>;
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int ncols, int k_begin) const {
        base.template init<T>(st, j0, tid, ncols, k_begin);
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int, int tid, Regs<T>& r) const {
        static_assert(T == 128 || T == 256, "one or two items per thread");
        const int plane = base.Hs * base.Ws;
        const int slice = kk0 / KH;
        const int cb = base.divRS.div(slice), tap = slice - cb * (base.R * base.S);
        const int tr = base.divS.div(tap), ts = tap - tr * base.S;
        const int tapoff = MODE == 0 ? tr * base.Ws + ts : (base.R - 1 - tr) * base.Ws + (base.S - 1 - ts);
        const int voff = st.vbase | bit_to_all_ones(st.inv, tap);
        const int g0 = __builtin_amdgcn_readfirstlane(tid / T);
#pragma unroll
        for (int i = 0; i < ITEMS(T); i++) {
            const int ch = cb * 16 + 8 * (g0 + (NT / T) * i);
            const int soff = (ch * plane + tapoff) * 4, step = plane * 4;
#pragma unroll
            for (int e = 0; e < 8; e++) r.v[i][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(st.rsrc, voff, soff + e * step, 0));
        }
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < ITEMS(T); i++) {
            uintx4 hi, lo;
            unsigned h[4], l[4];
#pragma unroll
            for (int k = 0; k < 4; k++) split_pair(r.v[i][2 * k], r.v[i][2 * k + 1], h[k], l[k]);
            hi.x = h[0]; hi.y = h[1]; hi.z = h[2]; hi.w = h[3];
            lo.x = l[0]; lo.y = l[1]; lo.z = l[2]; lo.w = l[3];
            unsigned short* at = lds + (tid % T) * HSTRIDE + 8 * (tid / T + (NT / T) * i);
            *(uintx4*)at = hi;
            *(uintx4*)(at + 16) = lo;
        }
    }
};
// Operands whose slices are [hi | lo] parts: the engine multiplies hi x hi + hi x lo + lo x hi instead of the two halves.
template <class BL> struct SplitProducts { static constexpr bool V = false; };
template <int MODE> struct SplitProducts<LoadIm2colPixTapS<MODE>> { static constexpr bool V = true; };

// Filter bank rounded to bfloat16 and re-laid-out for the blocked tap-major order:
// packed[row][(cb*RS + tap)*32 + l] = bf16(w[row*row_stride + (cb*32 + l)*red_stride + tap])
//   forward:       rows = output channels, reduced channels = input channels:  row_stride = C*RS, red_stride = RS
//   backward data: rows = input channels,  reduced channels = output channels: row_stride = RS,   red_stride = C*RS
static __global__ void __launch_bounds__(256) pack_filter_tap_bf16_kernel(const float* __restrict__ w, unsigned short* __restrict__ packed,
                                                                   int rows, int Cred, int RS, int row_stride, int red_stride, long total) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int per_row = Cred * RS;
    const int row = (int)(i / per_row), kk = (int)(i - (long)row * per_row);
    const int l = kk & 31, slice = kk >> 5;
    const int cb = slice / RS, tap = slice - cb * RS;
    packed[i] = float_to_bf16_bits(w[(long)row * row_stride + (long)(cb * 32 + l) * red_stride + tap]);
}

// Order of the tiles over the workgroup index: rows fastest unless the epilogue type says otherwise.
template <class EP> struct TileOrder { static constexpr bool COLUMNS_FASTEST = false; };

// Out tile = A tile x B tile over this workgroup's share of the reduction; tile decoding and epilogues are
// those of the float engine (igemm_kernel), slices are KH deep.
// How many workgroups a compute unit is to hold at least (the register budget follows): three with the
// convolution operands, which the compiler meets without spills; an operand type that needs more registers says so.
template <class AL, class BL> struct MinResident { static constexpr int V = 3; };

template <int TM, int TN, class AL, class BL, class EP>
__global__ void __launch_bounds__(NT, (MinResident<AL, BL>::V)) igemm_bf16_kernel(const AL al, const BL bl, const EP ep, const GemmDims d) {
    static_assert(TM % 64 == 0 && TN % 64 == 0 && (TM / 64) * (TN / 64) == 4, "four 64x64 wave tiles");
    __shared__ __attribute__((aligned(16))) unsigned short As[2][TM * HSTRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short Bs[2][TN * HSTRIDE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int ntiles_all = d.mtiles * d.ntiles;
    int tile, ks;
    bool whole;
    if ((int)blockIdx.x < d.full_tiles) {
        tile = xcd_remap(blockIdx.x, d.full_tiles); ks = 0; whole = true;
    } else if (d.full_tiles > 0) {
        const int r = blockIdx.x - d.full_tiles, tl = ntiles_all - d.full_tiles;
        tile = d.full_tiles + r % tl; ks = r / tl; whole = false;
    } else {
        const int bid = xcd_remap(blockIdx.x, gridDim.x);
        tile = bid % ntiles_all; ks = bid / ntiles_all; whole = d.splits == 1;
    }
    // the column tile runs fastest for epilogues that ask for it (workgroups at work together then write one run of rows)
    const int mt = TileOrder<EP>::COLUMNS_FASTEST ? tile / d.ntiles : tile % d.mtiles;
    const int nt = TileOrder<EP>::COLUMNS_FASTEST ? tile % d.ntiles : tile / d.mtiles;
    const int m0 = mt * TM, j0 = nt * TN;
    const int k_begin = whole ? 0 : ks * d.kchunk;
    const int k_end = whole ? d.K : min(d.K, k_begin + d.kchunk);

    typename AL::template State<TM> sa;
    typename BL::template State<TN> sb;
    al.template init<TM>(sa, m0, tid, d.M, k_begin);
    bl.template init<TN>(sb, j0, tid, d.N, k_begin);

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int wm0 = (wave % (TM / 64)) * 64, wn0 = (wave / (TM / 64)) * 64;
    const int l32 = lane & 31, lk = lane >> 5;
    typename AL::template Regs<TM> ra;
    typename BL::template Regs<TN> rb;

    // slice s is multiplied from LDS buffer s%2 while slice s+1 (fetched during slice s-1) is written to the
    // other buffer and slice s+2 is fetched; one barrier per slice. Fetches past the end of the range are
    // never used (buffer loads cannot fault).
    const int nslices = (k_end - k_begin + KH - 1) / KH;
    al.template load<TM>(sa, k_begin, k_end, tid, ra);
    bl.template load<TN>(sb, k_begin, k_end, tid, rb);
    AL::template store<TM>(As[0], tid, ra);
    BL::template store<TN>(Bs[0], tid, rb);
    al.template load<TM>(sa, k_begin + KH, k_end, tid, ra);
    bl.template load<TN>(sb, k_begin + KH, k_end, tid, rb);
    __syncthreads();
    for (int s = 0; s < nslices; s++) {
        const int cur = s & 1, nxt = cur ^ 1;
        const unsigned short* ap = As[cur] + (wm0 + l32) * HSTRIDE + 8 * lk;
        const unsigned short* bp = Bs[cur] + (wn0 + l32) * HSTRIDE + 8 * lk;
        bf16x8 a[2][2], b[2][2];
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                a[h][i] = *(const bf16x8*)(ap + i * 32 * HSTRIDE + 16 * h);
                b[h][i] = *(const bf16x8*)(bp + i * 32 * HSTRIDE + 16 * h);
            }
        if constexpr (SplitProducts<BL>::V) {
#pragma unroll
            for (int p = 0; p < 3; p++)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[p == 2][i], b[p == 1][j], acc[i][j], 0, 0, 0);
        } else {
#pragma unroll
            for (int h = 0; h < 2; h++)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[h][i], b[h][j], acc[i][j], 0, 0, 0);
        }
        AL::template store<TM>(As[nxt], tid, ra);
        BL::template store<TN>(Bs[nxt], tid, rb);
        __syncthreads();
        const int kk0 = k_begin + (s + 2) * KH;
        al.template load<TM>(sa, kk0, k_end, tid, ra);
        bl.template load<TN>(sb, kk0, k_end, tid, rb);
    }

    if (EP::TAIL && d.full_tiles > 0 && !whole)
        ep.store_tail(acc, wm0, wn0, lane, (long)(tile - d.full_tiles) * d.splits + ks, TM, TN);
    else
        ep.store(acc, m0 + wm0, j0 + wn0, lane, ks, d, !whole);
}

} // namespace vdnn

namespace vdnn {

typedef unsigned uintx2 __attribute__((ext_vector_type(2)));

// ---- backward filter on the bfloat16 matrix cores: the reduction runs over output pixels (n, p, q) ----
// dy as A[k][(n,p,q)]: thread t fetches pixels 4*(t%8) .. +3 (64 bits) of rows t/8 + 32*i. The byte offset is
// carried from slice to slice with adds and selects (P*Q >= 32: at most one sample wrap per step; P*Q a
// multiple of four). Pixels past the end of the reduction lie beyond the descriptor's range: zero.
struct LoadDyRedIncH {
    const bf16_t* dy;
    int N, K, PQ;
    int kchunk, Ktot;
    template <int T> struct Regs { uintx2 v[T / 32]; };
    template <int T> struct State { int mrow[T / 32]; int pq, off; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int k_begin) const {
        const int n_first = k_begin / PQ;
        int k_last = k_begin + kchunk; if (k_last > Ktot) k_last = Ktot;
        const int n_last = k_last > k_begin ? (k_last - 1) / PQ : n_first;
        st.rsrc = make_rsrc(dy + (long)n_first * K * PQ, clamp_range((long)(n_last - n_first + 1) * K * PQ * 2));
        const int kk = k_begin + 4 * (tid & 7);
        const int n = kk / PQ;
        st.pq = kk - n * PQ;
        st.off = (int)(((long)(n - n_first) * K * PQ + st.pq) * 2);
#pragma unroll
        for (int i = 0; i < T / 32; i++) { const int m = row0 + (tid >> 3) + 32 * i; st.mrow[i] = m < K ? m * PQ * 2 : SENT; }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int, int, Regs<T>& r) const {
#pragma unroll
        for (int i = 0; i < T / 32; i++) r.v[i] = __builtin_bit_cast(uintx2, __builtin_amdgcn_raw_buffer_load_b64(st.rsrc, st.mrow[i] + st.off, 0, 0));
        st.pq += KH;
        const bool wrap = st.pq >= PQ;
        st.pq -= wrap ? PQ : 0;
        st.off += wrap ? (KH + (K - 1) * PQ) * 2 : KH * 2;
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 32; i++) *(uintx2*)(lds + ((tid >> 3) + 32 * i) * HSTRIDE + 4 * (tid & 7)) = r.v[i];
    }
};

// im2col operand in tap-major column order (as LoadIm2colRedTap): B[(tap, c)][(n,p,q)]. Thread t owns the
// pixel pair 2*(t%16), +1 of the slice (both in one output row: Q is even) and the columns t/16 + 16*i; the two
// 16-bit values of a column are packed into one LDS word. The pair's input row / column / byte offset are
// carried from slice to slice (Q >= 11: at most three row wraps per 32 pixels; P*Q >= 32: one sample wrap).
template <int NTAP, bool PAIR32 = false>
struct LoadIm2colRedTapH {
    const bf16_t* x;
    int N, C, H, W, R, S, P, Q, ph, pw, sh, sw;
    int ncols; // C*R*S
    int kchunk, Ktot;
    FastDiv divC, divS;
    template <int T> struct Regs { unsigned s[T / 16]; };
    template <int T> struct State {
        int ih, iw;   // input row / column of the pair's first pixel through the first group's tap
        int off;      // byte offset of that element in the thread's first channel plane
        int dih[NTAP], diw[NTAP], doff[NTAP];
        int iw_wrap, ih_wrap;
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
        // the descriptor's base is kept four-byte aligned (x is): the 32-bit pair loads rely on it
        const long base_e = (long)n_first * chw + shift;
        const int odd = (int)(base_e & 1);
        st.rsrc = make_rsrc(x + base_e - odd, clamp_range(((long)(n_last - n_first + 1) * chw - shift + odd) * 2));
        const int kk = k_begin + 2 * (tid & 15);
        const int n = kk / PQ, pq = kk - n * PQ;
        const int p = pq / Q, q = pq - p * Q;
        int r0 = 0, s0 = 0, c0 = 0;
#pragma unroll
        for (int g = 0; g < NTAP; g++) {
            const int jg = j0 + g * (T / NTAP);
            const int tap = divC.div(jg);
            const int r = divS.div(tap), s_ = tap - r * S;
            const int c = jg - tap * C;
            if (g == 0) { r0 = r; s0 = s_; c0 = c; st.dih[0] = 0; st.diw[0] = 0; st.doff[0] = 0; }
            else {
                st.dih[g] = jg < ncols ? r - r0 : 0x20000000;
                st.diw[g] = s_ - s0;
                st.doff[g] = (((r - r0) * W + (s_ - s0)) + (c - c0) * H * W) * 2;
            }
        }
        st.ih = p * sh - ph + r0; st.iw = q * sw - pw + s0;
        st.iw_wrap = Q * sw - pw + s0; st.ih_wrap = P * sh - ph + r0;
        st.off = (int)(((long)(n - n_first) * chw + (long)(c0 + (tid >> 4)) * H * W + (long)(p * sh + r0) * W + q * sw + s0 + odd) * 2);
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int, int, Regs<T>& r) const {
        int base0[NTAP], base1[NTAP];
        unsigned keep[NTAP]; // PAIR32: which halves of the loaded word lie inside the image
        int down[NTAP];      // PAIR32: 16 when the word was fetched one element lower
#pragma unroll
        for (int g = 0; g < NTAP; g++) {
            const int ih = g == 0 ? st.ih : st.ih + st.dih[g], iw = g == 0 ? st.iw : st.iw + st.diw[g];
            const int o = g == 0 ? st.off : st.off + st.doff[g];
            const bool row_ok = (unsigned)ih < (unsigned)H;
            const bool ok0 = (unsigned)iw < (unsigned)W, ok1 = (unsigned)(iw + sw) < (unsigned)W;
            if (PAIR32) {
                // A pair whose second pixel reads past the right edge is fetched one element lower and shifted
                // down afterwards: its first element may be the last one of the descriptor's range, and a
                // 32-bit load that crosses the end of the range returns zero.
                base0[g] = (ok1 ? o : o - 2) | (row_ok ? 0 : SENT);
                base1[g] = 0;
                down[g] = ok1 ? 0 : 16;
                keep[g] = (ok0 ? 0x0000FFFFu : 0u) | (ok1 ? 0xFFFF0000u : 0u);
            } else {
                base0[g] = o | ((row_ok & ok0) ? 0 : SENT);
                base1[g] = (o + sw * 2) | ((row_ok & ok1) ? 0 : SENT);
                keep[g] = 0; down[g] = 0;
            }
        }
        constexpr int PERG = T / 16 / NTAP;
        const int plane16 = 16 * H * W * 2;
#pragma unroll
        for (int i = 0; i < T / 16; i++) {
            if (PAIR32) {
                // the pair is two neighbouring elements of an input row: one load (two-byte alignment suffices)
                const unsigned word = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(st.rsrc, base0[i / PERG], (i % PERG) * plane16, 0);
                r.s[i] = __builtin_amdgcn_alignbit(0u, word, (unsigned)down[i / PERG]) & keep[i / PERG];
            } else {
                const unsigned lo = (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(st.rsrc, base0[i / PERG], (i % PERG) * plane16, 0);
                const unsigned hi = (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(st.rsrc, base1[i / PERG], (i % PERG) * plane16, 0);
                r.s[i] = lo | (hi << 16);
            }
        }
        // next slice: KH pixels further
        st.iw += KH * sw; st.off += KH * sw * 2;
        const int qsw = Q * sw;
        const int wraps = (st.iw >= st.iw_wrap ? 1 : 0) + (st.iw >= st.iw_wrap + qsw ? 1 : 0) + (st.iw >= st.iw_wrap + 2 * qsw ? 1 : 0);
        st.iw -= __mul24(wraps, qsw);
        st.ih += __mul24(wraps, sh);
        st.off += __mul24(wraps, (sh * W - qsw) * 2);
        const bool next = st.ih >= st.ih_wrap;
        st.ih -= next ? P * sh : 0;
        st.off += next ? (C * H * W - P * sh * W) * 2 : 0;
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 16; i++) *(unsigned*)(lds + ((tid >> 4) + 16 * i) * HSTRIDE + 2 * (tid & 15)) = r.s[i];
    }
};

// ---- backward filter of 3x3 / stride 1 / padding 1 layers: vector loads along the reduction -------------
// Through tap (r, s) output pixel j of a sample reads element j + (r-1)*W + (s-1) of an input plane: one tap's
// im2col operand is the plane shifted by a constant, and so are G consecutive pixels as long as they share an
// image row (G divides W) - one G-element load per (column, pixel group), at two-byte alignment for the outer
// filter columns (buffer loads take it; a double word that would cross the end of the descriptor's range
// reads as zero, so no load here may do that). A group in an image row outside the input is not fetched. The
// one element per row that reads the padding left or right of the image belongs to the row's first / last
// group: that group is fetched through the centre tap's position, moved one element up / down in registers,
// and zero enters at the free end - so no load reaches below the first or past the last element of a plane.
// G = 8 (128-bit loads) or 4 (64-bit); dy, the other operand, comes in groups of GA pixels (GA divides P*Q:
// a group never leaves its sample).
template <int G> struct PixVec;
template <> struct PixVec<8> {
    typedef uintx4 type;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int voff) {
        return __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, 0, 0));
    }
    // element e of the result = element e+1 of v where `edge`, the last one zero
    static __device__ __forceinline__ type down(type v, bool edge) {
        const unsigned sh = edge ? 16u : 0u;
        type o;
        o.x = __builtin_amdgcn_alignbit(v.y, v.x, sh); o.y = __builtin_amdgcn_alignbit(v.z, v.y, sh);
        o.z = __builtin_amdgcn_alignbit(v.w, v.z, sh); o.w = __builtin_amdgcn_alignbit(0u, v.w, sh);
        return o;
    }
    // element e of the result = element e-1 of v where `edge`, the first one zero
    static __device__ __forceinline__ type up(type v, bool edge) {
        type o;
        o.w = edge ? __builtin_amdgcn_alignbit(v.w, v.z, 16u) : v.w; o.z = edge ? __builtin_amdgcn_alignbit(v.z, v.y, 16u) : v.z;
        o.y = edge ? __builtin_amdgcn_alignbit(v.y, v.x, 16u) : v.y; o.x = edge ? v.x << 16 : v.x;
        return o;
    }
};
template <> struct PixVec<4> {
    typedef uintx2 type;
    static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, int voff) {
        return __builtin_bit_cast(uintx2, __builtin_amdgcn_raw_buffer_load_b64(r, voff, 0, 0));
    }
    static __device__ __forceinline__ type down(type v, bool edge) {
        const unsigned sh = edge ? 16u : 0u;
        type o;
        o.x = __builtin_amdgcn_alignbit(v.y, v.x, sh); o.y = __builtin_amdgcn_alignbit(0u, v.y, sh);
        return o;
    }
    static __device__ __forceinline__ type up(type v, bool edge) {
        type o;
        o.y = edge ? __builtin_amdgcn_alignbit(v.y, v.x, 16u) : v.y; o.x = edge ? v.x << 16 : v.x;
        return o;
    }
};

// dy as A[k][(n,p,q)]: thread t fetches pixel group t % (32/GA) of rows t / (32/GA) + (8*GA)*i.
template <int GA>
struct LoadDyRedVecH {
    const bf16_t* dy;
    int N, K, PQ;
    int kchunk, Ktot;
    static constexpr int PG = KH / GA; // pixel groups of a slice
    static constexpr int RL = NT / PG; // rows one load instruction of the workgroup covers
    typedef typename PixVec<GA>::type V;
    template <int T> struct Regs { V v[T / RL]; };
    template <int T> struct State { int mrow[T / RL]; int pq, off; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int k_begin) const {
        const int n_first = k_begin / PQ;
        int k_last = k_begin + kchunk; if (k_last > Ktot) k_last = Ktot;
        const int n_last = k_last > k_begin ? (k_last - 1) / PQ : n_first;
        st.rsrc = make_rsrc(dy + (long)n_first * K * PQ, clamp_range((long)(n_last - n_first + 1) * K * PQ * 2));
        const int kk = k_begin + GA * (tid % PG);
        const int n = kk / PQ;
        st.pq = kk - n * PQ;
        st.off = (int)(((long)(n - n_first) * K * PQ + st.pq) * 2);
#pragma unroll
        for (int i = 0; i < T / RL; i++) { const int m = row0 + tid / PG + RL * i; st.mrow[i] = m < K ? m * PQ * 2 : SENT; }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int, int, Regs<T>& r) const {
#pragma unroll
        for (int i = 0; i < T / RL; i++) r.v[i] = PixVec<GA>::load(st.rsrc, st.mrow[i] + st.off);
        st.pq += KH;
        const bool wrap = st.pq >= PQ;
        st.pq -= wrap ? PQ : 0;
        st.off += wrap ? (KH + (K - 1) * PQ) * 2 : KH * 2;
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / RL; i++) *(V*)(lds + (tid / PG + RL * i) * HSTRIDE + GA * (tid % PG)) = r.v[i];
    }
};

// im2col operand in tap-major column order, B[(tap, c)][(n,p,q)]: thread t fetches pixel group t % (32/G) of the
// columns t / (32/G) + (8*G)*i. The columns of one load instruction share a tap (T/NTAP is a multiple of 8*G), so
// the tap's row and column are wave-uniform and select the code path.
template <int NTAP, int G>
struct LoadIm2colRedTapVecH {
    const bf16_t* x;
    int N, C, H, W;
    int ncols; // 9*C
    int kchunk, Ktot;
    FastDiv divC;
    static constexpr int PG = KH / G;
    static constexpr int CL = NT / PG; // columns one load instruction of the workgroup covers
    typedef typename PixVec<G>::type V;
    // as fetched; the move of a row's first / last group waits until the values are stored, so that a slice's
    // loads are all issued before any of them is waited for
    template <int T> struct Regs { V v[T / CL]; bool edge[T / CL]; int ts[T / CL]; };
    template <int T> struct State {
        int p0, q0; // output row / column of the group's first pixel
        int pos;    // byte offset of input element (p0, q0) of channel 0 in the group's sample, from the descriptor's base
        int coloff[T / CL]; // + the column's channel plane and its tap's shift; SENT past the last column
        int tr[T / CL], ts[T / CL]; // the load's filter row / column (wave-uniform)
        __amdgpu_buffer_rsrc_t rsrc;
    };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int, int k_begin) const {
        static_assert((T / NTAP) % CL == 0, "the columns of one load share a tap");
        const int PQ = H * W;
        const long chw = (long)C * PQ;
        const int n_first = k_begin / PQ;
        int k_last = k_begin + kchunk; if (k_last > Ktot) k_last = Ktot;
        const int n_last = k_last > k_begin ? (k_last - 1) / PQ : n_first;
        st.rsrc = make_rsrc(x + (long)n_first * chw, clamp_range((long)(n_last - n_first + 1) * chw * 2));
        const int kk = k_begin + G * (tid % PG);
        const int n = kk / PQ, pq = kk - n * PQ;
        st.p0 = pq / W; st.q0 = pq - st.p0 * W;
        st.pos = (int)(((long)(n - n_first) * chw + pq) * 2);
#pragma unroll
        for (int i = 0; i < T / CL; i++) {
            const int jl = j0 + CL * i;             // first column of this load: uniform
            const int tap = divC.div(jl);
            const int r = tap / 3, s_ = tap - 3 * r;
            const int c = jl - tap * C + tid / PG;
            const bool valid = jl < ncols;
            st.tr[i] = valid ? r : 1; st.ts[i] = valid ? s_ : 1;
            st.coloff[i] = valid ? (c * PQ + (r - 1) * W + (s_ - 1)) * 2 : SENT;
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int, int, int, Regs<T>& r) const {
#pragma unroll
        for (int i = 0; i < T / CL; i++) {
            const int tr = __builtin_amdgcn_readfirstlane(st.tr[i]), ts = __builtin_amdgcn_readfirstlane(st.ts[i]);
            const bool row_ok = (unsigned)(st.p0 + tr - 1) < (unsigned)H;
            const int at = st.pos + st.coloff[i];
            // the group that holds the row's padded element is fetched through the centre tap's position
            const bool edge = st.q0 == (ts == 0 ? 0 : W - G) && ts != 1;
            r.v[i] = PixVec<G>::load(st.rsrc, row_ok ? at + (edge ? 2 - 2 * ts : 0) : OOB);
            r.edge[i] = edge; r.ts[i] = ts;
        }
        // next slice: KH pixels further (W >= G; rows of fewer than KH pixels wrap more than once)
        st.q0 += KH; st.pos += KH * 2;
#pragma unroll
        for (int w = 0; w < 3; w++) {
            const bool wrap = st.q0 >= W;
            st.q0 -= wrap ? W : 0; st.p0 += wrap ? 1 : 0;
        }
        const bool next = st.p0 >= H;
        st.p0 -= next ? H : 0;
        st.pos += next ? (C - 1) * H * W * 2 : 0;
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / CL; i++) {
            const int ts = __builtin_amdgcn_readfirstlane(r.ts[i]);
            const V v = ts == 0 ? PixVec<G>::up(r.v[i], r.edge[i]) : (ts == 2 ? PixVec<G>::down(r.v[i], r.edge[i]) : r.v[i]);
            *(V*)(lds + (tid / PG + CL * i) * HSTRIDE + G * (tid % PG)) = v;
        }
    }
};

} // namespace vdnn

namespace vdnn {

// ---- im2col operand of forward (unit column stride) / backward data, a pixel pair per lane --------------
// The engine is bound by the number of load instructions. Two neighbouring output pixels of a row read two
// neighbouring elements of an input row through any tap: one 32-bit load (two-byte alignment suffices for
// buffer loads, and with consecutive lanes on consecutive pairs a wavefront's load still covers one run of
// a plane). Item = (pixel pair, eight consecutive channels): eight loads, a 2x8 transpose of 16-bit values
// (v_perm_b32), two 128-bit LDS stores. A pixel left or right of the image is read from the neighbouring row
// and masked; a pair whose second pixel is past the right edge is fetched one element lower (the last element
// of the descriptor's range must not be the first half of a word) and unpacked from the upper halves.
// Needs an even output row length, unit column stride in forward, at most 16 taps per filter row.
template <int MODE>
struct LoadIm2colPixTapH2 {
    LoadIm2colPix<MODE, false, bf16_t> base; // geometry only
    template <int T> struct Regs { uintx4 v[T / 128][2]; }; // [item][pixel of the pair]
    template <int T> struct State {
        int vbase[T / 128];       // byte offset of the pair's first pixel from the descriptor base
        unsigned invrow[T / 128]; // bit r set: filter row r reads outside the image
        unsigned colbad[T / 128]; // bit 2*s + e set: pixel e of the pair reads outside the image through filter column s
        __amdgpu_buffer_rsrc_t rsrc;
    };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int j0, int tid, int ncols, int) const {
        constexpr int PAIRS = T / 2;
        const int opix = base.OH * base.OW;
        const int n_first = j0 / opix;
        const long first = (long)n_first * base.sample_elems;
        const long shift = MODE == 0 ? -((long)base.ph * base.Ws + base.pw) : (long)(base.ph - base.R + 1) * base.Ws + (base.pw - base.S + 1);
        int n_last = (j0 + T - 1) / opix;
        if (n_last > base.nsamples - 1) n_last = base.nsamples - 1;
        st.rsrc = make_rsrc(base.src + first + shift, clamp_range(((long)(n_last - n_first + 1) * base.sample_elems - shift) * 2));
        const int j = j0 + 2 * (tid % PAIRS);
        const bool valid = j < ncols;
        const int jj = valid ? j : j0;
        const int n = jj / opix, pix = jj - n * opix;
        const int oh = pix / base.OW, ow = pix - oh * base.OW;
        const int ih0 = MODE == 0 ? oh * base.sh - base.ph : oh + base.ph;
        const int iw0 = MODE == 0 ? ow - base.pw : ow + base.pw;
        unsigned vrow = 0, bad = 0;
        for (int r = 0; r < base.R; r++)
            if ((unsigned)(MODE == 0 ? ih0 + r : ih0 - r) < (unsigned)base.Hs) vrow |= 1u << r;
        for (int s = 0; s < base.S; s++)
            for (int e = 0; e < 2; e++)
                if (!((unsigned)(MODE == 0 ? iw0 + e + s : iw0 + e - s) < (unsigned)base.Ws)) bad |= 1u << (2 * s + e);
        if (!valid) { vrow = 0; bad = ~0u; }
#pragma unroll
        for (int i = 0; i < T / 128; i++) { // the items of a thread differ in their channels only
            st.vbase[i] = (int)(((long)(n - n_first) * base.sample_elems + (long)(MODE == 0 ? oh * base.sh : oh) * base.Ws + ow) * 2);
            st.invrow[i] = ~vrow; st.colbad[i] = bad;
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int, int tid, Regs<T>& r) const {
        constexpr int PAIRS = T / 2;
        const int plane = base.Hs * base.Ws;
        const int slice = kk0 / KH;
        const int cb = base.divRS.div(slice), tap = slice - cb * (base.R * base.S);
        const int tr = base.divS.div(tap), ts = tap - tr * base.S;
        const int tapoff = MODE == 0 ? tr * base.Ws + ts : (base.R - 1 - tr) * base.Ws + (base.S - 1 - ts);
        const int g0 = __builtin_amdgcn_readfirstlane(tid / PAIRS);
#pragma unroll
        for (int i = 0; i < T / 128; i++) {
            const unsigned m0 = (unsigned)bit_to_all_ones(st.colbad[i], 2 * ts), m1 = (unsigned)bit_to_all_ones(st.colbad[i], 2 * ts + 1);
            // second pixel outside: fetch one element lower, the first pixel is then the upper half of each word
            const int voff = (st.vbase[i] + (int)(m1 & 0xFFFFFFFEu)) | bit_to_all_ones(st.invrow[i], tr); // m1 is 0 or -1: adds -2
            const unsigned sel0 = m1 ? 0x07060302u : 0x05040100u;
            const int ch = cb * KH + 8 * (g0 + (NT / PAIRS) * i);
            const int soff = (ch * plane + tapoff) * 2, step = plane * 2;
            unsigned c[8];
#pragma unroll
            for (int e = 0; e < 8; e++) c[e] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(st.rsrc, voff, soff + e * step, 0);
            r.v[i][0].x = __builtin_amdgcn_perm(c[1], c[0], sel0) & ~m0; r.v[i][0].y = __builtin_amdgcn_perm(c[3], c[2], sel0) & ~m0;
            r.v[i][0].z = __builtin_amdgcn_perm(c[5], c[4], sel0) & ~m0; r.v[i][0].w = __builtin_amdgcn_perm(c[7], c[6], sel0) & ~m0;
            r.v[i][1].x = __builtin_amdgcn_perm(c[1], c[0], 0x07060302u) & ~m1; r.v[i][1].y = __builtin_amdgcn_perm(c[3], c[2], 0x07060302u) & ~m1;
            r.v[i][1].z = __builtin_amdgcn_perm(c[5], c[4], 0x07060302u) & ~m1; r.v[i][1].w = __builtin_amdgcn_perm(c[7], c[6], 0x07060302u) & ~m1;
        }
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
        constexpr int PAIRS = T / 2;
#pragma unroll
        for (int i = 0; i < T / 128; i++)
#pragma unroll
            for (int e = 0; e < 2; e++)
                *(uintx4*)(lds + (2 * (tid % PAIRS) + e) * HSTRIDE + 8 * (tid / PAIRS + (NT / PAIRS) * i)) = r.v[i][e];
    }
};

} // namespace vdnn
