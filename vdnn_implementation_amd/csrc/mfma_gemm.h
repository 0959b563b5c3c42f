// fp32 MFMA tile engine shared by the convolution and fully-connected kernels.
//
// One workgroup of 256 threads (4 wavefronts of 64) produces a TM x TN tile of
//     Out[m][j] = sum_kk A[m][kk] * B[kk][j]
// from KB-deep slices staged in LDS. Each wavefront owns a 64x64 sub-tile = 2x2 MFMA tiles of
// v_mfma_f32_32x32x2_f32 (64 accumulator registers per lane). Operands come from "loader" policies:
// a loader says how element (row, kk) of its operand is fetched from global memory (a dense matrix,
// a filter bank, or an im2col view of an NCHW tensor computed on the fly - the im2col matrix only
// ever exists as LDS tiles). Global loads run two slices ahead in registers, LDS is double-buffered,
// and the loop has one barrier per slice and no branch (see igemm_kernel).
//
// The matrix pipe and the vector ALU of a SIMD do not overlap well, so every vector instruction in
// the loop costs MFMA time. The loaders therefore fetch through buffer descriptors: an element that
// must read as zero (outside the matrix, a padding tap, beyond the reduction range) is given an
// out-of-range offset and the hardware returns 0 - no branch, no select, and nothing depends on the
// loaded value until it is written to LDS. Uniform parts of an address go into the scalar offset.
//
// LDS layouts:
//   reduction-major operand (a thread's load runs along kk): lds[row * (KB+4) + kk], moved as
//       128-bit chunks of four consecutive kk where the source allows
//   row-major operand (lanes run along the row/column index): lds[kk * T + row]
// MFMA operand mapping for 32x32x2: lane l supplies A[i = l%32][k = l/32] and B[k = l/32][j = l%32];
// result register v of lane l is D[8*(v/4) + 4*(l/32) + v%4][l%32]. The order in which the KB
// reduction indices of a slice are consumed is free as long as A and B agree: step (g, i) uses
// k = 8g + 4*(l/32) + i, so a lane's four values of a reduction-major operand are one 128-bit read.
#pragma once
#include <hip/hip_runtime.h>

namespace vdnn {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int KB = 16;              // reduction depth of one LDS slice
constexpr int NT = 256;             // threads per workgroup
constexpr int RED_STRIDE = KB + 4;  // row stride of a reduction-major LDS tile (80 bytes: 128-bit reads of 8 consecutive rows hit 8 different bank groups)
constexpr int OOB = -1;             // byte offset that is out of range for every descriptor
constexpr int SENT = 0x40000000;    // out-of-range marker that survives one addition of a second offset below 1 GiB
constexpr unsigned MAX_SUM_RANGE = 0x40000000u; // descriptors addressed with summed offsets must be smaller than this

// MI355X has 8 XCDs, each with its own L2; consecutive workgroup ids are dealt round-robin to the
// XCDs. Remap so that consecutive *logical* tiles (which share operand tiles) land on one XCD.
__device__ __forceinline__ int xcd_remap(int bid, int nblocks) {
    constexpr int XCD = 8;
    const int per = nblocks / XCD, rem = nblocks % XCD;
    const int xcd = bid % XCD, idx = bid / XCD;
    // XCD x holds logical ids [start_x, start_x + per + (x < rem))
    const int start = xcd * per + (xcd < rem ? xcd : rem);
    return start + idx;
}

// Division of a small non-negative integer by a loop-invariant divisor as a multiply-high with the
// 33-bit constant ceil(2^32 / d), kept as (hi, lo) so that d == 1 needs no branch.
// Exact while x * d < 2^32 (callers bound x below 2^24 and d by 256).
struct FastDiv {
    unsigned lo, hi;
    __host__ __device__ static FastDiv make(int divisor) {
        const unsigned long long m = (0x100000000ull + (unsigned)divisor - 1) / (unsigned)divisor;
        FastDiv f;
        f.lo = (unsigned)m;
        f.hi = (unsigned)(m >> 32);
        return f;
    }
    __device__ __forceinline__ int div(int x) const { return (int)(__umulhi((unsigned)x, lo) + (unsigned)x * hi); }
};

// ---- buffer descriptors: loads that return 0 outside [0, bytes) ----------------------------------
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}
// voff: per-lane byte offset; soff: wave-uniform byte offset. Out of range if voff + soff >= bytes
// (no 32-bit wrap-around: OOB + anything stays out of range).
__device__ __forceinline__ float buf_load(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
__device__ __forceinline__ floatx4 buf_load4(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    return __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}
// Descriptor range for `bytes` remaining after the base, clamped to what a descriptor can hold.
__device__ __forceinline__ unsigned clamp_range(long bytes) {
    return bytes <= 0 ? 0u : (bytes > 0xFFFFFFF0l ? 0xFFFFFFF0u : (unsigned)bytes);
}

// ---- element types of activation tensors -------------------------------------------------------------
// Activations are float or bfloat16 in memory; every kernel computes in float. A bf16 value is the
// upper half of the float with the same value; storing rounds to nearest, ties to even, NaN stays NaN.
struct bf16_t { unsigned short bits; };
template <class E> struct ElemBytes { static constexpr int V = (int)sizeof(E); };

__host__ __device__ __forceinline__ float bf16_bits_to_float(unsigned bits) {
    return __builtin_bit_cast(float, bits << 16);
}
// On the device the conversion is one instruction (v_cvt_pk_bf16_f32, two values at a time); it gives the bits of
// the arithmetic below for every one of the 2^32 inputs, NaN payloads and denormals included.
__host__ __device__ __forceinline__ unsigned short float_to_bf16_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(unsigned short, (__bf16)f);
#else
    unsigned u = __builtin_bit_cast(unsigned, f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (unsigned short)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
#endif
}
// two values in one word, the first in the lower half
__device__ __forceinline__ unsigned pack2_bf16(float lo, float hi) {
    typedef float float_x2 __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16_x2 __attribute__((ext_vector_type(2)));
    float_x2 f; f.x = lo; f.y = hi;
    return __builtin_bit_cast(unsigned, __builtin_convertvector(f, bf16_x2));
}
__device__ __forceinline__ float load_elem(const float* p) { return *p; }
__device__ __forceinline__ float load_elem(const bf16_t* p) { return bf16_bits_to_float(p->bits); }
__device__ __forceinline__ void store_elem(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_elem(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

// one element / four consecutive elements through a descriptor, as float (offsets in bytes)
// max(v, 0) that lets NaN through
__device__ __forceinline__ float relu_value(float v) { return v > 0.0f ? v : (v != v ? v : 0.0f); }

template <class E> __device__ __forceinline__ float buf_load_e(__amdgpu_buffer_rsrc_t r, int voff, int soff);
template <> __device__ __forceinline__ float buf_load_e<float>(__amdgpu_buffer_rsrc_t r, int voff, int soff) { return buf_load(r, voff, soff); }
template <> __device__ __forceinline__ float buf_load_e<bf16_t>(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    return bf16_bits_to_float((unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(r, voff, soff, 0));
}
template <class E> __device__ __forceinline__ floatx4 buf_load4_e(__amdgpu_buffer_rsrc_t r, int voff, int soff);
template <> __device__ __forceinline__ floatx4 buf_load4_e<float>(__amdgpu_buffer_rsrc_t r, int voff, int soff) { return buf_load4(r, voff, soff); }
template <> __device__ __forceinline__ floatx4 buf_load4_e<bf16_t>(__amdgpu_buffer_rsrc_t r, int voff, int soff) {
    typedef unsigned uintx2 __attribute__((ext_vector_type(2)));
    const uintx2 w = __builtin_bit_cast(uintx2, __builtin_amdgcn_raw_buffer_load_b64(r, voff, soff, 0));
    floatx4 v;
    v.x = __builtin_bit_cast(float, w.x << 16); v.y = __builtin_bit_cast(float, w.x & 0xFFFF0000u);
    v.z = __builtin_bit_cast(float, w.y << 16); v.w = __builtin_bit_cast(float, w.y & 0xFFFF0000u);
    return v;
}

// ---- LDS tile geometry ------------------------------------------------------------------------------
template <int T, bool RED_MAJOR>
struct LdsTile {
    static constexpr int SIZE = RED_MAJOR ? T * RED_STRIDE : KB * T;
    static constexpr int ROW_STRIDE = RED_MAJOR ? RED_STRIDE : 1;
};

// Four reduction values (k = 8g + 4*lk + i, i = 0..3) of row l32 of a 32-row tile at `tile`.
template <int T, bool RED_MAJOR>
__device__ __forceinline__ floatx4 read_frag(const float* tile, int l32, int lk, int g) {
    if (RED_MAJOR) {
        return *(const floatx4*)(tile + l32 * RED_STRIDE + 8 * g + 4 * lk);
    } else {
        const float* p = tile + (8 * g + 4 * lk) * T + l32;
        floatx4 v;
        v.x = p[0]; v.y = p[T]; v.z = p[2 * T]; v.w = p[3 * T];
        return v;
    }
}

// Launch geometry of one igemm call. Split s covers reduction indices [s*kchunk, min(K, (s+1)*kchunk)).
// full_tiles > 0 (tail mode): the first full_tiles tiles are computed whole by one workgroup each, only the
// remaining tiles - the ones that would start a nearly empty last round - are split.
struct GemmDims {
    int M, N, K;
    int mtiles, ntiles, splits, kchunk;
    int full_tiles;
};

// Number of reduction splits for a grid of `tiles` output tiles over a reduction of K, at most
// max_splits. Measured on the part: workgroups are resident three to a compute unit, so a grid runs
// fastest when it is a little under a multiple of the unit count, best a multiple of three units'
// worth; one more workgroup than that starts a nearly empty round. The estimate below counts, per
// compute unit, rounds x (slices per split + a fixed prologue/epilogue) with the measured efficiency
// of a round count, plus the traffic of writing and re-reading one partial result per split.
static inline int choose_splits(long tiles, long K, long max_splits, int num_cu, size_t out_bytes, double tile_flops_per_slice) {
    if (max_splits < 1) max_splits = 1;
    const long useful = 12l * num_cu / tiles + 1; // beyond twelve rounds the estimate only grows
    if (max_splits > useful) max_splits = useful;
    const double us_per_slice = tile_flops_per_slice / (118e6 / num_cu); // one unit at ~118 TFLOP/s / units
    const double us_per_split = (double)out_bytes * 2.0 / 4e6;           // partials at ~4 TB/s
    double best = 0.0;
    int best_s = 1;
    for (long s = 1; s <= max_splits; s++) {
        long kchunk = (K + s - 1) / s;
        kchunk = (kchunk + KB - 1) / KB * KB;
        const long splits = (K + kchunk - 1) / kchunk;
        const long rounds = (tiles * splits + num_cu - 1) / num_cu;
        const double eff = rounds == 1 ? 0.72 : rounds == 2 ? 0.92 : rounds == 4 ? 0.93 : rounds % 3 == 0 ? 1.0 : 0.97;
        const double cost = (double)rounds * (double)(kchunk / KB + 6) * us_per_slice / eff + (splits > 1 ? (double)splits * us_per_split : 0.0);
        if (s == 1 || cost < best) { best = cost; best_s = (int)s; }
    }
    return best_s;
}

template <int TM, int TN, class AL, class BL, class EP>
__global__ void __launch_bounds__(NT) igemm_kernel(const AL al, const BL bl, const EP ep, const GemmDims d) {
    static_assert(TM % 64 == 0 && TN % 64 == 0 && (TM / 64) * (TN / 64) == 4, "four 64x64 wave tiles");
    using LA = LdsTile<TM, AL::RED_MAJOR>;
    using LB = LdsTile<TN, BL::RED_MAJOR>;
    __shared__ __attribute__((aligned(16))) float As[2][LA::SIZE];
    __shared__ __attribute__((aligned(16))) float Bs[2][LB::SIZE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    // m-tile fastest: workgroups that share a B tile (the large operand) are neighbours
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
    const int mt = tile % d.mtiles, nt = tile / d.mtiles;
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
    typename AL::template Regs<TM> ra;
    typename BL::template Regs<TN> rb;

    // Software pipeline, one barrier per slice - in the middle of it - and no branch in the loop.
    // A slice's 32 MFMAs per wavefront run as two groups of 16 (reduction indices 0-7 and 8-15).
    //   first half of slice s:  read the fragments of (s, group 1) from LDS buffer s%2, multiply group 0
    //                           (fragments already in registers), write the registers holding slice s+1
    //                           (fetched during slice s-1) to the other LDS buffer;
    //   barrier;
    //   second half:            issue the fetch of slice s+2 into the same registers, read the fragments
    //                           of (s+1, group 0) from the buffer just completed, multiply group 1.
    // Each group's fragments are thus read while the previous group is multiplied, across the barrier as
    // well, so no wavefront waits for LDS; a global load has a full slice of MFMA time to return. All
    // reads of a buffer precede the barrier after which it may be overwritten. Fetches past the end of
    // the range read as zero or are never used: buffer loads cannot fault, the last rounds need no guard.
    const int nslices = (k_end - k_begin + KB - 1) / KB;
    const int l32 = lane & 31, lk = lane >> 5;
    constexpr int A_TILE = 32 * LA::ROW_STRIDE, B_TILE = 32 * LB::ROW_STRIDE;
    const int a_off = wm0 * LA::ROW_STRIDE, b_off = wn0 * LB::ROW_STRIDE;
    al.template load<TM>(sa, k_begin, k_end, tid, ra);
    bl.template load<TN>(sb, k_begin, k_end, tid, rb);
    AL::template store<TM>(As[0], tid, ra);
    BL::template store<TN>(Bs[0], tid, rb);
    al.template load<TM>(sa, k_begin + KB, k_end, tid, ra);
    bl.template load<TN>(sb, k_begin + KB, k_end, tid, rb);
    __syncthreads();
    floatx4 a0[2], b0[2], a1[2], b1[2];
#pragma unroll
    for (int i = 0; i < 2; i++) a0[i] = read_frag<TM, AL::RED_MAJOR>(As[0] + a_off + i * A_TILE, l32, lk, 0);
#pragma unroll
    for (int j = 0; j < 2; j++) b0[j] = read_frag<TN, BL::RED_MAJOR>(Bs[0] + b_off + j * B_TILE, l32, lk, 0);
    for (int s = 0; s < nslices; s++) {
        const int cur = s & 1, nxt = cur ^ 1;
#pragma unroll
        for (int i = 0; i < 2; i++) a1[i] = read_frag<TM, AL::RED_MAJOR>(As[cur] + a_off + i * A_TILE, l32, lk, 1);
#pragma unroll
        for (int j = 0; j < 2; j++) b1[j] = read_frag<TN, BL::RED_MAJOR>(Bs[cur] + b_off + j * B_TILE, l32, lk, 1);
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[i][e], b0[j][e], acc[i][j], 0, 0, 0);
        AL::template store<TM>(As[nxt], tid, ra);
        BL::template store<TN>(Bs[nxt], tid, rb);
        // issue order of the first half: every MFMA is followed by one LDS access
#pragma unroll
        for (int i = 0; i < 16; i++) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x300, 2, 0); }
        __syncthreads();
        const int kk0 = k_begin + (s + 2) * KB;
        al.template load<TM>(sa, kk0, k_end, tid, ra);
        bl.template load<TN>(sb, kk0, k_end, tid, rb);
#pragma unroll
        for (int i = 0; i < 2; i++) a0[i] = read_frag<TM, AL::RED_MAJOR>(As[nxt] + a_off + i * A_TILE, l32, lk, 0);
#pragma unroll
        for (int j = 0; j < 2; j++) b0[j] = read_frag<TN, BL::RED_MAJOR>(Bs[nxt] + b_off + j * B_TILE, l32, lk, 0);
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[i][e], b1[j][e], acc[i][j], 0, 0, 0);
        // second half: every MFMA is followed by a global load and an LDS read
#pragma unroll
        for (int i = 0; i < 16; i++) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
    }

    if (EP::TAIL && d.full_tiles > 0 && !whole)
        ep.store_tail(acc, wm0, wn0, lane, (long)(tile - d.full_tiles) * d.splits + ks, TM, TN);
    else
        ep.store(acc, m0 + wm0, j0 + wn0, lane, ks, d, !whole);
}

// ---- dense reduction-major operand: element (row, kk) at base[row*ld + kk] -------------------------
// VEC4: rows are 16-byte aligned and the reduction range is a multiple of four, so a thread moves
// 128-bit chunks (thread t: chunk t%4 of rows t/4 + 64*i). Otherwise 32-bit elements
// (thread t: kk t%16 of rows t/16 + 16*i).
template <bool VEC4, class E = float>
struct LoadDenseRed {
    static constexpr bool RED_MAJOR = true;
    static constexpr int ES = ElemBytes<E>::V;
    const E* base;
    long ld;          // elements between rows
    int rows;         // valid rows
    unsigned bytes;   // extent of the matrix in bytes (below 2 GiB)
    template <int T> struct Regs { floatx4 v[T / 64]; float s[VEC4 ? 1 : T / 16]; };
    template <int T> struct State { int vrow[VEC4 ? T / 64 : T / 16]; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(base, bytes);
        if (VEC4) {
#pragma unroll
            for (int i = 0; i < T / 64; i++) {
                const int row = row0 + (tid >> 2) + 64 * i;
                st.vrow[i] = row < rows ? (int)(((long)row * ld + 4 * (tid & 3)) * ES) : OOB;
            }
        } else {
#pragma unroll
            for (int i = 0; i < T / 16; i++) {
                const int row = row0 + (tid >> 4) + 16 * i;
                st.vrow[i] = row < rows ? (int)(((long)row * ld + (tid & 15)) * ES) : OOB;
            }
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int kend, int tid, Regs<T>& r) const {
        const int soff = kk0 * ES;
        // only the last slice of a range can be partial; there a thread past the end reads out of range
        const bool tail = kk0 + KB > kend;
        if (VEC4) {
            const bool dead = tail && (kk0 + 4 * (tid & 3) >= kend);
#pragma unroll
            for (int i = 0; i < T / 64; i++) r.v[i] = buf_load4_e<E>(st.rsrc, dead ? OOB : st.vrow[i], soff);
        } else {
            const bool dead = tail && (kk0 + (tid & 15) >= kend);
#pragma unroll
            for (int i = 0; i < T / 16; i++) r.s[i] = buf_load_e<E>(st.rsrc, dead ? OOB : st.vrow[i], soff);
        }
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

// ---- dense row-major operand: element (row, kk) at base[kk*ld_k + row] ------------------------------
// lanes run along rows (coalesced); the reduction index is wave-uniform and lives in the scalar offset
template <class E = float>
struct LoadDenseRow {
    static constexpr bool RED_MAJOR = false;
    static constexpr int ES = ElemBytes<E>::V;
    const E* base;
    long ld_k;        // elements between consecutive kk
    int rows;
    unsigned bytes;   // extent in bytes (below 2 GiB)
    template <int T> struct Regs { float s[T * KB / NT]; };
    template <int T> struct State { int vrow; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(base, bytes);
        const int row = row0 + tid % T;
        st.vrow = row < rows ? row * ES : OOB;
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int kend, int tid, Regs<T>& r) const {
        const int kbase = __builtin_amdgcn_readfirstlane(kk0 + tid / T);
#pragma unroll
        for (int i = 0; i < T * KB / NT; i++) {
            const int kk = kbase + (NT / T) * i;
            const int soff = kk < kend ? (int)((long)kk * ld_k * ES) : 0x7FFFFFF0;
            r.s[i] = buf_load_e<E>(st.rsrc, st.vrow, soff);
        }
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T * KB / NT; i++) lds[(tid / T + (NT / T) * i) * T + tid % T] = r.s[i];
    }
};

// the float nearest to v among those exactly representable in bfloat16 (ties to even, NaN stays NaN)
__device__ __forceinline__ float round_to_bf16_value(float v) { return bf16_bits_to_float(float_to_bf16_bits(v)); }

// An operand whose values are rounded to bfloat16 on their way into LDS: the filter operands of layers whose
// activations are stored as bfloat16 (the filter itself stays a float master copy in memory).
template <class L>
struct RoundedToBf16 : L {
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const typename L::template Regs<T>& r) {
        typename L::template Regs<T> q = r;
        float* f = (float*)&q;
#pragma unroll
        for (int i = 0; i < (int)(sizeof(q) / sizeof(float)); i++) f[i] = round_to_bf16_value(f[i]);
        L::template store<T>(lds, tid, q);
    }
};

// ---- dense result: out[m*ld_m + j] = alpha*acc (+ old if accumulate) (+ bias[j]); or a split's
//      partial sums to scratch[ks][m*ld_m + j] ------------------------------------------------------
template <class E = float>
struct StoreDense {
    E* out;
    float* partial;     // used when splits > 1
    const float* bias_j; // optional, indexed by column
    long ld_m;
    long partial_stride; // elements per split
    float alpha;
    int accumulate;
    int relu;      // rectify the result (after the bias)
    const E* gate; // optional, same layout as out: the result is kept where gate > 0 and zero elsewhere
    static constexpr bool TAIL = false;
    __device__ __forceinline__ void store_tail(const floatx16 (&)[2][2], int, int, int, long, int, int) const {}
    __device__ __forceinline__ void store(const floatx16 (&acc)[2][2], int m0, int j0, int lane, int ks, const GemmDims& d, bool to_partial) const {
        const int l32 = lane & 31, lk = lane >> 5;
        // What the result is combined with is read sixteen elements ahead of the stores: a load issued after a store
        // through the same pointer would have to wait for it (the compiler cannot know that the rows differ), and
        // sixty-four round trips to memory in a row are the kernel's whole time when the output is large (the filter of
        // a fully connected layer, updated in place). Sixteen, not more: the registers they wait in count against the
        // workgroups a compute unit holds.
        const bool combine = !to_partial && (accumulate || gate != nullptr);
#pragma unroll
        for (int jt = 0; jt < 2; jt++) {
            const int j = j0 + jt * 32 + l32;
            if (j >= d.N) continue;
            const float bj = (!to_partial && bias_j) ? bias_j[j] : 0.0f;
#pragma unroll
            for (int it = 0; it < 2; it++) {
                float aux[16]; // the old value (accumulate) or the gate: a call asks for one of the two at most
                if (combine) {
#pragma unroll
                    for (int v = 0; v < 16; v++) {
                        const int m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                        const long idx = (long)m * ld_m + j;
                        aux[v] = m < d.M ? (accumulate ? load_elem(out + idx) : load_elem(gate + idx)) : 0.0f;
                    }
                }
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                    if (m >= d.M) continue;
                    const long idx = (long)m * ld_m + j;
                    const float a = acc[it][jt][v];
                    if (to_partial) {
                        partial[(long)ks * partial_stride + idx] = a;
                    } else {
                        // one fused multiply-add: every route to "out += alpha * sum" rounds the same way
                        float r = accumulate ? __fmaf_rn(alpha, a, aux[v]) : alpha * a;
                        if (bias_j) r += bj;
                        if (relu) r = relu_value(r);
                        if (gate) r = (accumulate ? load_elem(gate + idx) : aux[v]) > 0.0f ? r : 0.0f;
                        store_elem(out + idx, r);
                    }
                }
            }
        }
    }
};

} // namespace vdnn
