// fp32 MFMA tile engine shared by the convolution and fully-connected kernels.
//
// One workgroup of 256 threads (4 wavefronts of 64) produces a TM x TN tile of
//     Out[m][j] = sum_kk A[m][kk] * B[kk][j]
// from KB-deep slices staged in LDS. Each wavefront owns a 64x64 sub-tile = 2x2 MFMA tiles of
// v_mfma_f32_32x32x2_f32 (64 accumulator registers per lane). Operands come from "loader" policies:
// a loader says how element (row, kk) of its operand is fetched from global memory (a dense matrix,
// a filter bank, or an im2col view of an NCHW tensor computed on the fly - the im2col matrix only
// ever exists as LDS tiles). Loads for slice s+1 are issued into registers before slice s is
// multiplied, then written to the other LDS buffer: one barrier per slice.
//
// LDS layouts (chosen so both the global-load lane order and the MFMA operand reads are
// bank-conflict free):
//   reduction-major operand (lanes of a load run along kk):  lds[row * (KB+1) + kk]
//   row-major operand       (lanes of a load run along the row/column index): lds[kk * T + row]
// MFMA operand mapping for 32x32x2: lane l supplies A[i = l%32][k = l/32] and B[k = l/32][j = l%32];
// result register v of lane l is D[8*(v/4) + 4*(l/32) + v%4][l%32].
#pragma once
#include <hip/hip_runtime.h>

namespace vdnn {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int KB = 16;   // reduction depth of one LDS slice
constexpr int NT = 256;  // threads per workgroup

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

template <int T, bool RED_MAJOR>
struct LdsLayout {
    static constexpr int ROW_STRIDE = RED_MAJOR ? (KB + 1) : 1;
    static constexpr int K_STRIDE = RED_MAJOR ? 1 : T;
    static constexpr int SIZE = RED_MAJOR ? T * (KB + 1) : KB * T;
    static constexpr int NLOAD = T * KB / NT; // elements each thread moves per slice
    // element i of a thread: (row, kk) within the tile
    __device__ static __forceinline__ int row_of(int tid, int i) { return RED_MAJOR ? (tid / KB + (NT / KB) * i) : (tid % T); }
    __device__ static __forceinline__ int kk_of(int tid, int i) { return RED_MAJOR ? (tid % KB) : (tid / T + (NT / T) * i); }
    __device__ static __forceinline__ void store(float* lds, int tid, const float (&r)[NLOAD]) {
#pragma unroll
        for (int i = 0; i < NLOAD; i++) lds[row_of(tid, i) * ROW_STRIDE + kk_of(tid, i) * K_STRIDE] = r[i];
    }
};

template <int A_RS, int A_KS, int B_RS, int B_KS>
__device__ __forceinline__ void mfma_slice(const float* __restrict__ As, const float* __restrict__ Bs,
                                           floatx16 (&acc)[2][2], int lane) {
    const int l32 = lane & 31, lk = lane >> 5;
    // operand fragments of step t+1 are read from LDS while the four MFMAs of step t execute
    float a[2][2], b[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++) a[0][i] = As[(i * 32 + l32) * A_RS + lk * A_KS];
#pragma unroll
    for (int j = 0; j < 2; j++) b[0][j] = Bs[(j * 32 + l32) * B_RS + lk * B_KS];
#pragma unroll
    for (int t = 0; t < KB / 2; t++) {
        const int cur = t & 1, nxt = cur ^ 1;
        if (t + 1 < KB / 2) {
            const int k = 2 * (t + 1) + lk;
#pragma unroll
            for (int i = 0; i < 2; i++) a[nxt][i] = As[(i * 32 + l32) * A_RS + k * A_KS];
#pragma unroll
            for (int j = 0; j < 2; j++) b[nxt][j] = Bs[(j * 32 + l32) * B_RS + k * B_KS];
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][i], b[cur][j], acc[i][j], 0, 0, 0);
    }
}

// Launch geometry of one igemm call. Split s covers reduction indices [s*kchunk, min(K, (s+1)*kchunk)).
struct GemmDims {
    int M, N, K;
    int mtiles, ntiles, splits, kchunk;
};

template <int TM, int TN, class AL, class BL, class EP>
__global__ void __launch_bounds__(NT) igemm_kernel(const AL al, const BL bl, const EP ep, const GemmDims d) {
    static_assert(TM % 64 == 0 && TN % 64 == 0 && (TM / 64) * (TN / 64) == 4, "four 64x64 wave tiles");
    using LA = LdsLayout<TM, AL::RED_MAJOR>;
    using LB = LdsLayout<TN, BL::RED_MAJOR>;
    __shared__ float As[2][LA::SIZE];
    __shared__ float Bs[2][LB::SIZE];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int bid = xcd_remap(blockIdx.x, gridDim.x);
    // m-tile fastest: workgroups that share a B tile (the large operand) are neighbours
    const int mt = bid % d.mtiles;
    const int rest = bid / d.mtiles;
    const int nt = rest % d.ntiles;
    const int ks = rest / d.ntiles;
    const int m0 = mt * TM, j0 = nt * TN;
    const int k_begin = ks * d.kchunk;
    const int k_end = min(d.K, k_begin + d.kchunk);

    typename AL::State sa;
    typename BL::State sb;
    al.template init<TM>(sa, m0, tid, d.M);
    bl.template init<TN>(sb, j0, tid, d.N);

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;

    const int wm0 = (wave % (TM / 64)) * 64, wn0 = (wave / (TM / 64)) * 64;
    float ra[LA::NLOAD], rb[LB::NLOAD];

    const int nslices = (k_end - k_begin + KB - 1) / KB;
    if (nslices > 0) {
        al.template load<TM>(sa, k_begin, k_end, tid, ra);
        bl.template load<TN>(sb, k_begin, k_end, tid, rb);
        LA::store(As[0], tid, ra);
        LB::store(Bs[0], tid, rb);
    }
    __syncthreads();
    for (int s = 0; s < nslices; s++) {
        const int cur = s & 1;
        const bool more = s + 1 < nslices;
        if (more) {
            const int kk0 = k_begin + (s + 1) * KB;
            al.template load<TM>(sa, kk0, k_end, tid, ra);
            bl.template load<TN>(sb, kk0, k_end, tid, rb);
        }
        mfma_slice<LA::ROW_STRIDE, LA::K_STRIDE, LB::ROW_STRIDE, LB::K_STRIDE>(
            As[cur] + wm0 * LA::ROW_STRIDE, Bs[cur] + wn0 * LB::ROW_STRIDE, acc, lane);
        if (more) {
            LA::store(As[cur ^ 1], tid, ra);
            LB::store(Bs[cur ^ 1], tid, rb);
        }
        __syncthreads();
    }

    ep.store(acc, m0 + wm0, j0 + wn0, lane, ks, d);
}

// ---- dense operand: element (row, kk) at base[row*ld_row + kk*ld_k] -----------------------------
template <bool RED_MAJOR_>
struct LoadDense {
    static constexpr bool RED_MAJOR = RED_MAJOR_;
    const float* base;
    long ld_row, ld_k;
    int rows; // valid rows
    const float* zeros; // a readable zero: elements outside the matrix are loaded from here
    struct State { int row0; };
    template <int T>
    __device__ __forceinline__ void init(State& st, int row0, int, int) const { st.row0 = row0; }
    template <int T>
    __device__ __forceinline__ void load(const State& st, int kk0, int kend, int tid, float (&r)[LdsLayout<T, RED_MAJOR>::NLOAD]) const {
        using L = LdsLayout<T, RED_MAJOR>;
        // branch-free, and nothing depends on the loaded value until it is written to LDS
#pragma unroll
        for (int i = 0; i < L::NLOAD; i++) {
            const int row = st.row0 + L::row_of(tid, i);
            const int kk = kk0 + L::kk_of(tid, i);
            const bool ok = (row < rows) & (kk < kend);
            const float* p = ok ? base + ((long)row * ld_row + (long)kk * ld_k) : zeros;
            r[i] = *p;
        }
    }
};

// ---- dense result: out[m*ld_m + j] = alpha*acc (+ old if accumulate) (+ bias[j]); or a split's
//      partial sums to scratch[ks][m*ld_m + j] ------------------------------------------------------
struct StoreDense {
    float* out;
    float* partial;     // used when splits > 1
    const float* bias_j; // optional, indexed by column
    long ld_m;
    long partial_stride; // elements per split
    float alpha;
    int accumulate;
    __device__ __forceinline__ void store(const floatx16 (&acc)[2][2], int m0, int j0, int lane, int ks, const GemmDims& d) const {
        const int l32 = lane & 31, lk = lane >> 5;
#pragma unroll
        for (int jt = 0; jt < 2; jt++) {
            const int j = j0 + jt * 32 + l32;
            if (j >= d.N) continue;
#pragma unroll
            for (int it = 0; it < 2; it++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                    if (m >= d.M) continue;
                    const long idx = (long)m * ld_m + j;
                    const float a = acc[it][jt][v];
                    if (d.splits > 1) {
                        partial[(long)ks * partial_stride + idx] = a;
                    } else {
                        float r = alpha * a;
                        if (accumulate) r = out[idx] + r;
                        if (bias_j) r += bias_j[j];
                        out[idx] = r;
                    }
                }
        }
    }
};

} // namespace vdnn
