// Winograd F(4x4, 3x3) for the forward and backward-data passes of 3x3 / stride 1 / padding 1 layers with float
// activations: the perf-optimal mode's workspace-using variant (the reference asks cuDNN for its fastest algorithm and
// hands it the workspace that algorithm wants, layer.cu:1013-1089, 268-294).
//
// An output tile of 4x4 pixels is computed from the 6x6 input patch around it as
//     Y = At [ sum_c (G g_c Gt) .* (Bt d_c B) ] A
// (g_c: the 3x3 filter of one input channel, d_c: the patch of that channel): 36 multiplies per channel for 16
// outputs instead of 144 - a quarter of the direct convolution's. The sum over channels, for each of the 36 positions
// xi of the transformed patch, is a matrix product  M_xi[m][t] = sum_c U_xi[m][c] * V_xi[c][t]  over all tiles t of a
// chunk of samples; the 36 products run as ONE launch of the fp32 MFMA tile engine (columns j = xi * Tpad + t; the A
// loader below picks U_xi from the column tile's index). Four kernels per call:
//   1. wino_filter_kernel    U[xi][m][c]   = (G g Gt)[xi]            (backward data: the filter flipped and transposed)
//   2. wino_input_kernel     V[c][xi][t]   = (Bt d B)[xi]            per chunk of samples
//   3. igemm_kernel          M[m][xi][t]   = sum_c U[xi][m][c] V[c][xi][t]
//   4. wino_output_kernel    y[n][m][tile] = At M A + bias, rectifier / gate applied
// U, V and M live in the caller's workspace. Backward data is the same computation on dy with the filter
// w'[c][k][r][s] = w[k][c][2-r][2-s]. Tiles at the right / lower edge of a plane whose extent is not a multiple of
// four are computed whole and stored in part. The sums differ from the direct kernels' in order and by the
// transforms' rounding (about 1.5e-5 of the largest output for 512 channels, against 3e-7 direct): results are
// not bit-equal to the memory-optimal mode's, and equal from run to run and policy to policy within this mode.
#pragma once
#include "mfma_gemm.h"

namespace vdnn {

constexpr int WINO_XI = 36;   // positions of the transformed 6x6 patch
constexpr int WINO_TN = 128;  // column tile of the product: a tile's columns share one xi

// Bt v for the six values of a patch row / column
__device__ __forceinline__ void wino_bt6(const float (&d)[6], float (&t)[6]) {
    t[0] = 4.0f * d[0] - 5.0f * d[2] + d[4];
    t[1] = -4.0f * (d[1] + d[2]) + d[3] + d[4];
    t[2] = 4.0f * (d[1] - d[2]) - d[3] + d[4];
    t[3] = 2.0f * (d[3] - d[1]) - d[2] + d[4];
    t[4] = 2.0f * (d[1] - d[3]) - d[2] + d[4];
    t[5] = 4.0f * d[1] - 5.0f * d[3] + d[5];
}
// At v: four outputs from six transformed values
__device__ __forceinline__ void wino_at4(const float (&m)[6], float (&o)[4]) {
    const float s12 = m[1] + m[2], d12 = m[1] - m[2], s34 = m[3] + m[4], d34 = m[3] - m[4];
    o[0] = m[0] + s12 + s34;
    o[1] = d12 + 2.0f * d34;
    o[2] = s12 + 4.0f * s34;
    o[3] = d12 + 8.0f * d34 + m[5];
}
// G v: six transformed values from three filter taps
__device__ __forceinline__ void wino_g6(const float (&g)[3], float (&u)[6]) {
    u[0] = g[0] * 0.25f;
    u[1] = -(g[0] + g[1] + g[2]) * (1.0f / 6.0f);
    u[2] = (g[1] - g[0] - g[2]) * (1.0f / 6.0f);
    u[3] = g[0] * (1.0f / 24.0f) + g[1] * (1.0f / 12.0f) + g[2] * (1.0f / 6.0f);
    u[4] = g[0] * (1.0f / 24.0f) - g[1] * (1.0f / 12.0f) + g[2] * (1.0f / 6.0f);
    u[5] = g[2];
}

// U[(xi * rows + m) * cred + c]. Forward: m = k, c = c, taps as stored. Backward data: m = c, reduced index = k, taps
// flipped. One thread per (m, c), lanes along c.
template <bool BWD>
__global__ void __launch_bounds__(256) wino_filter_kernel(const float* __restrict__ w, float* __restrict__ U, int rows, int cred) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)rows * cred) return;
    const int m = (int)(i / cred), c = (int)(i - (long)m * cred);
    // filter element (k, cc, r, s) at ((k * C + cc) * 3 + r) * 3 + s, with C = cred (forward) or rows (backward data)
    const float* g = BWD ? w + ((long)c * rows + m) * 9 : w + ((long)m * cred + c) * 9;
    float a[3][3];
#pragma unroll
    for (int r = 0; r < 3; r++)
#pragma unroll
        for (int s = 0; s < 3; s++) a[r][s] = BWD ? g[(2 - r) * 3 + (2 - s)] : g[r * 3 + s];
    float t[6][3]; // G a
#pragma unroll
    for (int s = 0; s < 3; s++) {
        const float col[3] = {a[0][s], a[1][s], a[2][s]};
        float u[6];
        wino_g6(col, u);
#pragma unroll
        for (int x = 0; x < 6; x++) t[x][s] = u[x];
    }
#pragma unroll
    for (int x = 0; x < 6; x++) {
        float u[6];
        wino_g6(t[x], u);
#pragma unroll
        for (int y = 0; y < 6; y++) U[((long)(x * 6 + y) * rows + m) * cred + c] = u[y];
    }
}

struct WinoTiles {
    int H, W;          // plane (input and output planes have one extent)
    int th, tw;        // tiles per column / row: ceil(H/4), ceil(W/4)
    int chan;          // channels of the tensor (input transform: reduced channels; output transform: rows)
    int T;             // tiles of the chunk: samples * th * tw
    long Tpad;         // T rounded up to the product's column tile
};

// V[(c * 36 + xi) * Tpad + t] for the chunk's samples (src points at the chunk's first sample). One thread per
// (c, t), lanes along t: the 36 stores of a wavefront are 256 contiguous bytes each. VEC: rows are whole groups of four
// pixels, so a tile's four inner columns are one aligned 128-bit load.
template <bool VEC>
__global__ void __launch_bounds__(256) wino_input_kernel(const float* __restrict__ src, float* __restrict__ V, const WinoTiles g) {
    const int t = blockIdx.x * 256 + threadIdx.x, c = blockIdx.y;
    if (t >= g.Tpad) return;
    if (t >= g.T) { // the columns that round the chunk up to whole tiles of the product: zero, so that sums over them add nothing
        float* pad = V + (long)c * WINO_XI * g.Tpad + t;
#pragma unroll
        for (int xi = 0; xi < WINO_XI; xi++) pad[(long)xi * g.Tpad] = 0.0f;
        return;
    }
    const int per = g.th * g.tw;
    const int n = t / per, rem = t - n * per;
    const int ty = rem / g.tw, tx = rem - ty * g.tw;
    const float* plane = src + ((long)n * g.chan + c) * g.H * g.W;
    float d[6][6];
#pragma unroll
    for (int i = 0; i < 6; i++) {
        const int row = 4 * ty - 1 + i;
        const bool rok = (unsigned)row < (unsigned)g.H;
        const float* p = plane + (long)row * g.W + 4 * tx;
        if (VEC) {
            floatx4 v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (rok) v = *(const floatx4*)p;
            d[i][0] = (rok && tx > 0) ? p[-1] : 0.0f;
            d[i][1] = v.x; d[i][2] = v.y; d[i][3] = v.z; d[i][4] = v.w;
            d[i][5] = (rok && 4 * tx + 4 < g.W) ? p[4] : 0.0f;
        } else {
#pragma unroll
            for (int j = 0; j < 6; j++) {
                const int col = 4 * tx - 1 + j;
                d[i][j] = (rok && (unsigned)col < (unsigned)g.W) ? p[j - 1] : 0.0f;
            }
        }
    }
    // Bt d: down the columns; then (Bt d) B: along the rows
#pragma unroll
    for (int j = 0; j < 6; j++) {
        const float col[6] = {d[0][j], d[1][j], d[2][j], d[3][j], d[4][j], d[5][j]};
        float r[6];
        wino_bt6(col, r);
#pragma unroll
        for (int i = 0; i < 6; i++) d[i][j] = r[i];
    }
    float* out = V + (long)c * WINO_XI * g.Tpad + t;
#pragma unroll
    for (int i = 0; i < 6; i++) {
        float r[6];
        wino_bt6(d[i], r);
#pragma unroll
        for (int j = 0; j < 6; j++) out[(long)(i * 6 + j) * g.Tpad] = r[j];
    }
}

// dst[n][m][4 ty + i][4 tx + j] = (At M A)[i][j] + bias[m], rectified / gated like the direct kernels' epilogue
// (bias, then the rectifier, then the gate: kept where gate > 0). M[(m * 36 + xi) * Tpad + t]. One thread per (m, t),
// lanes along t. A gate that is the output tensor itself is read by the thread that overwrites it, before it does.
template <bool VEC>
__global__ void __launch_bounds__(256) wino_output_kernel(const float* __restrict__ M, float* dst, const float* __restrict__ bias, const float* gate,
                                                          int relu, const WinoTiles g) {
    const int t = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
    if (t >= g.T) return;
    const int per = g.th * g.tw;
    const int n = t / per, rem = t - n * per;
    const int ty = rem / g.tw, tx = rem - ty * g.tw;
    const float* in = M + (long)m * WINO_XI * g.Tpad + t;
    float a[4][6]; // At M
#pragma unroll
    for (int j = 0; j < 6; j++) {
        float col[6];
#pragma unroll
        for (int i = 0; i < 6; i++) col[i] = in[(long)(i * 6 + j) * g.Tpad];
        float o[4];
        wino_at4(col, o);
#pragma unroll
        for (int i = 0; i < 4; i++) a[i][j] = o[i];
    }
    const float b = bias ? bias[m] : 0.0f;
    const long plane = ((long)n * g.chan + m) * g.H * g.W;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = 4 * ty + i;
        if (row >= g.H) break;
        float o[4];
        wino_at4(a[i], o);
        const long at = plane + (long)row * g.W + 4 * tx;
        if (VEC) {
            floatx4 gt = {1.0f, 1.0f, 1.0f, 1.0f};
            if (gate) gt = *(const floatx4*)(gate + at);
            floatx4 r;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float v = o[j] + b;
                if (relu) v = relu_value(v);
                r[j] = gt[j] > 0.0f ? v : 0.0f;
            }
            *(floatx4*)(dst + at) = r;
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                if (4 * tx + j >= g.W) break;
                float v = o[j] + b;
                if (relu) v = relu_value(v);
                if (gate) v = gate[at + j] > 0.0f ? v : 0.0f;
                dst[at + j] = v;
            }
        }
    }
}

// The product's A operand: U_xi, a dense reduction-major matrix of `rows` x `ld`, where xi belongs to the column tile
// of the workgroup. The loader decodes the workgroup's tile the way igemm_kernel does for an unsplit launch.
struct LoadWinoU : LoadDenseRed<true, float> {
    long xi_stride;   // elements of one U_xi
    int mtiles, ntiles_all, tiles_per_xi;
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        const int bid = xcd_remap(blockIdx.x, gridDim.x);
        const int nt = (bid % ntiles_all) / mtiles;
        const int xi = nt / tiles_per_xi;
        st.rsrc = make_rsrc(base + (long)xi * xi_stride, bytes);
#pragma unroll
        for (int i = 0; i < T / 64; i++) {
            const int row = row0 + (tid >> 2) + 64 * i;
            st.vrow[i] = row < rows ? (int)(((long)row * ld + 4 * (tid & 3)) * 4) : OOB;
        }
    }
};

// The product's B operand: V as a dense row-major matrix (element (column j, kk) at base[kk * ld_k + j]) whose rows
// are whole groups of four columns, 16-byte aligned, and whose reduction is a whole number of slices: a thread moves two
// 128-bit chunks per slice (chunk tid % (T/4) of reduction rows tid / (T/4) + (NT / (T/4)) * i) instead of eight single
// elements. The thread's own reduction row rides in its vector offset, the slice's in the scalar offset.
struct LoadDenseRowVec4 {
    static constexpr bool RED_MAJOR = false;
    const float* base;
    long ld_k;        // elements between consecutive kk (a multiple of four)
    int rows;         // columns of the matrix (a multiple of four)
    unsigned bytes;   // extent in bytes (below 2 GiB)
    template <int T> struct Regs { floatx4 v[T * KB / (4 * NT)]; };
    template <int T> struct State { int vrow; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(base, bytes);
        const int row = row0 + 4 * (tid % (T / 4));
        st.vrow = row < rows ? (int)(((long)(tid / (T / 4)) * ld_k + row) * 4) : OOB;
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int kend, int, Regs<T>& r) const {
        constexpr int PER = NT / (T / 4); // reduction rows covered by one round of the workgroup's loads
#pragma unroll
        for (int i = 0; i < T * KB / (4 * NT); i++) {
            const int kk = kk0 + PER * i; // wave-uniform; a slice lies wholly inside the reduction or wholly beyond it
            const int soff = kk < kend ? (int)((long)kk * ld_k * 4) : 0x7FFFFFF0;
            r.v[i] = buf_load4(st.rsrc, st.vrow, soff);
        }
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
        constexpr int PER = NT / (T / 4);
#pragma unroll
        for (int i = 0; i < T * KB / (4 * NT); i++) *(floatx4*)(lds + (tid / (T / 4) + PER * i) * T + 4 * (tid % (T / 4))) = r.v[i];
    }
};

// ---- the 36 products of forward / backward data, several column tiles per workgroup ------------------------------
// M[m][xi * Tpad + t] = sum_c U[xi][m][c] * V[c][xi * Tpad + t]. The reduction is only cred / 16 slices long (8 for 128
// channels): with one 128 x 128 tile per workgroup (igemm_kernel) the wait for the first operands and the 64 stores per
// lane at the end weigh as much as the multiplies. Here a workgroup computes `group` consecutive column tiles of one
// (xi, 128 rows): the software pipeline of igemm_kernel - global loads two slices ahead, LDS double-buffered, one barrier
// per slice, fragments of the next half slice read while the current one is multiplied - runs on across the tile
// boundaries (the slice after a tile's last is the next tile's first), so only the first tile pays the wait, and a tile's
// result is stored while the wavefronts of the other resident workgroups multiply. Same products, same order of summation.
struct WinoGemm {
    const float* U;   // [36][rows][cred]
    const float* V;   // [cred][36 * Tpad]
    float* M;         // [rows][36 * Tpad]
    int rows, cred;
    long Tpad;        // a multiple of 128
    int mtiles, tiles_per_xi, group, groups_per_xi;
};

__global__ void __launch_bounds__(NT) wino_gemm_kernel(const WinoGemm g) {
    constexpr int TM = 128, TN = 128;
    __shared__ __attribute__((aligned(16))) float As[2][TM * RED_STRIDE];
    __shared__ __attribute__((aligned(16))) float Bs[2][KB * TN];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int mt = bid % g.mtiles, rest = bid / g.mtiles;
    const int grp = rest % g.groups_per_xi, xi = rest / g.groups_per_xi;
    const int tile0 = grp * g.group;
    const int ntile = min(g.group, g.tiles_per_xi - tile0);
    const int m0 = mt * TM;
    const int nsl = g.cred / KB;
    const long ld = (long)WINO_XI * g.Tpad;          // row length of V and of M
    const long col0 = (long)xi * g.Tpad + (long)tile0 * TN; // first column of the workgroup

    // A: rows tid/4 + 64 i of U_xi, four reduction values at 4 (tid % 4); B: reduction rows tid/32 + 8 i, columns 4 (tid % 32)
    const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.U + (long)xi * g.rows * g.cred, (unsigned)((size_t)g.rows * g.cred * sizeof(float)));
    const __amdgpu_buffer_rsrc_t rsB = make_rsrc(g.V + col0, clamp_range(((long)(g.cred - 1) * ld + (long)ntile * TN) * 4));
    int arow[2];
#pragma unroll
    for (int i = 0; i < 2; i++) {
        const int row = m0 + (tid >> 2) + 64 * i;
        arow[i] = row < g.rows ? (row * g.cred + 4 * (tid & 3)) * 4 : OOB;
    }
    const int brow = (int)(((long)(tid >> 5) * ld + 4 * (tid & 31)) * 4);
    floatx4 ra[2], rb[2];
    // the slice the next fetch is for: its reduction offset and its tile's column offset (bytes)
    int ps = 0, pcol = 0, ptile = 0;
    auto fetch = [&]() {
        const bool live = ptile < ntile;   // past the last tile nothing is fetched (the values would never be used)
#pragma unroll
        for (int i = 0; i < 2; i++) ra[i] = buf_load4(rsA, live ? arow[i] : OOB, ps * KB * 4);
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const long soff = ((long)(ps * KB + 8 * i) * ld) * 4 + pcol;
            rb[i] = buf_load4(rsB, live ? brow : OOB, (int)soff);
        }
        ps += 1;
        const bool wrap = ps == nsl;
        ps = wrap ? 0 : ps; pcol += wrap ? TN * 4 : 0; ptile += wrap ? 1 : 0;
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < 2; i++) *(floatx4*)(As[buf] + ((tid >> 2) + 64 * i) * RED_STRIDE + 4 * (tid & 3)) = ra[i];
#pragma unroll
        for (int i = 0; i < 2; i++) *(floatx4*)(Bs[buf] + ((tid >> 5) + 8 * i) * TN + 4 * (tid & 31)) = rb[i];
    };

    floatx16 acc[2][2];
    auto clear = [&]() {
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    };
    clear();
    const int wm0 = (wave & 1) * 64, wn0 = (wave >> 1) * 64;
    const int l32 = lane & 31, lk = lane >> 5;
    constexpr int A_TILE = 32 * RED_STRIDE, B_TILE = 32;
    const int a_off = wm0 * RED_STRIDE, b_off = wn0;

    fetch();
    stash(0);
    fetch();
    __syncthreads();
    floatx4 a0[2], b0[2], a1[2], b1[2];
#pragma unroll
    for (int i = 0; i < 2; i++) a0[i] = read_frag<TM, true>(As[0] + a_off + i * A_TILE, l32, lk, 0);
#pragma unroll
    for (int j = 0; j < 2; j++) b0[j] = read_frag<TN, false>(Bs[0] + b_off + j * B_TILE, l32, lk, 0);
    int v = 0; // slices done so far (over all tiles): LDS buffer v & 1 holds the current one
    for (int t = 0; t < ntile; t++) {
        for (int s2 = 0; s2 < nsl; s2++, v++) {
            const int cur = v & 1, nxt = cur ^ 1;
#pragma unroll
            for (int i = 0; i < 2; i++) a1[i] = read_frag<TM, true>(As[cur] + a_off + i * A_TILE, l32, lk, 1);
#pragma unroll
            for (int j = 0; j < 2; j++) b1[j] = read_frag<TN, false>(Bs[cur] + b_off + j * B_TILE, l32, lk, 1);
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0[i][e], b0[j][e], acc[i][j], 0, 0, 0);
            stash(nxt);
#pragma unroll
            for (int i = 0; i < 16; i++) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x300, 2, 0); }
            __syncthreads();
            fetch();
#pragma unroll
            for (int i = 0; i < 2; i++) a0[i] = read_frag<TM, true>(As[nxt] + a_off + i * A_TILE, l32, lk, 0);
#pragma unroll
            for (int j = 0; j < 2; j++) b0[j] = read_frag<TN, false>(Bs[nxt] + b_off + j * B_TILE, l32, lk, 0);
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1[i][e], b1[j][e], acc[i][j], 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        }
        // the tile's result: acc[it][jt][v2] is row m0 + wm0 + 32 it + 8 (v2 / 4) + 4 lk + v2 % 4, column wn0 + 32 jt + l32
        float* out = g.M + col0 + (long)t * TN + wn0 + l32;
#pragma unroll
        for (int jt = 0; jt < 2; jt++)
#pragma unroll
            for (int it = 0; it < 2; it++)
#pragma unroll
                for (int v2 = 0; v2 < 16; v2++) {
                    const int m = m0 + wm0 + it * 32 + 8 * (v2 / 4) + 4 * lk + (v2 % 4);
                    if (m < g.rows) out[(long)m * ld + jt * 32] = acc[it][jt][v2];
                }
        clear();
    }
}

// ---- backward filter: F(3x3, 4x4) --------------------------------------------------------------------------------
// The filter gradient of one 4x4 tile of output pixels is the 3x3 "output" of correlating the 6x6 input patch with the
// 4x4 tile of dy as a "filter": dW = A't [ sum over tiles and samples of (G' dy G't) .* (Bt x B) ] A' with the same
// six interpolation points (0, 1, -1, 2, -2, infinity), hence the same Bt (and the same transformed input V as the
// forward pass), G' = the 6x4 and A't the 3x6 matrices of those points. The sum over tiles, for each of the 36
// positions, is a matrix product S_xi[k][c] = sum_t D_xi[k][t] V_xi[c][t] with a long reduction (all tiles of the
// batch): split along t, partial sums added in split order, then transformed back and applied to the filter.
__device__ __forceinline__ void wino_g6x4(const float (&g)[4], float (&u)[6]) {
    const float e = g[0] + g[2], o = g[1] + g[3];
    u[0] = g[0] * 0.25f;
    u[1] = -(e + o) * (1.0f / 6.0f);
    u[2] = (o - e) * (1.0f / 6.0f);
    const float a = g[0] * (1.0f / 24.0f) + g[2] * (1.0f / 6.0f), b = g[1] * (1.0f / 12.0f) + g[3] * (1.0f / 3.0f);
    u[3] = a + b;
    u[4] = a - b;
    u[5] = g[3];
}
__device__ __forceinline__ void wino_at3(const float (&m)[6], float (&o)[3]) {
    const float s12 = m[1] + m[2], d12 = m[1] - m[2], s34 = m[3] + m[4], d34 = m[3] - m[4];
    o[0] = m[0] + s12 + s34;
    o[1] = d12 + 2.0f * d34;
    o[2] = s12 + 4.0f * s34 + m[5];
}

// D[(k * 36 + xi) * Tpad + t] = (G' dy_tile G't)[xi]; pixels of the tile outside the plane count as zero; columns
// t >= T are zero. One thread per (k, t), lanes along t. BIAS: the workgroup also adds up the dy values it read - the
// bias gradient's share of its 256 tiles - in a fixed order (lanes by halving, then the four wavefronts in turn) and
// leaves the sum at bias_partial[k * bias_parts + bias_first + blockIdx.x].
template <bool VEC, bool BIAS>
__global__ void __launch_bounds__(256) wino_dy_kernel(const float* __restrict__ src, float* __restrict__ D, const WinoTiles g,
                                                      float* __restrict__ bias_partial, int bias_parts, int bias_first) {
    __shared__ float wave_sums[4];
    const int t = blockIdx.x * 256 + threadIdx.x, k = blockIdx.y;
    float mine = 0.0f;
    if (t < g.Tpad) {
        float* out = D + (long)k * WINO_XI * g.Tpad + t;
        if (t >= g.T) {
#pragma unroll
            for (int xi = 0; xi < WINO_XI; xi++) out[(long)xi * g.Tpad] = 0.0f;
        } else {
            const int per = g.th * g.tw;
            const int n = t / per, rem = t - n * per;
            const int ty = rem / g.tw, tx = rem - ty * g.tw;
            const float* plane = src + ((long)n * g.chan + k) * g.H * g.W;
            float d[4][4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = 4 * ty + i;
                const bool rok = row < g.H;
                const float* p = plane + (long)row * g.W + 4 * tx;
                if (VEC) {
                    floatx4 v = {0.0f, 0.0f, 0.0f, 0.0f};
                    if (rok) v = *(const floatx4*)p;
                    d[i][0] = v.x; d[i][1] = v.y; d[i][2] = v.z; d[i][3] = v.w;
                } else {
#pragma unroll
                    for (int j = 0; j < 4; j++) d[i][j] = (rok && 4 * tx + j < g.W) ? p[j] : 0.0f;
                }
                if (BIAS) mine += (d[i][0] + d[i][1]) + (d[i][2] + d[i][3]);
            }
            float h[6][4]; // G' d
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float col[4] = {d[0][j], d[1][j], d[2][j], d[3][j]};
                float u[6];
                wino_g6x4(col, u);
#pragma unroll
                for (int i = 0; i < 6; i++) h[i][j] = u[i];
            }
#pragma unroll
            for (int i = 0; i < 6; i++) {
                float u[6];
                wino_g6x4(h[i], u);
#pragma unroll
                for (int j = 0; j < 6; j++) out[(long)(i * 6 + j) * g.Tpad] = u[j];
            }
        }
    }
    if (BIAS) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) mine += __shfl_xor(mine, off);
        if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = mine;
        __syncthreads();
        if (threadIdx.x == 0)
            bias_partial[(long)k * bias_parts + bias_first + blockIdx.x] = ((wave_sums[0] + wave_sums[1]) + wave_sums[2]) + wave_sums[3];
    }
}

// An operand of the backward-filter product: rows (output channels of D, input channels of V) by tiles, reduction-major,
// element (row, kk) of position xi at base[(row * 36 + xi) * Tpad + kk]. The product's columns are j = xi * cpad + c.
// BY_COLUMN_TILE (the A operand, D): xi comes from the workgroup's column tile, decoded the way igemm_kernel does;
// otherwise (the B operand, V) from the tile's first column, which init is handed.
template <bool BY_COLUMN_TILE>
struct LoadWinoRed {
    static constexpr bool RED_MAJOR = true;
    const float* base;
    long tpad;        // reduction extent per (row, xi); rows are 36 * tpad apart
    int rows;         // valid rows of the tensor
    unsigned bytes;   // extent of the tensor in bytes (below 2 GiB)
    int cpad;         // columns per xi
    int mtiles, ntiles_all, tn;
    template <int T> struct Regs { floatx4 v[T / 64]; };
    template <int T> struct State { int vrow[T / 64]; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        int xi, first;
        if (BY_COLUMN_TILE) {
            const int bid = xcd_remap(blockIdx.x, gridDim.x);
            const int nt = (bid % ntiles_all) / mtiles;
            xi = nt * tn / cpad; first = row0;
        } else {
            xi = row0 / cpad; first = row0 - xi * cpad;
        }
        st.rsrc = make_rsrc(base + (long)xi * tpad, bytes - (unsigned)(xi * tpad * 4));
#pragma unroll
        for (int i = 0; i < T / 64; i++) {
            const int row = first + (tid >> 2) + 64 * i;
            st.vrow[i] = row < rows ? (int)(((long)row * WINO_XI * tpad + 4 * (tid & 3)) * 4) : OOB;
        }
    }
    // the reduction is a whole number of slices; a fetch past a split's end reads the next split's values or zeros and is never used
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int, int, Regs<T>& r) const {
#pragma unroll
        for (int i = 0; i < T / 64; i++) r.v[i] = buf_load4(st.rsrc, st.vrow[i], kk0 * 4);
    }
    template <int T>
    __device__ static __forceinline__ void store(float* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 64; i++) *(floatx4*)(lds + ((tid >> 2) + 64 * i) * RED_STRIDE + 4 * (tid & 3)) = r.v[i];
    }
};

// partial[0][i] = sum over p, in order, of partial[p][i]: the partial results of all chunks and splits, one thread per
// element (each thread reads its own element of the first result before it overwrites it).
__global__ void __launch_bounds__(256) wino_wgrad_sum_kernel(float* partial, long part_stride, int nparts, long count) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= count) return;
    float sum = 0.0f;
    for (int p = 0; p < nparts; p++) sum += partial[(long)p * part_stride + i];
    partial[i] = sum;
}

// w[k][c][r][s] = (accumulate ? w : 0) + alpha * (A't S A')[r][s], S[xi] = sum over the partial results, in their order,
// of partial[p][k][xi * cpad + c]. One thread per (k, c), lanes along c.
__global__ void __launch_bounds__(256) wino_wgrad_out_kernel(const float* __restrict__ partial, long part_stride, int nparts, float* w, int K, int C, int cpad,
                                                             float alpha, int accumulate) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)K * C) return;
    const int k = (int)(i / C), c = (int)(i - (long)k * C);
    const float* in = partial + (long)k * WINO_XI * cpad + c;
    float a[3][6]; // A't S
#pragma unroll
    for (int y = 0; y < 6; y++) {
        float col[6];
#pragma unroll
        for (int x = 0; x < 6; x++) {
            float sum = 0.0f;
            for (int p = 0; p < nparts; p++) sum += in[(long)p * part_stride + (long)(x * 6 + y) * cpad];
            col[x] = sum;
        }
        float o[3];
        wino_at3(col, o);
#pragma unroll
        for (int r = 0; r < 3; r++) a[r][y] = o[r];
    }
    float* out = w + i * 9;
#pragma unroll
    for (int r = 0; r < 3; r++) {
        float o[3];
        wino_at3(a[r], o);
#pragma unroll
        for (int s2 = 0; s2 < 3; s2++) out[r * 3 + s2] = accumulate ? __fmaf_rn(alpha, o[s2], out[r * 3 + s2]) : alpha * o[s2];
    }
}

} // namespace vdnn
