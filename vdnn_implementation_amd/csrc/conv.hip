// Convolution forward, backward-data and backward-filter as implicit GEMM on fp32 MFMA.
// Replaces cudnnConvolutionForward/AddTensor/BackwardData/BackwardFilter (layer.cu:539-665).
//
// GEMM views (NCHW activations, KCRS filters, cross-correlation):
//   forward      Out[k][(n,p,q)]   = sum_{(c,r,s)} w[k][(c,r,s)]   * x[n,c,p*sh-ph+r,q*sw-pw+s]
//   backward data Out[c][(n,h,w)]  = sum_{(k,r,s)} w[k,c,r,s]      * dy[n,k,(h+ph-r)/sh,(w+pw-s)/sw]
//   backward filter Out[k][(c,r,s)] = sum_{(n,p,q)} dy[n,k,p,q]    * x[n,c,p*sh-ph+r,q*sw-pw+s]
// The im2col operand is never materialised: each thread computes the addresses of its elements
// and the tiles exist only in LDS.
#include "backend_internal.h"
#include "mfma_gemm.h"

namespace vdnn {

struct ConvGeo {
    int N, C, H, W, K, R, S, P, Q, ph, pw, sh, sw;
};

static bool geo_from_shape(const vdnn_shape_t* s, ConvGeo& g) {
    g.N = s->n; g.C = s->c; g.H = s->h; g.W = s->w; g.K = s->k; g.R = s->r; g.S = s->s;
    g.ph = s->pad_h; g.pw = s->pad_w; g.sh = s->stride_h; g.sw = s->stride_w;
    if (g.N <= 0 || g.C <= 0 || g.H <= 0 || g.W <= 0 || g.K <= 0 || g.R <= 0 || g.S <= 0) return false;
    if (g.sh <= 0 || g.sw <= 0 || g.ph < 0 || g.pw < 0) return false;
    if (g.R > 16 || g.S > 16) return false; // tap masks are 16 bits wide
    g.P = vdnn_out_dim(g.H, g.ph, g.R, g.sh);
    g.Q = vdnn_out_dim(g.W, g.pw, g.S, g.sw);
    if (g.P <= 0 || g.Q <= 0) return false;
    // element counts of one sample must fit 31 bits (per-sample offsets are 32-bit)
    if ((long)g.C * g.H * g.W >= (1l << 31) || (long)g.K * g.P * g.Q >= (1l << 31)) return false;
    if ((long)g.N * g.P * g.Q >= (1l << 31) || (long)g.N * g.H * g.W >= (1l << 31)) return false;
    if ((long)g.C * g.R * g.S >= (1l << 24) || (long)g.K * g.R * g.S >= (1l << 24)) return false;
    return true;
}

// ---- im2col operand, columns = output pixels (row-major in LDS: lanes run along pixels) ---------
// MODE 0: forward gather from x.          src[n, ch, oh*sh-ph+r, ow*sw-pw+s]
// MODE 1: backward data, stride 1.        src[n, ch, oh+ph-r,    ow+pw-s]          (src = dy)
// MODE 2: backward data, any stride.      src[n, ch, (oh+ph-r)/sh, (ow+pw-s)/sw] where divisible
template <int MODE>
struct LoadIm2colPix {
    static constexpr bool RED_MAJOR = false;
    const float* src;
    int Hs, Ws;      // extent of one source plane
    int OH, OW;      // extent of the output pixel grid
    int R, S, ph, pw, sh, sw;
    long sample_stride; // channels_of_src * Hs * Ws
    FastDiv divRS, divS;
    const float* zeros; // a readable zero: masked taps are loaded from here
    struct State {
        const float* base;
        int off0, ih0, iw0;
        unsigned rowmask, colmask;
        bool valid;
    };
    template <int T>
    __device__ __forceinline__ void init(State& st, int j0, int tid, int ncols) const {
        const int j = j0 + tid % T;
        st.valid = j < ncols;
        const int jj = st.valid ? j : 0;
        const int opix = OH * OW;
        const int n = jj / opix, pix = jj - n * opix;
        const int oh = pix / OW, ow = pix - oh * OW;
        st.base = src + (long)n * sample_stride;
        st.rowmask = 0; st.colmask = 0;
        if (MODE == 0) {
            st.ih0 = oh * sh - ph; st.iw0 = ow * sw - pw;
            for (int r = 0; r < R; r++) if (st.ih0 + r >= 0 && st.ih0 + r < Hs) st.rowmask |= 1u << r;
            for (int s = 0; s < S; s++) if (st.iw0 + s >= 0 && st.iw0 + s < Ws) st.colmask |= 1u << s;
        } else {
            st.ih0 = oh + ph; st.iw0 = ow + pw;
            if (MODE == 1) {
                for (int r = 0; r < R; r++) if (st.ih0 - r >= 0 && st.ih0 - r < Hs) st.rowmask |= 1u << r;
                for (int s = 0; s < S; s++) if (st.iw0 - s >= 0 && st.iw0 - s < Ws) st.colmask |= 1u << s;
            } else {
                for (int r = 0; r < R; r++) { const int t = st.ih0 - r; if (t >= 0 && t % sh == 0 && t / sh < Hs) st.rowmask |= 1u << r; }
                for (int s = 0; s < S; s++) { const int t = st.iw0 - s; if (t >= 0 && t % sw == 0 && t / sw < Ws) st.colmask |= 1u << s; }
            }
        }
        st.off0 = st.ih0 * Ws + st.iw0;
        if (!st.valid) { st.rowmask = 0; st.colmask = 0; }
    }
    template <int T>
    __device__ __forceinline__ void load(const State& st, int kk0, int kend, int tid, float (&r)[LdsLayout<T, false>::NLOAD]) const {
        using L = LdsLayout<T, false>;
        const int RS = R * S, plane = Hs * Ws;
        // every lane of a wavefront shares kk: keep the tap arithmetic on the scalar unit
        const int kbase = __builtin_amdgcn_readfirstlane(kk0 + tid / T);
        // branch-free, and nothing depends on the loaded value until it is written to LDS
#pragma unroll
        for (int i = 0; i < L::NLOAD; i++) {
            const int kk = kbase + (NT / T) * i;
            const int ch = divRS.div(kk), rs = kk - ch * RS;
            const int tr = divS.div(rs), ts = rs - tr * S;
            const bool ok = (kk < kend) & (((st.rowmask >> tr) & (st.colmask >> ts) & 1u) != 0);
            int off;
            if (MODE == 0) off = st.off0 + ch * plane + tr * Ws + ts;
            else if (MODE == 1) off = st.off0 + ch * plane - tr * Ws - ts;
            else off = ch * plane + ((st.ih0 - tr) / sh) * Ws + (st.iw0 - ts) / sw;
            const float* p = ok ? st.base + off : zeros;
            r[i] = *p;
        }
    }
};

// ---- filter bank as the A operand of backward data: A[c][(k,r,s)] = w[k,c,r,s] ------------------
struct LoadFilterT {
    static constexpr bool RED_MAJOR = true;
    const float* w;
    int C, RS;
    const float* zeros;
    struct State { int row0; };
    template <int T>
    __device__ __forceinline__ void init(State& st, int row0, int, int) const { st.row0 = row0; }
    template <int T>
    __device__ __forceinline__ void load(const State& st, int kk0, int kend, int tid, float (&r)[LdsLayout<T, true>::NLOAD]) const {
        using L = LdsLayout<T, true>;
        const int kk = kk0 + tid % KB;
        const int k = kk / RS, rs = kk - k * RS;
        const long kbase = (long)k * C * RS + rs;
#pragma unroll
        for (int i = 0; i < L::NLOAD; i++) {
            const int c = st.row0 + L::row_of(tid, i);
            const bool ok = (kk < kend) & (c < C);
            const float* p = ok ? w + (kbase + (long)c * RS) : zeros;
            r[i] = *p;
        }
    }
};

// ---- dy as the A operand of backward filter: A[k][(n,p,q)] = dy[n,k,p,q] -------------------------
struct LoadDyRed {
    static constexpr bool RED_MAJOR = true;
    const float* dy;
    int K, PQ;
    const float* zeros;
    struct State { int row0; };
    template <int T>
    __device__ __forceinline__ void init(State& st, int row0, int, int) const { st.row0 = row0; }
    template <int T>
    __device__ __forceinline__ void load(const State& st, int kk0, int kend, int tid, float (&r)[LdsLayout<T, true>::NLOAD]) const {
        using L = LdsLayout<T, true>;
        const int kk = kk0 + tid % KB;
        const bool kok = kk < kend;
        const int kc = kok ? kk : 0;
        const int n = kc / PQ, pq = kc - n * PQ;
        const float* base = dy + (long)n * K * PQ + pq;
#pragma unroll
        for (int i = 0; i < L::NLOAD; i++) {
            const int m = st.row0 + L::row_of(tid, i);
            const bool ok = kok & (m < K);
            const float* p = ok ? base + (long)m * PQ : zeros;
            r[i] = *p;
        }
    }
};

// ---- im2col operand of backward filter: B[(n,p,q)][(c,r,s)] = x[n,c,p*sh-ph+r,q*sw-pw+s] ---------
// reduction-major: lanes of a load run along the pixel index, which is contiguous in x for sw == 1.
struct LoadIm2colRed {
    static constexpr bool RED_MAJOR = true;
    const float* x;
    int C, H, W, R, S, P, Q, ph, pw, sh, sw;
    int ncols; // C*R*S
    const float* zeros;
    static constexpr int MAXROWS = 256 * KB / NT; // rows per thread for the widest tile
    struct State {
        int joff[MAXROWS]; // c*H*W + r*W + s, or -1 when the column is out of range
        int jrs[MAXROWS];  // r << 8 | s
    };
    template <int T>
    __device__ __forceinline__ void init(State& st, int j0, int tid, int) const {
        using L = LdsLayout<T, true>;
        const int RS = R * S;
#pragma unroll
        for (int i = 0; i < L::NLOAD; i++) {
            const int j = j0 + L::row_of(tid, i);
            if (j < ncols) {
                const int c = j / RS, rs = j - c * RS;
                const int r = rs / S, s = rs - r * S;
                st.joff[i] = c * H * W + r * W + s;
                st.jrs[i] = (r << 8) | s;
            } else {
                st.joff[i] = -1;
                st.jrs[i] = 0;
            }
        }
    }
    template <int T>
    __device__ __forceinline__ void load(const State& st, int kk0, int kend, int tid, float (&r)[LdsLayout<T, true>::NLOAD]) const {
        using L = LdsLayout<T, true>;
        const int kk = kk0 + tid % KB;
        const bool kok = kk < kend;
        const int kc = kok ? kk : 0;
        const int PQ = P * Q;
        const int n = kc / PQ, pq = kc - n * PQ;
        const int p = pq / Q, q = pq - p * Q;
        const int ih0 = p * sh - ph, iw0 = q * sw - pw;
        const float* sample = x + (long)n * C * H * W;
        const int poff = ih0 * W + iw0;
#pragma unroll
        for (int i = 0; i < L::NLOAD; i++) {
            const int tr = st.jrs[i] >> 8, ts = st.jrs[i] & 255;
            const int ih = ih0 + tr, iw = iw0 + ts;
            const bool ok = kok & (st.joff[i] >= 0) & ((unsigned)ih < (unsigned)H) & ((unsigned)iw < (unsigned)W);
            const float* p = ok ? sample + (poff + st.joff[i]) : zeros;
            r[i] = *p;
        }
    }
};

// ---- result of forward / backward data: out[n][m][pix] = acc (+ bias[m]) --------------------------
struct StoreNCHW {
    float* out;
    const float* bias; // optional, per output channel
    int opix;          // pixels of one output plane
    __device__ __forceinline__ void store(const floatx16 (&acc)[2][2], int m0, int j0, int lane, int, const GemmDims& d) const {
        const int l32 = lane & 31, lk = lane >> 5;
#pragma unroll
        for (int jt = 0; jt < 2; jt++) {
            const int j = j0 + jt * 32 + l32;
            if (j >= d.N) continue;
            const int n = j / opix, pix = j - n * opix;
            float* o = out + (size_t)n * d.M * opix + pix;
#pragma unroll
            for (int it = 0; it < 2; it++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int m = m0 + it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                    if (m >= d.M) continue;
                    float r = acc[it][jt][v];
                    if (bias) r += bias[m];
                    o[(size_t)m * opix] = r;
                }
        }
    }
};

static GemmDims make_dims(int M, int N, int K, int TM, int TN, int splits) {
    GemmDims d;
    d.M = M; d.N = N; d.K = K;
    d.mtiles = (M + TM - 1) / TM;
    d.ntiles = (N + TN - 1) / TN;
    if (splits < 1) splits = 1;
    int kchunk = (K + splits - 1) / splits;
    kchunk = (kchunk + KB - 1) / KB * KB;
    d.kchunk = kchunk;
    d.splits = (K + kchunk - 1) / kchunk;
    return d;
}

// names of the kernel classes in the timing report: {pass}_{tile}
struct PassNames { const char* t64; const char* t128; };
static const PassNames kFwdNames{"conv_fwd_64x256", "conv_fwd_128x128"};
static const PassNames kBwdDataNames{"conv_bwd_data_64x256", "conv_bwd_data_128x128"};
static const PassNames kBwdFilterNames{"conv_bwd_filter_64x256", "conv_bwd_filter_128x128"};

template <int TM, int TN, class AL, class BL, class EP>
static int launch_igemm(vdnn_ctx* ctx, hipStream_t stream, const char* name, const AL& al, const BL& bl, const EP& ep, const GemmDims& d) {
    const long blocks = (long)d.mtiles * d.ntiles * d.splits;
    if (blocks <= 0 || blocks >= (1l << 31)) { set_error("igemm: grid of %ld workgroups out of range", blocks); return VDNN_EINVAL; }
    ProfScope prof(ctx, stream, name, 2.0 * d.M * (double)d.N * d.K, 0.0);
    hipLaunchKernelGGL((igemm_kernel<TM, TN, AL, BL, EP>), dim3((unsigned)blocks), dim3(NT), 0, stream, al, bl, ep, d);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

// Tile shape by output-channel count: 64-row tiles for narrow layers, 128 otherwise.
template <class AL, class BL, class EP>
static int launch_by_m(vdnn_ctx* ctx, hipStream_t stream, const PassNames& names, const AL& al, const BL& bl, const EP& ep, int M, int N, int K, int splits) {
    if (M <= 64) return launch_igemm<64, 256>(ctx, stream, names.t64, al, bl, ep, make_dims(M, N, K, 64, 256, splits));
    return launch_igemm<128, 128>(ctx, stream, names.t128, al, bl, ep, make_dims(M, N, K, 128, 128, splits));
}

int launch_reduce_splits(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count,
                         int splits, float alpha, int accumulate, const float* bias_j, int ncols);

} // namespace vdnn

using namespace vdnn;

extern "C" {

size_t vdnn_conv_workspace_bytes(const vdnn_shape_t* shape, int algo_mode, int pass) {
    ConvGeo g;
    if (!shape || !geo_from_shape(shape, g)) return 0;
    if (algo_mode == 0 /* VDNN_MEMORY_OPT_ALGO */) return 0;
    (void)pass;
    return 0; // the workspace-using variants are selected per pass below once they exist
}

int vdnn_conv_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                  const float* x, const float* w, const float* bias, float* y,
                  void* workspace, size_t workspace_bytes) {
    VDNN_KERNEL_PROLOGUE(ctx);
    (void)algo_mode; (void)workspace; (void)workspace_bytes;
    ConvGeo g;
    VDNN_REQUIRE(shape && geo_from_shape(shape, g), "unsupported convolution geometry");
    VDNN_REQUIRE(x && w && y, "null tensor");
    hipStream_t st = stream_of(ctx, stream);
    LoadDense<true> al{w, (long)g.C * g.R * g.S, 1, g.K, ctx->zeros};
    LoadIm2colPix<0> bl{x, g.H, g.W, g.P, g.Q, g.R, g.S, g.ph, g.pw, g.sh, g.sw, (long)g.C * g.H * g.W, FastDiv::make(g.R * g.S), FastDiv::make(g.S), ctx->zeros};
    StoreNCHW ep{y, bias, g.P * g.Q};
    return launch_by_m(ctx, st, kFwdNames, al, bl, ep, g.K, g.N * g.P * g.Q, g.C * g.R * g.S, 1);
}

int vdnn_conv_bwd_data(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                       const float* dy, const float* w, float* dx,
                       void* workspace, size_t workspace_bytes) {
    VDNN_KERNEL_PROLOGUE(ctx);
    (void)algo_mode; (void)workspace; (void)workspace_bytes;
    ConvGeo g;
    VDNN_REQUIRE(shape && geo_from_shape(shape, g), "unsupported convolution geometry");
    VDNN_REQUIRE(dy && w && dx, "null tensor");
    hipStream_t st = stream_of(ctx, stream);
    LoadFilterT al{w, g.C, g.R * g.S, ctx->zeros};
    StoreNCHW ep{dx, nullptr, g.H * g.W};
    const int M = g.C, N = g.N * g.H * g.W, K = g.K * g.R * g.S;
    if (g.sh == 1 && g.sw == 1) {
        LoadIm2colPix<1> bl{dy, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, 1, 1, (long)g.K * g.P * g.Q, FastDiv::make(g.R * g.S), FastDiv::make(g.S), ctx->zeros};
        return launch_by_m(ctx, st, kBwdDataNames, al, bl, ep, M, N, K, 1);
    }
    LoadIm2colPix<2> bl{dy, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, g.sh, g.sw, (long)g.K * g.P * g.Q, FastDiv::make(g.R * g.S), FastDiv::make(g.S), ctx->zeros};
    return launch_by_m(ctx, st, kBwdDataNames, al, bl, ep, M, N, K, 1);
}

int vdnn_conv_bwd_filter_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                             const float* x, const float* dy, float* w, float alpha,
                             void* workspace, size_t workspace_bytes) {
    VDNN_KERNEL_PROLOGUE(ctx);
    (void)algo_mode;
    ConvGeo g;
    VDNN_REQUIRE(shape && geo_from_shape(shape, g), "unsupported convolution geometry");
    VDNN_REQUIRE(x && dy && w, "null tensor");
    hipStream_t st = stream_of(ctx, stream);
    const int M = g.K, N = g.C * g.R * g.S;
    const long Kred = (long)g.N * g.P * g.Q;
    VDNN_REQUIRE(Kred < (1l << 31), "reduction too long");
    // Split the (n,p,q) reduction so the grid fills the chip; partial sums go to a staging area and
    // are added in split order by a second kernel (no floating-point atomics).
    const int TM = M <= 64 ? 64 : 128, TN = M <= 64 ? 256 : 128;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    float* staging = ctx->reduce_scratch;
    size_t staging_bytes = ctx->reduce_scratch_bytes;
    if (workspace && workspace_bytes > staging_bytes) { staging = (float*)workspace; staging_bytes = workspace_bytes; }
    const size_t out_bytes = (size_t)M * N * sizeof(float);
    long want = (4l * ctx->num_cu + tiles - 1) / tiles;
    const long by_depth = (Kred + 4 * KB - 1) / (4 * KB); // at least four slices per split
    if (want > by_depth) want = by_depth;
    const long by_mem = staging ? (long)(staging_bytes / out_bytes) : 1;
    if (want > by_mem) want = by_mem;
    if (want < 1) want = 1;
    GemmDims d = make_dims(M, N, (int)Kred, TM, TN, (int)want);
    LoadDyRed al{dy, g.K, g.P * g.Q, ctx->zeros};
    LoadIm2colRed bl{x, g.C, g.H, g.W, g.R, g.S, g.P, g.Q, g.ph, g.pw, g.sh, g.sw, N, ctx->zeros};
    StoreDense ep{w, staging, nullptr, (long)N, (long)M * N, alpha, 1};
    int rc = M <= 64 ? launch_igemm<64, 256>(ctx, st, kBwdFilterNames.t64, al, bl, ep, d) : launch_igemm<128, 128>(ctx, st, kBwdFilterNames.t128, al, bl, ep, d);
    if (rc != VDNN_OK) return rc;
    if (d.splits > 1) return launch_reduce_splits(ctx, st, w, staging, (size_t)M * N, d.splits, alpha, 1, nullptr, 0);
    return VDNN_OK;
}

} // extern "C"
