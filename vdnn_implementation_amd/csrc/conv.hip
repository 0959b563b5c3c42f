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
#include "conv_loaders.h"
#include "conv_loaders_tap.h"
#include "mfma_bf16.h"
#include "conv3x3_bf16.h"
#include "wgrad3x3_bf16.h"
#include "wgrad3x3_f32.h"
#include "wgrad3x3_split.h"
#include "conv_smallc.h"
#include "conv_smallc_mfma.h"
#include "winograd_f32.h"

namespace vdnn {

static bool geo_from_shape(const vdnn_shape_t* s, ConvGeo& g) {
    g.N = s->n; g.C = s->c; g.H = s->h; g.W = s->w; g.K = s->k; g.R = s->r; g.S = s->s;
    g.ph = s->pad_h; g.pw = s->pad_w; g.sh = s->stride_h; g.sw = s->stride_w;
    if (g.N <= 0 || g.C <= 0 || g.H <= 0 || g.W <= 0 || g.K <= 0 || g.R <= 0 || g.S <= 0) return false;
    if (g.sh <= 0 || g.sw <= 0 || g.ph < 0 || g.pw < 0) return false;
    if (g.R > 16 || g.S > 16) return false;        // tap masks are 16 bits per axis
    if (g.ph >= g.R || g.pw >= g.S) return false;  // padding of a full window or more is not supported
    g.P = vdnn_out_dim(g.H, g.ph, g.R, g.sh);
    g.Q = vdnn_out_dim(g.W, g.pw, g.S, g.sw);
    if (g.P <= 0 || g.Q <= 0) return false;
    const long x_sample = (long)g.C * g.H * g.W, y_sample = (long)g.K * g.P * g.Q;
    // one sample must fit 31 bits of elements; pixel and reduction counts must fit an int
    if (x_sample >= (1l << 29) || y_sample >= (1l << 29)) return false;
    if ((long)g.N * g.P * g.Q >= (1l << 31) || (long)g.N * g.H * g.W >= (1l << 31)) return false;
    if ((long)g.C * g.R * g.S >= (1l << 24) || (long)g.K * g.R * g.S >= (1l << 24)) return false;
    // the filter bank is addressed through one descriptor with summed offsets
    if ((long)g.K * g.C * g.R * g.S * 4 >= (long)MAX_SUM_RANGE) return false;
    return true;
}

// samples one tile of `tile` pixels can touch, times the sample size: must stay below 2 GiB so that
// per-lane byte offsets are positive ints and the exhausted-range scalar offset is out of range
static bool pixel_tile_span_ok(long sample_elems, int opix, int tile, int elem_bytes) {
    const long span = (long)(tile / opix + 2) * sample_elems * elem_bytes;
    return span < 0x7FFF0000l;
}

static GemmDims make_dims(int M, int N, int K, int TM, int TN, int splits, int depth = KB) {
    GemmDims d;
    d.M = M; d.N = N; d.K = K;
    d.mtiles = (M + TM - 1) / TM;
    d.ntiles = (N + TN - 1) / TN;
    if (splits < 1) splits = 1;
    int kchunk = (K + splits - 1) / splits;
    kchunk = (kchunk + depth - 1) / depth * depth;
    d.kchunk = kchunk;
    d.splits = (K + kchunk - 1) / kchunk;
    d.full_tiles = 0;
    return d;
}

// names of the kernel classes in the timing report: {pass}_{tile}
struct PassNames { const char* t64; const char* t128; };
static const PassNames kFwdNames{"conv_fwd_64x256", "conv_fwd_128x128"};
static const PassNames kBwdDataNames{"conv_bwd_data_64x256", "conv_bwd_data_128x128"};
static const PassNames kBwdFilterNames{"conv_bwd_filter_64x256", "conv_bwd_filter_128x128"};
static const PassNames kFwdPackedNames{"conv_fwd_packed_64x256", "conv_fwd_packed_128x128"};
static const PassNames kBwdDataPackedNames{"conv_bwd_data_packed_64x256", "conv_bwd_data_packed_128x128"};
static const PassNames kFwdHalfNames{"conv_fwd_bf16mfma_64x256", "conv_fwd_bf16mfma_128x128"};
static const PassNames kBwdDataHalfNames{"conv_bwd_data_bf16mfma_64x256", "conv_bwd_data_bf16mfma_128x128"};
static const PassNames kFwdWin3Names{"conv_fwd_bf16win_64x256", "conv_fwd_bf16win_64x256"};
static const PassNames kBwdDataWin3Names{"conv_bwd_data_bf16win_64x256", "conv_bwd_data_bf16win_64x256"};
static const PassNames kFwdSplitNames{"conv_fwd_split_64x256", "conv_fwd_split_64x256"};
static const PassNames kBwdDataSplitNames{"conv_bwd_data_split_64x256", "conv_bwd_data_split_64x256"};
static const PassNames kBwdFilterHalfNames{"conv_bwd_filter_bf16mfma_64x256", "conv_bwd_filter_bf16mfma_128x128"};
static const PassNames kBwdFilterWin3Names{"conv_bwd_filter_bf16win_64x192", "conv_bwd_filter_bf16win_128x192"};
static const PassNames kBwdFilterRow3Names{"conv_bwd_filter_row_64x192", "conv_bwd_filter_row_128x192"};

template <int TM, int TN, class AL, class BL, class EP, bool HALF = false>
static int launch_igemm(vdnn_ctx* ctx, hipStream_t stream, const char* name, const AL& al, const BL& bl, const EP& ep, const GemmDims& d, double flops = 0.0) {
    const long all_tiles = (long)d.mtiles * d.ntiles;
    const long blocks = d.full_tiles > 0 ? d.full_tiles + (all_tiles - d.full_tiles) * d.splits : all_tiles * d.splits;
    if (blocks <= 0 || blocks >= (1l << 31)) { set_error("igemm: grid of %ld workgroups out of range", blocks); return VDNN_EINVAL; }
    // reported work is the algorithmic count where the caller gives one (backward data of a strided or
    // unpadded layer multiplies taps that fall outside the output; they are not counted)
    ProfScope prof(ctx, stream, name, flops > 0.0 ? flops : 2.0 * d.M * (double)d.N * d.K, 0.0);
    if constexpr (HALF) hipLaunchKernelGGL((igemm_bf16_kernel<TM, TN, AL, BL, EP>), dim3((unsigned)blocks), dim3(NT), 0, stream, al, bl, ep, d);
    else hipLaunchKernelGGL((igemm_kernel<TM, TN, AL, BL, EP>), dim3((unsigned)blocks), dim3(NT), 0, stream, al, bl, ep, d);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

int launch_reduce_tail_nchw(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, int tail_tiles, int splits, int TM, int TN,
                            int M, int N, int mtiles, int full_tiles, const float* bias, int opix, int relu, const float* gate);
int launch_reduce_tail_nchw(vdnn_ctx* ctx, hipStream_t stream, bf16_t* out, const float* partial, int tail_tiles, int splits, int TM, int TN,
                            int M, int N, int mtiles, int full_tiles, const float* bias, int opix, int relu, const bf16_t* gate);
int launch_reduce_splits_tap(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count, int splits,
                             float alpha, int accumulate, int C, int RS);
int launch_reduce_splits_nchw(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count, int splits,
                              const float* bias, int opix, int channels, int relu, const float* gate);
int launch_reduce_splits_nchw(vdnn_ctx* ctx, hipStream_t stream, bf16_t* out, const float* partial, size_t count, int splits,
                              const float* bias, int opix, int channels, int relu, const bf16_t* gate);

// Forward / backward data. Tile shape by output-row count: 64-row tiles for narrow layers, 128
// otherwise. A grid that cannot fill the chip (few output pixels: the fully connected layers written
// as convolutions) splits its reduction; the partial sums go to the staging area and are added in split
// order, with the bias, by a second kernel. The split count depends on the shape only.
// HALF: the bfloat16 engine (32-deep slices); partial_bytes: room behind ep.partial (the context's staging
// area unless part of it is taken by something else).
template <class AL, class BL, class E, bool HALF = false>
static int launch_by_m(vdnn_ctx* ctx, hipStream_t stream, const PassNames& names, const AL& al, const BL& bl, const StoreNCHW<E>& ep, int M, int N, int K, double flops = 0.0,
                       size_t partial_bytes = ~(size_t)0) {
    constexpr int DEPTH = HALF ? KH : KB;
    if (partial_bytes == ~(size_t)0) partial_bytes = ctx->reduce_scratch_bytes;
    const bool narrow = M <= 64;
    const int TM = narrow ? 64 : 128, TN = narrow ? 256 : 128;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    int splits = 1;
    const size_t out_bytes = (size_t)M * N * sizeof(float);
    if (tiles < 2l * ctx->num_cu && ctx->reduce_scratch && ep.partial) {
        long cap = ((long)K + 8 * DEPTH - 1) / (8 * DEPTH); // at least eight slices per split
        const long by_mem = (long)(partial_bytes / out_bytes);
        if (cap > by_mem) cap = by_mem;
        splits = choose_splits(tiles, K, cap, ctx->num_cu, out_bytes, 2.0 * TM * TN * KB);
    }
    GemmDims d = make_dims(M, N, K, TM, TN, splits, DEPTH);
    // Tail mode: when the tiles make whole rounds of resident workgroups (three per compute unit) plus a
    // small remainder, that remainder would run as a nearly empty last round as long as a full one. Its
    // tiles are split so that together they fill about one round of short workgroups instead.
    const long slots = 3l * ctx->num_cu;
    const long rem = tiles % slots;
    int tail_tiles = 0;
    if (splits == 1 && tiles > slots && rem > 0 && 2 * rem <= slots && ctx->reduce_scratch && ep.partial) {
        long s = slots / rem;
        const long by_depth = (long)K / (8 * DEPTH); // at least eight slices per split
        const long by_mem = (long)(partial_bytes / ((size_t)rem * TM * TN * sizeof(float)));
        if (s > by_depth) s = by_depth;
        if (s > by_mem) s = by_mem;
        if (s >= 2) {
            d = make_dims(M, N, K, TM, TN, (int)s, DEPTH);
            if (d.splits >= 2) { d.full_tiles = (int)(tiles - rem); tail_tiles = (int)rem; }
            else d = make_dims(M, N, K, TM, TN, 1, DEPTH);
        }
    }
    const int rc = narrow ? launch_igemm<64, 256, AL, BL, StoreNCHW<E>, HALF>(ctx, stream, names.t64, al, bl, ep, d, flops)
                          : launch_igemm<128, 128, AL, BL, StoreNCHW<E>, HALF>(ctx, stream, names.t128, al, bl, ep, d, flops);
    if (rc != VDNN_OK || d.splits == 1) return rc;
    if (tail_tiles > 0)
        return launch_reduce_tail_nchw(ctx, stream, ep.out, ep.partial, tail_tiles, d.splits, TM, TN, M, N, d.mtiles, d.full_tiles, ep.bias, ep.opix, ep.relu, ep.gate);
    return launch_reduce_splits_nchw(ctx, stream, ep.out, ep.partial, (size_t)M * N, d.splits, ep.bias, ep.opix, M, ep.relu, ep.gate);
}

// The windowed 3x3 kernel (conv3x3_bf16.h): tiles of 64 rows by 256 pixels, three workgroups resident per compute
// unit (two on float layers, where the kernel holds more registers), the reduction cut at multiples of one filter
// row of a channel block. Splits and tail mode as in launch_by_m. K counts 16-bit values of a row of the filter
// operand (float layers: two per filter element).
constexpr int kWin3SplitPerCU = 2;
template <int MODE, class E>
static int launch_win3x3(vdnn_ctx* ctx, hipStream_t stream, const PassNames& names, const LoadPackedH& al, const Win3x3T<E>& geo, const StoreNCHW<E>& ep,
                         int M, int N, int K, double flops, size_t partial_bytes) {
    constexpr bool SPLIT = sizeof(E) == 4;
    const int TM = W3_TM, TN = W3_TN;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    int splits = 1;
    const size_t out_bytes = (size_t)M * N * sizeof(float);
    if (tiles < 2l * ctx->num_cu && ep.partial) {
        long cap = ((long)K + 4 * W3_DEPTH - 1) / (4 * W3_DEPTH); // at least four filter rows per split
        const long by_mem = (long)(partial_bytes / out_bytes);
        if (cap > by_mem) cap = by_mem;
        splits = choose_splits(tiles, K, cap, ctx->num_cu, out_bytes, 2.0 * TM * TN * KB);
    }
    GemmDims d = make_dims(M, N, K, TM, TN, splits, W3_DEPTH);
    const long slots = (SPLIT ? kWin3SplitPerCU : 3l) * ctx->num_cu;
    const long rem = tiles % slots;
    int tail_tiles = 0;
    if (splits == 1 && tiles > slots && rem > 0 && 2 * rem <= slots && ep.partial) {
        long s = slots / rem;
        const long by_depth = (long)K / (4 * W3_DEPTH);
        const long by_mem = (long)(partial_bytes / ((size_t)rem * TM * TN * sizeof(float)));
        if (s > by_depth) s = by_depth;
        if (s > by_mem) s = by_mem;
        if (s >= 2) {
            d = make_dims(M, N, K, TM, TN, (int)s, W3_DEPTH);
            if (d.splits >= 2) { d.full_tiles = (int)(tiles - rem); tail_tiles = (int)rem; }
            else d = make_dims(M, N, K, TM, TN, 1, W3_DEPTH);
        }
    }
    const long all_tiles = (long)d.mtiles * d.ntiles;
    const long blocks = d.full_tiles > 0 ? d.full_tiles + (all_tiles - d.full_tiles) * d.splits : all_tiles * d.splits;
    if (blocks <= 0 || blocks >= (1l << 31)) { set_error("conv3x3: grid of %ld workgroups out of range", blocks); return VDNN_EINVAL; }
    {
        ProfScope prof(ctx, stream, names.t64, flops, 0.0);
        hipLaunchKernelGGL((conv3x3_bf16_kernel<MODE, E, SPLIT ? kWin3SplitPerCU : 3>), dim3((unsigned)blocks), dim3(NT), 0, stream, al, geo, ep, d);
        VDNN_LAUNCH_CHECK();
    }
    if (d.splits == 1) return VDNN_OK;
    if (tail_tiles > 0)
        return launch_reduce_tail_nchw(ctx, stream, ep.out, ep.partial, tail_tiles, d.splits, TM, TN, M, N, d.mtiles, d.full_tiles, ep.bias, ep.opix, ep.relu, ep.gate);
    return launch_reduce_splits_nchw(ctx, stream, ep.out, ep.partial, (size_t)M * N, d.splits, ep.bias, ep.opix, M, ep.relu, ep.gate);
}

// what the windowed kernel needs: a 3x3 window at stride 1 with one pixel of padding (input and output planes of
// one extent), rows of an even number of pixels, and tiles whose samples fit one descriptor
static bool win3x3_ok(const int R, const int S, int ph, int pw, int sh, int sw, int Hs, int Ws, int OH, int OW, long sample_elems, int elem_bytes = 2) {
    return R == 3 && S == 3 && ph == 1 && pw == 1 && sh == 1 && sw == 1 && Hs == OH && Ws == OW && Ws % 2 == 0 && Ws >= 2 &&
           pixel_tile_span_ok(sample_elems, OH * OW, W3_TN, elem_bytes);
}

static inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

int launch_reduce_splits(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count,
                         int splits, float alpha, int accumulate, const float* bias_j, int ncols, int relu = 0, const float* gate = nullptr);

// forward with the given A loader (128-bit or 32-bit filter loads)
template <class AL, class E>
static int conv_fwd_with(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const AL& al, const E* x, const float* bias, E* y, int relu) {
    StoreNCHW<E> ep{y, bias, g.P * g.Q, ctx->reduce_scratch, relu, nullptr};
    const int M = g.K, N = g.N * g.P * g.Q, K = g.C * g.R * g.S;
    const FastDiv dRS = FastDiv::make(g.R * g.S), dS = FastDiv::make(g.S);
    if (g.R * g.S <= 32) {
        LoadIm2colPix<0, false, E> bl{x, g.H, g.W, g.P, g.Q, g.R, g.S, g.ph, g.pw, g.sh, g.sw, (long)g.C * g.H * g.W, g.N, dRS, dS};
        return launch_by_m(ctx, st, kFwdNames, al, bl, ep, M, N, K);
    }
    LoadIm2colPix<0, true, E> bl{x, g.H, g.W, g.P, g.Q, g.R, g.S, g.ph, g.pw, g.sh, g.sw, (long)g.C * g.H * g.W, g.N, dRS, dS};
    return launch_by_m(ctx, st, kFwdNames, al, bl, ep, M, N, K);
}

template <class AL, class BL>
static int conv_wgrad_with(vdnn_ctx* ctx, hipStream_t st, const AL& al, const BL& bl, const StoreDense<float>& ep, const GemmDims& d, bool narrow) {
    return narrow ? launch_igemm<64, 256>(ctx, st, kBwdFilterNames.t64, al, bl, ep, d)
                  : launch_igemm<128, 128>(ctx, st, kBwdFilterNames.t128, al, bl, ep, d);
}

// Workspace planning has no context at hand: it assumes the 256 compute units of the target part.
constexpr int kPlanningCUs = 256;
constexpr size_t kDefaultStagingBytes = (size_t)64 << 20;
constexpr size_t kMaxWgradWorkspace = (size_t)256 << 20;

// A window that covers the whole unpadded input (the fully connected layers OverFeat writes as
// convolutions, network.cu:449-481) is a dense GEMM over (c,h,w): the implicit-GEMM backward data would
// spend R*S times the work on taps that fall outside the single output pixel.
static bool is_dense(const ConvGeo& g) { return g.P == 1 && g.Q == 1 && g.ph == 0 && g.pw == 0 && g.R == g.H && g.S == g.W; }

static bool packed_fwd_ok(const ConvGeo& g) { return g.R * g.S <= 32 && g.C % KB == 0; }
static bool packed_bwd_data_ok(const ConvGeo& g) {
    return g.C > 4 && g.sh == 1 && g.sw == 1 && g.R * g.S <= 32 && g.K % KB == 0;
}

int launch_bias_grad_final(vdnn_ctx* ctx, hipStream_t st, const float* partial, float* bias, int K, int splits, float alpha, int accumulate);

// The bias gradient as a by-product of backward filter (cudnnConvolutionBackwardBias, layer.cu:631-637, reads the same dy
// as cudnnConvolutionBackwardFilter, :651-660): where the filter-gradient kernel of a shape can add up the dy values it
// streams, it leaves per-channel partial sums in the context's bias staging area and `done` is set; the caller runs the
// ordered final sum. out = (accumulate ? out : 0) + alpha * sum over n, p, q of dy.
struct BiasOut {
    float* out = nullptr;
    float alpha = 1.0f;
    int accumulate = 0;
    bool done = false;
    bool wanted() const { return out != nullptr; }
};
// room for K x parts partial sums in the bias staging area?
static bool bias_parts_fit(const vdnn_ctx* ctx, int K, long parts) {
    return ctx->bias_scratch && parts > 0 && (size_t)K * (size_t)parts * sizeof(float) <= ctx->bias_scratch_bytes;
}

// ---- Winograd F(4x4, 3x3): the perf-optimal mode's forward / backward data of wide 3x3 layers (winograd_f32.h) -----
// Samples are processed in chunks so that the transformed input V and the transformed output M of a chunk stay
// within g_wino_chunk_bytes (512 MiB unless vdnn_conv_winograd_chunk_bytes says otherwise; and each below 2 GiB, the range of the product's descriptors). The plan depends on the shape
// alone: vdnn_conv_workspace_bytes reports it, the pass follows it.
constexpr size_t kWinoChunkBytesDefault = (size_t)512 << 20;
static size_t g_wino_chunk_bytes = kWinoChunkBytesDefault; // vdnn_conv_winograd_chunk_bytes
constexpr int kWinoMinReduced = 128;  // reduced channels from which the product's short reduction pays
struct WinoPlan {
    int rows, cred;        // output rows of the product (forward: K, backward data: C) and its reduction (C / K)
    int th, tw, per;       // tiles per column, per row, per sample
    int nc, chunks;        // samples per chunk, chunks
    long Tpad;             // columns per xi of a full chunk
    size_t u_bytes, v_bytes, m_bytes, total;
};
static bool wino_ok(const ConvGeo& g, bool bwd) {
    const int rows = bwd ? g.C : g.K, cred = bwd ? g.K : g.C;
    return g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W &&
           cred >= kWinoMinReduced && cred % KB == 0 && rows > 64 && g.H >= 4 && g.W >= 4;
}
static WinoPlan wino_plan(const ConvGeo& g, bool bwd) {
    WinoPlan p;
    p.rows = bwd ? g.C : g.K; p.cred = bwd ? g.K : g.C;
    p.th = (g.H + 3) / 4; p.tw = (g.W + 3) / 4; p.per = p.th * p.tw;
    const size_t per_sample = (size_t)(p.rows + p.cred) * WINO_XI * p.per * sizeof(float);
    long most = (long)(g_wino_chunk_bytes / per_sample);
    if (most < 1) most = 1;
    if (most > g.N) most = g.N;
    p.chunks = (int)((g.N + most - 1) / most);
    p.nc = (g.N + p.chunks - 1) / p.chunks;
    p.Tpad = ((long)p.nc * p.per + WINO_TN - 1) / WINO_TN * WINO_TN;
    auto up = [](size_t b) { return (b + 255) / 256 * 256; };
    p.u_bytes = up((size_t)WINO_XI * p.rows * p.cred * sizeof(float));
    p.v_bytes = up((size_t)p.cred * WINO_XI * p.Tpad * sizeof(float));
    p.m_bytes = up((size_t)p.rows * WINO_XI * p.Tpad * sizeof(float));
    p.total = p.u_bytes + p.v_bytes + p.m_bytes;
    return p;
}
static bool wino_plan_ok(const WinoPlan& p) {
    return p.v_bytes < 0x7FFF0000ul && p.m_bytes < 0x7FFF0000ul && (long)WINO_XI * p.Tpad < (1l << 31) && p.rows <= 65535 && p.cred <= 65535;
}

// in: x (forward) or dy (backward data); out: y or dx. Returns VDNN_OK with *taken false when the shape or the
// workspace does not allow the variant.
static int launch_winograd(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, bool bwd, const float* in, const float* w, const float* bias, float* out,
                           int relu, const float* gate, void* workspace, size_t workspace_bytes, bool* taken) {
    *taken = false;
    if (!wino_ok(g, bwd) || !workspace || !aligned16(workspace)) return VDNN_OK;
    const WinoPlan p = wino_plan(g, bwd);
    if (!wino_plan_ok(p) || workspace_bytes < p.total) return VDNN_OK;
    *taken = true;
    float* U = (float*)workspace;
    float* V = (float*)((char*)workspace + p.u_bytes);
    float* Mo = (float*)((char*)workspace + p.u_bytes + p.v_bytes);
    {
        const long total = (long)p.rows * p.cred;
        ProfScope prof(ctx, st, "conv_wino_filter", 0.0, (9.0 + WINO_XI) * 4.0 * (double)total);
        if (bwd) hipLaunchKernelGGL(wino_filter_kernel<true>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, U, p.rows, p.cred);
        else hipLaunchKernelGGL(wino_filter_kernel<false>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, U, p.rows, p.cred);
        VDNN_LAUNCH_CHECK();
    }
    const long plane = (long)g.H * g.W;
    const bool vec = g.W % 4 == 0 && aligned16(in) && aligned16(out) && (!gate || aligned16(gate));
    for (int n0 = 0; n0 < g.N; n0 += p.nc) {
        const int nc = g.N - n0 < p.nc ? g.N - n0 : p.nc;
        const int T = nc * p.per;
        const long Tpad = ((long)T + WINO_TN - 1) / WINO_TN * WINO_TN;
        const unsigned tblocks = (unsigned)((T + 255) / 256), pblocks = (unsigned)((Tpad + 255) / 256);
        {
            const WinoTiles ti{g.H, g.W, p.th, p.tw, p.cred, T, Tpad};
            ProfScope prof(ctx, st, bwd ? "conv_bwd_data_wino_in" : "conv_fwd_wino_in", 0.0, 4.0 * ((double)nc * p.cred * plane + (double)p.cred * WINO_XI * T));
            const float* src = in + (long)n0 * p.cred * plane;
            if (vec) hipLaunchKernelGGL(wino_input_kernel<true>, dim3(pblocks, (unsigned)p.cred), dim3(256), 0, st, src, V, ti);
            else hipLaunchKernelGGL(wino_input_kernel<false>, dim3(pblocks, (unsigned)p.cred), dim3(256), 0, st, src, V, ti);
            VDNN_LAUNCH_CHECK();
        }
        {
            // several column tiles per workgroup, so that all workgroups make about one round of resident ones
            const int mtiles = (p.rows + 127) / 128, tiles_per_xi = (int)(Tpad / WINO_TN);
            const long all_tiles = (long)WINO_XI * mtiles * tiles_per_xi, slots = 3l * ctx->num_cu;
            int group = (int)((all_tiles + slots - 1) / slots);
            // ... unless that round would leave more than a seventh of the places idle (few tiles: 14 x 14 planes,
            // 256 produced rows at 28 x 28): single tiles then, which the hardware hands out as places come free
            if (20 * all_tiles < 17 * (long)group * slots) group = 1;
            if (group < 1) group = 1;
            if (group > tiles_per_xi) group = tiles_per_xi;
            const int groups_per_xi = (tiles_per_xi + group - 1) / group;
            const WinoGemm gm{U, V, Mo, p.rows, p.cred, Tpad, mtiles, tiles_per_xi, group, groups_per_xi};
            // work counted in the transformed domain: 36 products per 4x4 outputs and channel pair
            ProfScope prof(ctx, st, bwd ? "conv_bwd_data_wino_gemm" : "conv_fwd_wino_gemm", 2.0 * p.rows * (double)p.cred * WINO_XI * T, 0.0);
            hipLaunchKernelGGL(wino_gemm_kernel, dim3((unsigned)(WINO_XI * mtiles * groups_per_xi)), dim3(NT), 0, st, gm);
            VDNN_LAUNCH_CHECK();
        }
        {
            const WinoTiles to{g.H, g.W, p.th, p.tw, p.rows, T, Tpad};
            ProfScope prof(ctx, st, bwd ? "conv_bwd_data_wino_out" : "conv_fwd_wino_out", 0.0,
                           4.0 * ((double)p.rows * WINO_XI * T + (double)nc * p.rows * plane * (gate ? 2.0 : 1.0)));
            const long off = (long)n0 * p.rows * plane;
            if (vec) hipLaunchKernelGGL(wino_output_kernel<true>, dim3(tblocks, (unsigned)p.rows), dim3(256), 0, st, Mo, out + off, bias, gate ? gate + off : nullptr, relu, to);
            else hipLaunchKernelGGL(wino_output_kernel<false>, dim3(tblocks, (unsigned)p.rows), dim3(256), 0, st, Mo, out + off, bias, gate ? gate + off : nullptr, relu, to);
            VDNN_LAUNCH_CHECK();
        }
    }
    return VDNN_OK;
}

// Backward filter as Winograd F(3x3, 4x4) (winograd_f32.h): per chunk of samples the transformed input V and the
// transformed output gradient D, then one launch of the tile engine for the 36 products S_xi = D_xi V_xi^t with the
// reduction over the chunk's tiles split so that the grid fills the chip; every (chunk, split) leaves one partial
// result, and a last kernel adds them in order, transforms back and applies alpha. The plan depends on the shape alone.
constexpr size_t kWinoWgradPartialBytes = (size_t)256 << 20;
struct WinoWgradPlan {
    int th, tw, per, nc, chunks, splits;
    long Tpad;
    size_t v_bytes, d_bytes, part_bytes, total;   // part_bytes: one partial result
};
static bool wino_wgrad_ok(const ConvGeo& g) {
    return g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W &&
           g.C >= 128 && g.C % 128 == 0 && g.K > 64 && g.H >= 4 && g.W >= 4;
}
static WinoWgradPlan wino_wgrad_plan(const ConvGeo& g) {
    WinoWgradPlan p;
    p.th = (g.H + 3) / 4; p.tw = (g.W + 3) / 4; p.per = p.th * p.tw;
    const size_t per_sample = (size_t)(g.K + g.C) * WINO_XI * p.per * sizeof(float);
    long most = (long)(g_wino_chunk_bytes / per_sample);
    if (most < 1) most = 1;
    if (most > g.N) most = g.N;
    p.chunks = (int)((g.N + most - 1) / most);
    p.nc = (g.N + p.chunks - 1) / p.chunks;
    p.chunks = (g.N + p.nc - 1) / p.nc;
    p.Tpad = ((long)p.nc * p.per + WINO_TN - 1) / WINO_TN * WINO_TN;
    auto up = [](size_t b) { return (b + 255) / 256 * 256; };
    p.v_bytes = up((size_t)g.C * WINO_XI * p.Tpad * sizeof(float));
    p.d_bytes = up((size_t)g.K * WINO_XI * p.Tpad * sizeof(float));
    p.part_bytes = up((size_t)g.K * WINO_XI * g.C * sizeof(float));
    // splits of a chunk's reduction: one round of resident workgroups, at least eight slices each, partial results within their budget
    const long tiles = (long)WINO_XI * ((g.K + 127) / 128) * (g.C / 128);
    long splits = 3l * kPlanningCUs / tiles;
    const long by_len = p.Tpad / (8 * KB), by_mem = (long)(kWinoWgradPartialBytes / p.part_bytes) / p.chunks;
    if (splits > by_len) splits = by_len;
    if (splits > by_mem) splits = by_mem;
    if (splits < 1) splits = 1;
    // (the launch re-derives the split count from the chunk size through make_dims; this is its upper bound)
    p.splits = (int)splits;
    p.total = p.v_bytes + p.d_bytes + (size_t)p.chunks * p.splits * p.part_bytes;
    return p;
}
static bool wino_wgrad_plan_ok(const WinoWgradPlan& p, const ConvGeo& g) {
    return p.v_bytes < 0x7FFF0000ul && p.d_bytes < 0x7FFF0000ul && (long)WINO_XI * g.C < (1l << 24) && g.K <= 65535 && g.C <= 65535 &&
           (long)p.chunks * p.splits < 4096;
}

static int launch_winograd_wgrad(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const float* x, const float* dy, float* w, float alpha, int accumulate,
                                 void* workspace, size_t workspace_bytes, bool* taken, BiasOut* bias) {
    *taken = false;
    if (!wino_wgrad_ok(g) || !workspace || !aligned16(workspace)) return VDNN_OK;
    const WinoWgradPlan p = wino_wgrad_plan(g);
    if (!wino_wgrad_plan_ok(p, g) || workspace_bytes < p.total) return VDNN_OK;
    *taken = true;
    float* V = (float*)workspace;
    float* D = (float*)((char*)workspace + p.v_bytes);
    float* P = (float*)((char*)workspace + p.v_bytes + p.d_bytes);
    const long part_stride = (long)(p.part_bytes / sizeof(float));
    const long plane = (long)g.H * g.W;
    const bool vec = g.W % 4 == 0 && aligned16(x) && aligned16(dy);
    int nparts = 0;
    // the bias gradient: every workgroup of the dy transform leaves the sum of the values it read
    long bias_parts = 0;
    for (int n0 = 0; n0 < g.N; n0 += p.nc) {
        const int nc = g.N - n0 < p.nc ? g.N - n0 : p.nc;
        bias_parts += (((long)nc * p.per + WINO_TN - 1) / WINO_TN * WINO_TN + 255) / 256;
    }
    const bool with_bias = bias && bias->wanted() && bias_parts < (1 << 20) && bias_parts_fit(ctx, g.K, bias_parts);
    int bias_first = 0;
    for (int n0 = 0; n0 < g.N; n0 += p.nc) {
        const int nc = g.N - n0 < p.nc ? g.N - n0 : p.nc;
        const int T = nc * p.per;
        const long Tpad = ((long)T + WINO_TN - 1) / WINO_TN * WINO_TN;
        const unsigned pblocks = (unsigned)((Tpad + 255) / 256);
        {
            const WinoTiles ti{g.H, g.W, p.th, p.tw, g.C, T, Tpad};
            ProfScope prof(ctx, st, "conv_bwd_filter_wino_in", 0.0, 4.0 * ((double)nc * g.C * plane + (double)g.C * WINO_XI * Tpad));
            const float* src = x + (long)n0 * g.C * plane;
            if (vec) hipLaunchKernelGGL(wino_input_kernel<true>, dim3(pblocks, (unsigned)g.C), dim3(256), 0, st, src, V, ti);
            else hipLaunchKernelGGL(wino_input_kernel<false>, dim3(pblocks, (unsigned)g.C), dim3(256), 0, st, src, V, ti);
            VDNN_LAUNCH_CHECK();
        }
        {
            const WinoTiles td{g.H, g.W, p.th, p.tw, g.K, T, Tpad};
            ProfScope prof(ctx, st, "conv_bwd_filter_wino_dy", 0.0, 4.0 * ((double)nc * g.K * plane + (double)g.K * WINO_XI * Tpad));
            const float* src = dy + (long)n0 * g.K * plane;
            float* bp = with_bias ? ctx->bias_scratch : nullptr;
            if (vec && with_bias) hipLaunchKernelGGL((wino_dy_kernel<true, true>), dim3(pblocks, (unsigned)g.K), dim3(256), 0, st, src, D, td, bp, (int)bias_parts, bias_first);
            else if (vec) hipLaunchKernelGGL((wino_dy_kernel<true, false>), dim3(pblocks, (unsigned)g.K), dim3(256), 0, st, src, D, td, bp, 0, 0);
            else if (with_bias) hipLaunchKernelGGL((wino_dy_kernel<false, true>), dim3(pblocks, (unsigned)g.K), dim3(256), 0, st, src, D, td, bp, (int)bias_parts, bias_first);
            else hipLaunchKernelGGL((wino_dy_kernel<false, false>), dim3(pblocks, (unsigned)g.K), dim3(256), 0, st, src, D, td, bp, 0, 0);
            VDNN_LAUNCH_CHECK();
            bias_first += (int)pblocks;
        }
        {
            GemmDims d = make_dims(g.K, WINO_XI * g.C, (int)Tpad, 128, WINO_TN, p.splits);
            LoadWinoRed<true> al{D, Tpad, g.K, (unsigned)((size_t)g.K * WINO_XI * Tpad * sizeof(float)), g.C, d.mtiles, d.mtiles * d.ntiles, WINO_TN};
            LoadWinoRed<false> bl{V, Tpad, g.C, (unsigned)((size_t)g.C * WINO_XI * Tpad * sizeof(float)), g.C, d.mtiles, d.mtiles * d.ntiles, WINO_TN};
            float* slot = P + (long)nparts * part_stride;
            StoreDense<float> ep{slot, slot, nullptr, (long)WINO_XI * g.C, part_stride, 1.0f, 0, 0, nullptr};
            const int rc = launch_igemm<128, WINO_TN>(ctx, st, "conv_bwd_filter_wino_gemm", al, bl, ep, d, 2.0 * g.K * (double)g.C * WINO_XI * T);
            if (rc != VDNN_OK) return rc;
            nparts += d.splits;
        }
    }
    {
        const long total = (long)g.K * g.C, count = total * WINO_XI;
        ProfScope prof(ctx, st, "conv_bwd_filter_wino_out", 0.0, 4.0 * ((double)nparts * WINO_XI + 18.0) * (double)total);
        if (nparts > 2) {
            // many partial results: summed with one thread per element first
            hipLaunchKernelGGL(wino_wgrad_sum_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st, P, part_stride, nparts, count);
            VDNN_LAUNCH_CHECK();
            nparts = 1;
        }
        hipLaunchKernelGGL(wino_wgrad_out_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, P, part_stride, nparts, w, g.K, g.C, g.C, alpha, accumulate);
        VDNN_LAUNCH_CHECK();
    }
    if (with_bias) {
        const int rc = launch_bias_grad_final(ctx, st, ctx->bias_scratch, bias->out, g.K, (int)bias_parts, bias->alpha, bias->accumulate);
        if (rc != VDNN_OK) return rc;
        bias->done = true;
    }
    return VDNN_OK;
}

// The bfloat16 engine's filter operand lives at the front of the staging area (rounded and re-laid-out by a
// small kernel before every use: the master copy changes every step); what is left holds partial sums.
static bool half_engine_ok(const vdnn_ctx* ctx, int reduced_channels, int RS, size_t filter_elems) {
    return reduced_channels % KH == 0 && RS <= 32 && ctx->reduce_scratch && filter_elems * 2 + (16u << 20) <= ctx->reduce_scratch_bytes;
}

static int launch_pack_filter_bf16(vdnn_ctx* ctx, hipStream_t st, const float* w, unsigned short* packed, int rows, int Cred, int RS,
                                   int row_stride, int red_stride) {
    const long total = (long)rows * Cred * RS;
    ProfScope prof(ctx, st, "conv_pack_filter", 0.0, 6.0 * (double)total);
    hipLaunchKernelGGL(pack_filter_tap_bf16_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, packed, rows, Cred, RS,
                       row_stride, red_stride, total);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

// Takes bytes from the front of the context's staging area for as long as the object lives; everything that
// uses the staging area meanwhile (partial sums, intermediate products) sees the remainder.
struct StagingCarve {
    vdnn_ctx* ctx;
    float* base = nullptr;
    size_t total = 0;
    bool taken = false;
    explicit StagingCarve(vdnn_ctx* c) : ctx(c) {}
    void* take(size_t bytes) {
        base = ctx->reduce_scratch; total = ctx->reduce_scratch_bytes; taken = true;
        const size_t t = (bytes + 255) / 256 * 256;
        ctx->reduce_scratch = (float*)((char*)base + t);
        ctx->reduce_scratch_bytes = total - t;
        return base;
    }
    ~StagingCarve() { if (taken) { ctx->reduce_scratch = base; ctx->reduce_scratch_bytes = total; } }
};

// Room for a re-laid-out filter bank at the front of the staging area: only if nothing was taken from it yet and at
// least half of it stays for the partial sums of split reductions (the largest need of a layer is a round of partial
// tiles: 768 x 64 KB). Null otherwise.
static float* packed_filter_place(vdnn_ctx* ctx, StagingCarve& carve, size_t bytes) {
    if (carve.taken || !ctx->reduce_scratch || 2 * ((bytes + 255) / 256 * 256) > ctx->reduce_scratch_bytes) return nullptr;
    return (float*)carve.take(bytes);
}

__global__ void __launch_bounds__(256) round_filter_bf16_kernel(const float* __restrict__ w, float* __restrict__ out, long count) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i < count) out[i] = round_to_bf16_value(w[i]);
}

// Layers with bfloat16 activations multiply the filter rounded to bfloat16 (two bfloat16 factors per product)
// on every route. Routes outside the bfloat16 engine read a rounded float copy, made here at the front of the
// staging area. Returns null when it does not fit.
static const float* rounded_filter_copy(vdnn_ctx* ctx, hipStream_t st, StagingCarve& carve, const float* w, size_t count) {
    if (!ctx->reduce_scratch || count * sizeof(float) + (8u << 20) > ctx->reduce_scratch_bytes) return nullptr;
    float* wr = (float*)carve.take(count * sizeof(float));
    hipLaunchKernelGGL(round_filter_bf16_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, st, w, wr, (long)count);
    return wr;
}

// forward / backward data of a bfloat16 layer on the bfloat16 matrix cores; MODE as in LoadIm2colPixTapH
template <int MODE>
static int conv_half_engine(vdnn_ctx* ctx, hipStream_t st, const PassNames& names, const float* w, int rows, int Cred, int RS, int row_stride, int red_stride,
                            const LoadIm2colPix<MODE, false, bf16_t>& pix, StoreNCHW<bf16_t> ep, int N, double flops) {
    const size_t filter_elems = (size_t)rows * Cred * RS;
    unsigned short* packed = (unsigned short*)ctx->reduce_scratch;
    const size_t taken = (filter_elems * 2 + 255) / 256 * 256;
    const int rc = launch_pack_filter_bf16(ctx, st, w, packed, rows, Cred, RS, row_stride, red_stride);
    if (rc != VDNN_OK) return rc;
    ep.partial = (float*)((char*)ctx->reduce_scratch + taken);
    LoadPackedH al{packed, (long)Cred * RS, rows, (unsigned)(filter_elems * 2)};
    // 3x3 at stride 1 with padding 1: one staged window per filter row serves its three taps
    if (win3x3_ok(pix.R, pix.S, pix.ph, pix.pw, pix.sh, pix.sw, pix.Hs, pix.Ws, pix.OH, pix.OW, pix.sample_elems)) {
        const Win3x3 geo{pix.src, pix.Hs, pix.Ws, pix.sample_elems, pix.sample_elems * pix.nsamples, pix.nsamples};
        return launch_win3x3<MODE, bf16_t>(ctx, st, MODE == 0 ? kFwdWin3Names : kBwdDataWin3Names, al, geo, ep, rows, N, Cred * RS, flops, ctx->reduce_scratch_bytes - taken);
    }
    // a pixel pair per lane where the pairs of an output row are contiguous in the input
    if (pix.OW % 2 == 0 && pix.S <= 16 && pix.Ws >= pix.S && pix.Ws > pix.pw + 1 && (MODE == 1 || pix.sw == 1)) {
        LoadIm2colPixTapH2<MODE> bl2{pix};
        return launch_by_m<LoadPackedH, LoadIm2colPixTapH2<MODE>, bf16_t, true>(ctx, st, names, al, bl2, ep, rows, N, Cred * RS, flops, ctx->reduce_scratch_bytes - taken);
    }
    LoadIm2colPixTapH<MODE> bl{pix};
    return launch_by_m<LoadPackedH, LoadIm2colPixTapH<MODE>, bf16_t, true>(ctx, st, names, al, bl, ep, rows, N, Cred * RS, flops, ctx->reduce_scratch_bytes - taken);
}

// ---- perf-optimal mode, float layers: 3x3 / stride 1 / padding 1 on the bfloat16 matrix cores ------------------
// Every float operand as two bfloat16 parts, three matrix instructions per product (conv3x3_bf16.h): forward and
// backward data through the windowed kernel, the split filter bank (as many bytes as the filter) in the workspace.
// Which variant the perf-optimal mode takes where both apply: 0 = this one, through the windowed kernel or the general
// engine (faster than Winograd on every VGG16 / AlexNet / OverFeat layer, closer to the exact result, no transformed
// tensors; backward filter of the layers it does not take stays Winograd's), 1 = Winograd. vdnn_conv_perf_variant.
static int g_perf_variant = 0;

// MODE 0: rows = output channels, reduced = input channels; MODE 1: rows = input channels, reduced = output channels
static bool split3x3_ok(const ConvGeo& g, int mode) {
    const int reduced = mode == 0 ? g.C : g.K, rows = mode == 0 ? g.K : g.C;
    const long sample = mode == 0 ? (long)g.C * g.H * g.W : (long)g.K * g.P * g.Q;
    return reduced % 16 == 0 && g.C > 4 && (long)rows * reduced * 9 * 4 < (1l << 31) &&
           win3x3_ok(g.R, g.S, g.ph, g.pw, g.sh, g.sw, g.H, g.W, g.P, g.Q, sample, 4);
}

template <int MODE>
static int launch_split3x3(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const float* src, const float* w, const StoreNCHW<float>& ep,
                           void* workspace, size_t workspace_bytes, bool* taken) {
    *taken = false;
    const int rows = MODE == 0 ? g.K : g.C, reduced = MODE == 0 ? g.C : g.K;
    const size_t bank = (size_t)rows * reduced * 9 * 4;
    if (!split3x3_ok(g, MODE) || !workspace || workspace_bytes < bank || !aligned16(workspace)) return VDNN_OK;
    *taken = true;
    unsigned short* packed = (unsigned short*)workspace;
    {
        const long total = (long)rows * reduced * 9;
        ProfScope prof(ctx, st, "conv_pack_filter", 0.0, 8.0 * (double)total);
        hipLaunchKernelGGL(pack_filter_split_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, packed, rows, reduced, 9,
                           MODE == 0 ? g.C * 9 : 9, MODE == 0 ? 9 : g.C * 9, total);
        VDNN_LAUNCH_CHECK();
    }
    const long sample = MODE == 0 ? (long)g.C * g.H * g.W : (long)g.K * g.P * g.Q;
    const LoadPackedH al{packed, (long)reduced * 18, rows, (unsigned)bank};
    const Win3x3T<float> geo{src, g.H, g.W, sample, sample * g.N, g.N};
    return launch_win3x3<MODE, float>(ctx, st, MODE == 0 ? kFwdSplitNames : kBwdDataSplitNames, al, geo, ep, rows, g.N * g.H * g.W, reduced * 18,
                                      2.0 * g.N * (double)g.K * g.C * 9 * g.P * g.Q, ctx->reduce_scratch_bytes);
}

// The same products through the general bfloat16 engine, for stride-1 layers the windowed kernel does not take (other
// windows than 3x3, no or other padding, planes with odd rows): forward (MODE 0) and backward data (MODE 1), at most 32
// taps, reduced channels a multiple of 16.
static bool split_general_ok(const ConvGeo& g, int mode) {
    const int reduced = mode == 0 ? g.C : g.K, rows = mode == 0 ? g.K : g.C;
    return g.R * g.S <= 32 && reduced % 16 == 0 && g.C > 4 && (mode == 0 || (g.sh == 1 && g.sw == 1)) &&
           (long)rows * reduced * g.R * g.S * 4 < (1l << 31);
}

static const PassNames kFwdSplitGenNames{"conv_fwd_splitgen_64x256", "conv_fwd_splitgen_128x128"};
static const PassNames kBwdDataSplitGenNames{"conv_bwd_data_splitgen_64x256", "conv_bwd_data_splitgen_128x128"};

template <int MODE>
static int launch_split_general(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const float* src, const float* w, const StoreNCHW<float>& ep,
                                void* workspace, size_t workspace_bytes, bool* taken) {
    *taken = false;
    const int RS = g.R * g.S;
    const int rows = MODE == 0 ? g.K : g.C, reduced = MODE == 0 ? g.C : g.K;
    const size_t bank = (size_t)rows * reduced * RS * 4;
    if (!split_general_ok(g, MODE) || !workspace || workspace_bytes < bank || !aligned16(workspace)) return VDNN_OK;
    const long sample = MODE == 0 ? (long)g.C * g.H * g.W : (long)g.K * g.P * g.Q;
    const int opix = MODE == 0 ? g.P * g.Q : g.H * g.W;
    if (!pixel_tile_span_ok(sample, opix, 256, 4)) return VDNN_OK;
    *taken = true;
    unsigned short* packed = (unsigned short*)workspace;
    {
        const long total = (long)rows * reduced * RS;
        ProfScope prof(ctx, st, "conv_pack_filter", 0.0, 8.0 * (double)total);
        hipLaunchKernelGGL(pack_filter_split_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, packed, rows, reduced, RS,
                           MODE == 0 ? g.C * RS : RS, MODE == 0 ? RS : g.C * RS, total);
        VDNN_LAUNCH_CHECK();
    }
    const LoadPackedH al{packed, (long)reduced * RS * 2, rows, (unsigned)bank};
    const FastDiv dRS = FastDiv::make(RS), dS = FastDiv::make(g.S);
    const double flops = 2.0 * g.N * (double)g.K * g.C * RS * g.P * g.Q;
    if (MODE == 0) {
        const LoadIm2colPixTapS<MODE> bl{{src, g.H, g.W, g.P, g.Q, g.R, g.S, g.ph, g.pw, g.sh, g.sw, sample, g.N, dRS, dS}};
        return launch_by_m<LoadPackedH, LoadIm2colPixTapS<MODE>, float, true>(ctx, st, kFwdSplitGenNames, al, bl, ep, rows, g.N * opix, reduced * RS * 2, flops);
    }
    const LoadIm2colPixTapS<MODE> bl{{src, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, 1, 1, sample, g.N, dRS, dS}};
    return launch_by_m<LoadPackedH, LoadIm2colPixTapS<MODE>, float, true>(ctx, st, kBwdDataSplitGenNames, al, bl, ep, rows, g.N * opix, reduced * RS * 2, flops);
}

static int launch_pack_filter(vdnn_ctx* ctx, hipStream_t st, const float* w, float* packed, int rows, int Cred, int RS,
                              int row_stride, int red_stride) {
    const long total = (long)rows * Cred * RS;
    ProfScope prof(ctx, st, "conv_pack_filter", 0.0, 8.0 * (double)total);
    hipLaunchKernelGGL(pack_filter_tap_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, w, packed, rows, Cred, RS,
                       row_stride, red_stride, total);
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

// Workgroups of wgrad3x3_bf16_kernel that are resident on a compute unit (its launch bounds).
constexpr int kWgrad3PerCU = 2;


static bool wgrad3x3_ok(const ConvGeo& g) {
    return g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W &&
           g.W % 4 == 0 && g.W >= 16 && (g.H * g.W) % 8 == 0 && g.C % WG3_CH == 0; // a slice wraps at most two image rows
}

// One filter row, 64 input channels and 128 (64) output channels per workgroup; the pixel reduction is split so
// that one round of workgroups fills the chip, as far as the staging area holds the partial sums.
static int launch_wgrad3x3(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const bf16_t* x, const bf16_t* dy, float* w, float alpha, int accumulate,
                           float* staging, size_t staging_bytes, bool* taken, BiasOut* bias) {
    *taken = false;
    const int M = g.K, N = g.C * 9, PQ = g.H * g.W;
    const long Kred = (long)g.N * PQ;
    const bool narrow = M <= 64;
    const int TM = narrow ? 64 : 128;
    const int mtiles = (M + TM - 1) / TM, ntiles = 3 * (g.C / WG3_CH);
    const long tiles = (long)mtiles * ntiles;
    const size_t out_bytes = (size_t)M * N * sizeof(float);
    long splits = (long)kWgrad3PerCU * ctx->num_cu / tiles;
    const long by_len = Kred / (8 * KH); // at least eight slices per split
    const long by_mem = staging ? (long)(staging_bytes / out_bytes) : 1;
    if (splits > by_len) splits = by_len;
    if (splits > by_mem) splits = by_mem;
    if (splits < 1) splits = 1;
    GemmDims d = make_dims(M, N, (int)Kred, TM, 3 * WG3_CH, (int)splits, KH);
    d.mtiles = mtiles; d.ntiles = ntiles;
    const long nspan = d.kchunk / PQ + 2;
    if (nspan * g.K * PQ * 2 >= (long)MAX_SUM_RANGE || nspan * g.C * PQ * 2 >= (long)MAX_SUM_RANGE) return VDNN_OK; // not taken
    if (d.splits > 1 && !staging) return VDNN_OK;
    const long blocks = tiles * d.splits;
    if (blocks <= 0 || blocks >= (1l << 31)) return VDNN_OK;
    *taken = true;
    const bool with_bias = bias && bias->wanted() && bias_parts_fit(ctx, g.K, d.splits);
    const Wgrad3x3 geo{dy, x, g.N, g.K, g.C, g.H, g.W, w, staging, (long)M * N, alpha, accumulate, with_bias ? ctx->bias_scratch : nullptr, d.splits};
    {
        ProfScope prof(ctx, st, narrow ? kBwdFilterWin3Names.t64 : kBwdFilterWin3Names.t128, 2.0 * M * (double)N * (double)Kred, 0.0);
        const bool halfrow = g.W % 8 != 0 || g.W < KH; // the general variant: groups across two image rows, two row wraps per slice
        if (narrow && halfrow) hipLaunchKernelGGL((wgrad3x3_bf16_kernel<32, true>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else if (narrow) hipLaunchKernelGGL((wgrad3x3_bf16_kernel<32, false>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else if (halfrow) hipLaunchKernelGGL((wgrad3x3_bf16_kernel<64, true>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else hipLaunchKernelGGL((wgrad3x3_bf16_kernel<64, false>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        VDNN_LAUNCH_CHECK();
    }
    if (with_bias) {
        const int rc = launch_bias_grad_final(ctx, st, ctx->bias_scratch, bias->out, g.K, d.splits, bias->alpha, bias->accumulate);
        if (rc != VDNN_OK) return rc;
        bias->done = true;
    }
    if (d.splits > 1) return launch_reduce_splits_tap(ctx, st, w, staging, (size_t)M * N, d.splits, alpha, accumulate, g.C, 9);
    return VDNN_OK;
}

// The perf-optimal float counterpart of launch_wgrad3x3 (wgrad3x3_split.h): the same tiles and splits, slices of 16 pixels.
static int launch_wgrad3x3_split(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const float* x, const float* dy, float* w, float alpha, int accumulate,
                                 float* staging, size_t staging_bytes, bool* taken, BiasOut* bias) {
    *taken = false;
    const int M = g.K, N = g.C * 9, PQ = g.H * g.W;
    const long Kred = (long)g.N * PQ;
    const bool narrow = M <= 64;
    const int TM = narrow ? 64 : 128;
    const int mtiles = (M + TM - 1) / TM, ntiles = 3 * (g.C / WG3_CH);
    const long tiles = (long)mtiles * ntiles;
    const size_t out_bytes = (size_t)M * N * sizeof(float);
    const long slots = (long)kWgrad3PerCU * ctx->num_cu;
    // as many rounds of workgroups as the tiles alone need, each filled by the splits
    const long rounds = (tiles + slots - 1) / slots;
    long splits = rounds * slots / tiles;
    const long by_len = Kred / (16 * WG3S_SLICE); // at least sixteen slices per split
    const long by_mem = staging ? (long)(staging_bytes / out_bytes) : 1;
    if (splits > by_len) splits = by_len;
    if (splits > by_mem) splits = by_mem;
    if (splits < 1) splits = 1;
    GemmDims d = make_dims(M, N, (int)Kred, TM, 3 * WG3_CH, (int)splits, WG3S_SLICE);
    d.mtiles = mtiles; d.ntiles = ntiles;
    const long nspan = d.kchunk / PQ + 2;
    if (nspan * g.K * PQ * 4 >= (long)MAX_SUM_RANGE || nspan * g.C * PQ * 4 >= (long)MAX_SUM_RANGE) return VDNN_OK; // not taken
    if (d.splits > 1 && !staging) return VDNN_OK;
    const long blocks = tiles * d.splits;
    if (blocks <= 0 || blocks >= (1l << 31)) return VDNN_OK;
    *taken = true;
    const bool with_bias = bias && bias->wanted() && bias_parts_fit(ctx, g.K, d.splits);
    const Wgrad3x3S geo{dy, x, g.N, g.K, g.C, g.H, g.W, w, staging, (long)M * N, alpha, accumulate, with_bias ? ctx->bias_scratch : nullptr, d.splits};
    {
        ProfScope prof(ctx, st, narrow ? "conv_bwd_filter_split_64x192" : "conv_bwd_filter_split_128x192", 2.0 * M * (double)N * (double)Kred, 0.0);
        const bool halfrow = g.W % 8 != 0; // groups of eight pixels across two image rows
        if (narrow && halfrow) hipLaunchKernelGGL((wgrad3x3_split_kernel<32, true>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else if (narrow) hipLaunchKernelGGL((wgrad3x3_split_kernel<32, false>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else if (halfrow) hipLaunchKernelGGL((wgrad3x3_split_kernel<64, true>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else hipLaunchKernelGGL((wgrad3x3_split_kernel<64, false>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        VDNN_LAUNCH_CHECK();
    }
    if (with_bias) {
        const int rc = launch_bias_grad_final(ctx, st, ctx->bias_scratch, bias->out, g.K, d.splits, bias->alpha, bias->accumulate);
        if (rc != VDNN_OK) return rc;
        bias->done = true;
    }
    if (d.splits > 1) return launch_reduce_splits_tap(ctx, st, w, staging, (size_t)M * N, d.splits, alpha, accumulate, g.C, 9);
    return VDNN_OK;
}

// Workgroups of wgrad3x3_f32_kernel that are resident on a compute unit (its launch bounds; three, at 167 registers, measured 10 % slower).
constexpr int kWgrad3FPerCU = 2;

static bool wgrad3x3_f32_ok(const ConvGeo& g) {
    return g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W &&
           g.W % 2 == 0 && g.W >= 14 && (g.H * g.W) % 4 == 0 && g.C % WG3F_CH == 0; // a slice wraps at most two image rows
}

// The float counterpart of launch_wgrad3x3.
static int launch_wgrad3x3_f32(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const float* x, const float* dy, float* w, float alpha, int accumulate,
                               float* staging, size_t staging_bytes, bool* taken, BiasOut* bias) {
    *taken = false;
    const int M = g.K, N = g.C * 9, PQ = g.H * g.W;
    const long Kred = (long)g.N * PQ;
    const bool narrow = M <= 64;
    const int TM = narrow ? 64 : 128;
    const int mtiles = (M + TM - 1) / TM, ntiles = 3 * (g.C / WG3F_CH);
    const long tiles = (long)mtiles * ntiles;
    const size_t out_bytes = (size_t)M * N * sizeof(float);
    const long slots = (long)kWgrad3FPerCU * ctx->num_cu;
    // as many rounds of workgroups as the tiles alone need, each filled by the splits
    const long rounds = (tiles + slots - 1) / slots;
    long splits = rounds * slots / tiles;
    const long by_len = Kred / (8 * KB); // at least eight slices per split
    const long by_mem = staging ? (long)(staging_bytes / out_bytes) : 1;
    if (splits > by_len) splits = by_len;
    if (splits > by_mem) splits = by_mem;
    if (splits < 1) splits = 1;
    GemmDims d = make_dims(M, N, (int)Kred, TM, 3 * WG3F_CH, (int)splits, KB);
    d.mtiles = mtiles; d.ntiles = ntiles;
    const long nspan = d.kchunk / PQ + 2;
    if (nspan * g.K * PQ * 4 >= (long)MAX_SUM_RANGE || nspan * g.C * PQ * 4 >= (long)MAX_SUM_RANGE) return VDNN_OK; // not taken
    if (d.splits > 1 && !staging) return VDNN_OK;
    const long blocks = tiles * d.splits;
    if (blocks <= 0 || blocks >= (1l << 31)) return VDNN_OK;
    *taken = true;
    const bool with_bias = bias && bias->wanted() && bias_parts_fit(ctx, g.K, d.splits);
    const Wgrad3x3F geo{dy, x, g.N, g.K, g.C, g.H, g.W, w, staging, (long)M * N, alpha, accumulate, with_bias ? ctx->bias_scratch : nullptr, d.splits};
    {
        ProfScope prof(ctx, st, narrow ? kBwdFilterRow3Names.t64 : kBwdFilterRow3Names.t128, 2.0 * M * (double)N * (double)Kred, 0.0);
        const bool halfrow = g.W % 4 != 0 || g.W < KB; // the general variant: groups across two image rows, two row wraps per slice
        if (narrow && halfrow) hipLaunchKernelGGL((wgrad3x3_f32_kernel<32, true>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else if (narrow) hipLaunchKernelGGL((wgrad3x3_f32_kernel<32, false>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else if (halfrow) hipLaunchKernelGGL((wgrad3x3_f32_kernel<64, true>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        else hipLaunchKernelGGL((wgrad3x3_f32_kernel<64, false>), dim3((unsigned)blocks), dim3(NT), 0, st, geo, d);
        VDNN_LAUNCH_CHECK();
    }
    if (with_bias) {
        const int rc = launch_bias_grad_final(ctx, st, ctx->bias_scratch, bias->out, g.K, d.splits, bias->alpha, bias->accumulate);
        if (rc != VDNN_OK) return rc;
        bias->done = true;
    }
    if (d.splits > 1) return launch_reduce_splits_tap(ctx, st, w, staging, (size_t)M * N, d.splits, alpha, accumulate, g.C, 9);
    return VDNN_OK;
}

// Forward of a 3x3 / stride 1 / padding 1 layer with at most four input and 64 output channels: wavefronts stream over
// the pixels, three workgroups per compute unit.
static bool fwd_smallc3x3_ok(const ConvGeo& g, size_t elem_bytes) {
    return g.C <= 4 && g.K <= 64 && g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W &&
           (long)g.N * g.C * g.H * g.W * (long)elem_bytes < (1l << 31) && (long)g.N * g.K * g.H * g.W * (long)elem_bytes < (1l << 31);
}
template <class E>
static int launch_fwd_smallc3x3(vdnn_ctx* ctx, hipStream_t st, const ConvGeo& g, const E* x, const float* w, const float* bias, E* y, int relu) {
    // two blocks of 32 pixels per unit where that makes a store a whole 128-byte line (two-byte elements: 0.47 -> 0.38 ms
    // for VGG16's first layer at batch 128); with floats a block's 32 pixels are a line already and two measured the same
    const int up = sizeof(E) == 2 ? 2 : 1;
    const long units = ((long)g.N * g.H * g.W + 32 * up - 1) / (32 * up);
    long blocks = (units + 3) / 4;
    // bound by its stores from two workgroups per unit on (four measured 20 % slower); with two blocks per unit the
    // registers allow two
    const long resident = (up == 2 ? 2l : 3l) * ctx->num_cu;
    if (blocks > resident) blocks = resident;
    ProfScope prof(ctx, st, "conv_fwd_smallc", 2.0 * g.K * 9.0 * g.C * (double)g.N * g.H * g.W, 0.0);
#define VDNN_FWD_SMALLC_UP(CC, RB, UP) hipLaunchKernelGGL((conv_fwd_smallc3x3_kernel<CC, RB, UP, E>), dim3((unsigned)blocks), dim3(256), 0, st, x, w, bias, y, g.N, g.K, g.H, g.W, relu)
#define VDNN_FWD_SMALLC(CC)                                                                         \
    do {                                                                                            \
        if (g.K <= 32) { if (up == 2) VDNN_FWD_SMALLC_UP(CC, 1, 2); else VDNN_FWD_SMALLC_UP(CC, 1, 1); } \
        else { if (up == 2) VDNN_FWD_SMALLC_UP(CC, 2, 2); else VDNN_FWD_SMALLC_UP(CC, 2, 1); }           \
    } while (0)
    switch (g.C) {
    case 1: VDNN_FWD_SMALLC(1); break;
    case 2: VDNN_FWD_SMALLC(2); break;
    case 3: VDNN_FWD_SMALLC(3); break;
    default: VDNN_FWD_SMALLC(4); break;
    }
#undef VDNN_FWD_SMALLC_UP
#undef VDNN_FWD_SMALLC
    VDNN_LAUNCH_CHECK();
    return VDNN_OK;
}

// Backward filter of a bfloat16 3x3 / stride 1 / padding 1 layer with the vector loaders: picks the instantiation
// for the number of taps per tile and the pixel group (combinations whose loads would mix taps do not exist).
template <int TM, int TN, int NTAP, int G>
static int launch_wgrad_vec_one(vdnn_ctx* ctx, hipStream_t st, const char* name, const LoadDyRedVecH<8>& al, const LoadIm2colRedTapVecH<1, 4>& geo,
                                const StoreFilterTap& ep, const GemmDims& d) {
    if constexpr ((TN / NTAP) % (NT / (KH / G)) != 0) {
        set_error("backward filter: %d taps per %d-column tile with groups of %d pixels", NTAP, TN, G);
        return VDNN_EINVAL;
    } else {
        LoadIm2colRedTapVecH<NTAP, G> bl{geo.x, geo.N, geo.C, geo.H, geo.W, geo.ncols, geo.kchunk, geo.Ktot, geo.divC};
        return launch_igemm<TM, TN, LoadDyRedVecH<8>, LoadIm2colRedTapVecH<NTAP, G>, StoreFilterTap, true>(ctx, st, name, al, bl, ep, d);
    }
}
template <int TM, int TN>
static int launch_wgrad_vec(vdnn_ctx* ctx, hipStream_t st, const char* name, const LoadDyRedVecH<8>& al, const LoadIm2colRedTapVecH<1, 4>& geo,
                            const StoreFilterTap& ep, const GemmDims& d, int ntap, int group) {
    if (group != 4) { set_error("backward filter: groups of %d pixels", group); return VDNN_EINVAL; }
    if (ntap == 1) return launch_wgrad_vec_one<TM, TN, 1, 4>(ctx, st, name, al, geo, ep, d);
    if (ntap == 2) return launch_wgrad_vec_one<TM, TN, 2, 4>(ctx, st, name, al, geo, ep, d);
    return launch_wgrad_vec_one<TM, TN, 4, 4>(ctx, st, name, al, geo, ep, d);
}

} // namespace vdnn

using namespace vdnn;

template <class E>
static int conv_fwd_impl(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                         const E* x, const float* w, const float* bias, E* y,
                         void* workspace, size_t workspace_bytes, int relu) {
    VDNN_KERNEL_PROLOGUE(ctx);
    ConvGeo g;
    VDNN_REQUIRE(shape && geo_from_shape(shape, g), "unsupported convolution geometry");
    VDNN_REQUIRE(x && w && y, "null tensor");
    if (is_dense(g))
        return relu ? vdnn_fc_fwd_relu(ctx, stream, g.N, g.C * g.H * g.W, g.K, x, w, bias, y)
                    : vdnn_fc_fwd(ctx, stream, g.N, g.C * g.H * g.W, g.K, x, w, bias, y);
    VDNN_REQUIRE(pixel_tile_span_ok((long)g.C * g.H * g.W, g.P * g.Q, 256, (int)sizeof(E)), "input samples too large for one tile's descriptor");
    hipStream_t st = stream_of(ctx, stream);
    const int K = g.C * g.R * g.S;
    const unsigned wbytes = (unsigned)((long)g.K * K * 4);
    if constexpr (sizeof(E) == 2) {
        if (half_engine_ok(ctx, g.C, g.R * g.S, (size_t)g.K * K)) {
            const int RS = g.R * g.S;
            LoadIm2colPix<0, false, bf16_t> pix{x, g.H, g.W, g.P, g.Q, g.R, g.S, g.ph, g.pw, g.sh, g.sw, (long)g.C * g.H * g.W, g.N,
                                               FastDiv::make(RS), FastDiv::make(g.S)};
            StoreNCHW<bf16_t> ep{y, bias, g.P * g.Q, nullptr, relu, nullptr};
            return conv_half_engine<0>(ctx, st, kFwdHalfNames, w, g.K, g.C, RS, g.C * RS, RS, pix, ep, g.N * g.P * g.Q,
                                       2.0 * g.N * (double)g.K * K * g.P * g.Q);
        }
    }
    StagingCarve carve(ctx);
    if constexpr (sizeof(E) == 2) {
        w = rounded_filter_copy(ctx, st, carve, w, (size_t)g.K * K);
        VDNN_REQUIRE(w != nullptr, "filter too large for the staging area (bfloat16 layer outside the bfloat16 engine)");
        VDNN_LAUNCH_CHECK();
    }
    if (fwd_smallc3x3_ok(g, sizeof(E))) return launch_fwd_smallc3x3<E>(ctx, st, g, x, w, bias, y, relu);
    if constexpr (sizeof(E) == 4) {
        if (algo_mode == 1) {
            // perf-optimal: 3x3 layers on the bfloat16 matrix cores, or as Winograd F(4x4, 3x3), through the workspace
            bool taken = false;
            if (g_perf_variant == 0) {
                const StoreNCHW<float> eps{y, bias, g.P * g.Q, ctx->reduce_scratch, relu, nullptr};
                const int rc = launch_split3x3<0>(ctx, st, g, x, w, eps, workspace, workspace_bytes, &taken);
                if (taken || rc != VDNN_OK) return rc;
                const int rcg = launch_split_general<0>(ctx, st, g, x, w, eps, workspace, workspace_bytes, &taken);
                if (taken || rcg != VDNN_OK) return rcg;
            }
            const int rc = launch_winograd(ctx, st, g, false, x, w, bias, y, relu, nullptr, workspace, workspace_bytes, &taken);
            if (taken || rc != VDNN_OK) return rc;
        }
    }
    if (g.R * g.S <= 32 && g.C % KB == 0) {
        // blocked tap-major reduction: one slice = one tap x 16 input channels
        const int RS = g.R * g.S;
        LoadIm2colPixTap<0, E> bl{{x, g.H, g.W, g.P, g.Q, g.R, g.S, g.ph, g.pw, g.sh, g.sw, (long)g.C * g.H * g.W, g.N,
                                FastDiv::make(RS), FastDiv::make(g.S)}};
        // The filter bank re-laid-out in the blocked tap-major order is a dense operand read with 128-bit loads (in the
        // master copy's order a slice's sixteen channels of one tap lie R*S floats apart). Perf-optimal: in the
        // workspace. Memory-optimal: at the front of the context's staging area, where it leaves room for the partial sums.
        const bool in_workspace = algo_mode == 1 && workspace && workspace_bytes >= wbytes && aligned16(workspace);
        float* packed = in_workspace ? (float*)workspace : packed_filter_place(ctx, carve, wbytes);
        StoreNCHW<E> ep{y, bias, g.P * g.Q, ctx->reduce_scratch, relu, nullptr};
        if (packed) {
            const int rc = launch_pack_filter(ctx, st, w, packed, g.K, g.C, RS, g.C * RS, RS);
            if (rc != VDNN_OK) return rc;
            LoadDenseRed<true> alp{packed, (long)K, g.K, wbytes};
            return launch_by_m(ctx, st, in_workspace ? kFwdPackedNames : kFwdNames, alp, bl, ep, g.K, g.N * g.P * g.Q, K);
        }
        LoadFilterTap<false> al{w, g.C * RS, RS, g.K, RS, wbytes, FastDiv::make(RS)};
        return launch_by_m(ctx, st, kFwdNames, al, bl, ep, g.K, g.N * g.P * g.Q, K);
    }
    if (K % 4 == 0 && aligned16(w)) {
        LoadDenseRed<true> al{w, (long)K, g.K, wbytes};
        return conv_fwd_with(ctx, st, g, al, x, bias, y, relu);
    }
    LoadDenseRed<false> al{w, (long)K, g.K, wbytes};
    return conv_fwd_with(ctx, st, g, al, x, bias, y, relu);
}

// The kernels that a stride-1 layer with more than four input channels takes store through StoreNCHW or one of the
// split reductions: a lane reads the gate's element before it writes the gradient's, and no kernel reads the layer's
// input otherwise. (Layers that are one dense product are left out: their filter gradient is as large as the filter.)
static bool conv_bwd_data_in_place_ok(const ConvGeo& g) {
    return g.sh == 1 && g.sw == 1 && g.C > 4 && !is_dense(g);
}

template <class E>
static int conv_bwd_data_impl(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                              const E* dy, const float* w, E* dx,
                              void* workspace, size_t workspace_bytes, const E* gate) {
    VDNN_KERNEL_PROLOGUE(ctx);
    ConvGeo g;
    VDNN_REQUIRE(shape && geo_from_shape(shape, g), "unsupported convolution geometry");
    VDNN_REQUIRE(dy && w && dx, "null tensor");
    VDNN_REQUIRE((const void*)dx != (const void*)dy, "the input gradient cannot be written over the output gradient");
    VDNN_REQUIRE((const void*)dx != (const void*)gate || conv_bwd_data_in_place_ok(g),
                 "the input gradient may be written over the gating input only where vdnn_conv_bwd_data_in_place_ok says so");
    if (is_dense(g))
        return gate ? vdnn_fc_bwd_data_relu(ctx, stream, g.N, g.C * g.H * g.W, g.K, dy, w, gate, dx)
                    : vdnn_fc_bwd_data(ctx, stream, g.N, g.C * g.H * g.W, g.K, dy, w, dx);
    hipStream_t st = stream_of(ctx, stream);
    StagingCarve carve(ctx);
    const bool few_channels = g.C <= 4 && g.R * g.S <= SMALLC_MAXTAPS && !gate; // the vector-ALU kernels have no gated store
    bool half_engine = false;
    if constexpr (sizeof(E) == 2) {
        half_engine = !few_channels && g.sh == 1 && g.sw == 1 && half_engine_ok(ctx, g.K, g.R * g.S, (size_t)g.K * g.C * g.R * g.S);
        if (!half_engine) {
            w = rounded_filter_copy(ctx, st, carve, w, (size_t)g.K * g.C * g.R * g.S);
            VDNN_REQUIRE(w != nullptr, "filter too large for the staging area (bfloat16 layer outside the bfloat16 engine)");
            VDNN_LAUNCH_CHECK();
        }
    }
    if (few_channels) {
        if ((g.sh != 1 || g.sw != 1) && ctx->reduce_scratch && ctx->reduce_scratch_bytes >= (size_t)g.C * g.R * g.S * g.P * g.Q * sizeof(float) &&
                 pixel_tile_span_ok((long)g.K * g.P * g.Q, g.P * g.Q, 256, (int)sizeof(E))) {
            // Strided layer with few input channels (the 11x11 stride-4 first layers): its three or four
            // output rows cannot fill a matrix tile, so the products are formed once, as a 1x1 convolution
            // with C*R*S output channels over dy on the matrix cores, into the staging area, and gathered
            // into dx by a second kernel; as many samples at a time as the staging area holds.
            const int RS = g.R * g.S, CRS = g.C * RS, PQ = g.P * g.Q;
            const size_t per_sample = (size_t)CRS * PQ * sizeof(float);
            int nb = (int)(ctx->reduce_scratch_bytes / per_sample);
            if (nb > g.N) nb = g.N;
            float* T = ctx->reduce_scratch;
            LoadFilterT alt{w, CRS, 1, (unsigned)((long)g.K * CRS * 4), FastDiv::make(1)};
            for (int n0 = 0; n0 < g.N; n0 += nb) {
                const int nc = g.N - n0 < nb ? g.N - n0 : nb;
                LoadIm2colPix<0, false, E> bl{dy + (long)n0 * g.K * PQ, g.P, g.Q, g.P, g.Q, 1, 1, 0, 0, 1, 1, (long)g.K * PQ, nc,
                                              FastDiv::make(1), FastDiv::make(1)};
                StoreNCHW<float> ept{T, nullptr, PQ, nullptr, 0, nullptr};
                const int rc = launch_by_m(ctx, st, kBwdDataNames, alt, bl, ept, CRS, nc * PQ, g.K, 2.0 * nc * (double)g.K * CRS * PQ);
                if (rc != VDNN_OK) return rc;
                ConvGeo gc = g; gc.N = nc;
                const long total = (long)nc * g.C * g.H * g.W;
                ProfScope gather(ctx, st, "conv_bwd_data_gather", 0.0, (double)per_sample * nc + (double)total * sizeof(E));
                hipLaunchKernelGGL(conv_bwd_data_gather_taps_kernel<E>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st,
                                   T, dx + (long)n0 * g.C * g.H * g.W, gc, total);
                VDNN_LAUNCH_CHECK();
            }
            return VDNN_OK;
        }
        const long total = (long)g.N * g.H * g.W;
        const long blocks = (total + 255) / 256;
        VDNN_REQUIRE(blocks < (1l << 31), "grid too large");
        ProfScope prof(ctx, st, "conv_bwd_data_smallc", 2.0 * g.C * (double)g.N * g.P * g.Q * g.K * g.R * g.S, 0.0);
        const bool s1_3x3 = g.sh == 1 && g.sw == 1 && g.R == 3 && g.S == 3;
        // 3x3, padding 1, at most three input and 64 output channels: the products once, on the matrix cores, row by row
        if (s1_3x3 && g.C <= 3 && g.K <= 64 && g.ph == 1 && g.pw == 1 && g.P == g.H && g.Q == g.W &&
            (long)g.K * g.P * g.Q * (long)sizeof(E) < (long)MAX_SUM_RANGE) {
            // about three workgroups per compute unit, strips of at least eight image rows
            const int cblocks = (g.W + BDS_EMIT - 1) / BDS_EMIT;
            int strips = (int)((3l * ctx->num_cu + (long)g.N * cblocks - 1) / ((long)g.N * cblocks));
            int rows = (g.H + strips - 1) / strips;
            if (rows < 8) rows = 8;
            if (rows > g.H) rows = g.H;
            strips = (g.H + rows - 1) / rows;
            const dim3 grid((unsigned)(g.N * strips * cblocks));
            if (g.C == 1) hipLaunchKernelGGL((conv_bwd_data_smallc3x3_mfma_kernel<1, E>), grid, dim3(256), 0, st, dy, w, dx, g.N, g.K, g.H, g.W, rows);
            else if (g.C == 2) hipLaunchKernelGGL((conv_bwd_data_smallc3x3_mfma_kernel<2, E>), grid, dim3(256), 0, st, dy, w, dx, g.N, g.K, g.H, g.W, rows);
            else hipLaunchKernelGGL((conv_bwd_data_smallc3x3_mfma_kernel<3, E>), grid, dim3(256), 0, st, dy, w, dx, g.N, g.K, g.H, g.W, rows);
            VDNN_LAUNCH_CHECK();
            return VDNN_OK;
        }
        if (s1_3x3 && g.C == 3) hipLaunchKernelGGL((conv_bwd_data_smallc_s1_kernel<3, 3, 3, E>), dim3((unsigned)blocks), dim3(256), 0, st, dy, w, dx, g);
        else if (s1_3x3 && g.C == 4) hipLaunchKernelGGL((conv_bwd_data_smallc_s1_kernel<3, 3, 4, E>), dim3((unsigned)blocks), dim3(256), 0, st, dy, w, dx, g);
        else if (g.sh == 1 && g.sw == 1) hipLaunchKernelGGL(conv_bwd_data_smallc_kernel<E>, dim3((unsigned)blocks), dim3(256), 0, st, dy, w, dx, g);
        else {
            // one workgroup per 256 pixels of one (sample, residue class modulo the stride)
            const int Ht = (g.H + g.ph + g.sh - 1) / g.sh, Wt = (g.W + g.pw + g.sw - 1) / g.sw;
            const long per_class = ((long)Ht * Wt + 255) / 256;
            const long sblocks = per_class * g.sh * g.sw * g.N;
            VDNN_REQUIRE(sblocks < (1l << 31), "grid too large");
            hipLaunchKernelGGL(conv_bwd_data_smallc_strided_kernel<E>, dim3((unsigned)sblocks), dim3(256), 0, st, dy, w, dx, g, Ht, Wt, (int)per_class);
        }
        VDNN_LAUNCH_CHECK();
        return VDNN_OK;
    }
    VDNN_REQUIRE(pixel_tile_span_ok((long)g.K * g.P * g.Q, g.H * g.W, 256, (int)sizeof(E)), "output-gradient samples too large for one tile's descriptor");
    if constexpr (sizeof(E) == 4) {
        if (algo_mode == 1) {
            bool taken = false;
            if (g_perf_variant == 0) {
                const StoreNCHW<float> eps{dx, nullptr, g.H * g.W, ctx->reduce_scratch, 0, gate};
                const int rc = launch_split3x3<1>(ctx, st, g, dy, w, eps, workspace, workspace_bytes, &taken);
                if (taken || rc != VDNN_OK) return rc;
                const int rcg = launch_split_general<1>(ctx, st, g, dy, w, eps, workspace, workspace_bytes, &taken);
                if (taken || rcg != VDNN_OK) return rcg;
            }
            const int rc = launch_winograd(ctx, st, g, true, dy, w, nullptr, dx, 0, gate, workspace, workspace_bytes, &taken);
            if (taken || rc != VDNN_OK) return rc;
        }
    }
    const int RS = g.R * g.S;
    LoadFilterT al{w, g.C, RS, (unsigned)((long)g.K * g.C * RS * 4), FastDiv::make(RS)};
    StoreNCHW<E> ep{dx, nullptr, g.H * g.W, ctx->reduce_scratch, 0, gate};
    const int M = g.C, N = g.N * g.H * g.W, K = g.K * RS;
    const FastDiv dRS = FastDiv::make(RS), dS = FastDiv::make(g.S);
    const long sample = (long)g.K * g.P * g.Q;
    const double flops = 2.0 * g.N * (double)g.K * g.C * RS * g.P * g.Q;
    if constexpr (sizeof(E) == 2) {
        if (half_engine) {
            LoadIm2colPix<1, false, bf16_t> pix{dy, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, 1, 1, sample, g.N, dRS, dS};
            return conv_half_engine<1>(ctx, st, kBwdDataHalfNames, w, g.C, g.K, RS, RS, g.C * RS, pix, ep, N, flops);
        }
    }
    if (g.sh == 1 && g.sw == 1) {
        if (RS <= 32 && g.K % KB == 0) {
            // blocked tap-major reduction: one slice = one tap x 16 output channels
            const unsigned wbytes = (unsigned)((long)g.K * g.C * RS * 4);
            LoadIm2colPixTap<1, E> bl{{dy, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, 1, 1, sample, g.N, dRS, dS}};
            const bool in_workspace = algo_mode == 1 && workspace && workspace_bytes >= wbytes && aligned16(workspace);
            float* packed = in_workspace ? (float*)workspace : packed_filter_place(ctx, carve, wbytes); // [c][(kb*RS + tap)*16 + l]
            if (packed) {
                ep.partial = ctx->reduce_scratch; // (behind the filter bank, if that lies in the staging area)
                const int rc = launch_pack_filter(ctx, st, w, packed, g.C, g.K, RS, RS, g.C * RS);
                if (rc != VDNN_OK) return rc;
                LoadDenseRed<true> alp{packed, (long)K, g.C, wbytes};
                return launch_by_m(ctx, st, in_workspace ? kBwdDataPackedNames : kBwdDataNames, alp, bl, ep, M, N, K, flops);
            }
            LoadFilterTap<true> alt{w, RS, g.C * RS, g.C, RS, wbytes, dRS};
            return launch_by_m(ctx, st, kBwdDataNames, alt, bl, ep, M, N, K, flops);
        }
        if (RS <= 32) {
            LoadIm2colPix<1, false, E> bl{dy, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, 1, 1, sample, g.N, dRS, dS};
            return launch_by_m(ctx, st, kBwdDataNames, al, bl, ep, M, N, K, flops);
        }
        LoadIm2colPix<1, true, E> bl{dy, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, 1, 1, sample, g.N, dRS, dS};
        return launch_by_m(ctx, st, kBwdDataNames, al, bl, ep, M, N, K, flops);
    }
    LoadIm2colPix<2, true, E> bl{dy, g.P, g.Q, g.H, g.W, g.R, g.S, g.ph, g.pw, g.sh, g.sw, sample, g.N, dRS, dS};
    return launch_by_m(ctx, st, kBwdDataNames, al, bl, ep, M, N, K, flops);
}

// out = (accumulate ? out : 0) + alpha * dW; the bias gradient too where the chosen kernel can (bias->done)
template <class E>
static int conv_bwd_filter_core(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                                const E* x, const E* dy, float* w, float alpha, int accumulate,
                                void* workspace, size_t workspace_bytes, BiasOut* bias) {
    VDNN_KERNEL_PROLOGUE(ctx);
    ConvGeo g;
    VDNN_REQUIRE(shape && geo_from_shape(shape, g), "unsupported convolution geometry");
    VDNN_REQUIRE(x && dy && w, "null tensor");
    if (is_dense(g))
        return accumulate ? vdnn_fc_bwd_weight_sgd(ctx, stream, g.N, g.C * g.H * g.W, g.K, x, dy, w, alpha)
                          : vdnn_fc_bwd_weight(ctx, stream, g.N, g.C * g.H * g.W, g.K, x, dy, w);
    hipStream_t st = stream_of(ctx, stream);
    const int M = g.K, N = g.C * g.R * g.S, PQ = g.P * g.Q, RS = g.R * g.S;
    const long Kred = (long)g.N * PQ;
    VDNN_REQUIRE(Kred < (1l << 31), "reduction too long");
    VDNN_REQUIRE((long)(PQ + KB) * PQ < (1l << 32), "output plane too large for the pixel cursor's exact division");
    if constexpr (sizeof(E) == 4) {
        if (algo_mode == 1) {
            // perf-optimal: 3x3 layers on the bfloat16 matrix cores (partial sums in the staging area, or in the workspace
            // if that is larger), or as Winograd F(3x3, 4x4) through the workspace
            bool taken = false;
            if (g_perf_variant == 0 && wgrad3x3_ok(g)) {
                float* staging = ctx->reduce_scratch;
                size_t staging_bytes = ctx->reduce_scratch_bytes;
                if (workspace && workspace_bytes > staging_bytes && aligned16(workspace)) { staging = (float*)workspace; staging_bytes = workspace_bytes; }
                const int rcs = launch_wgrad3x3_split(ctx, st, g, x, dy, w, alpha, accumulate, staging, staging_bytes, &taken, bias);
                if (taken || rcs != VDNN_OK) return rcs;
            }
            const int rc = launch_winograd_wgrad(ctx, st, g, x, dy, w, alpha, accumulate, workspace, workspace_bytes, &taken, bias);
            if (taken || rc != VDNN_OK) return rc;
        }
    }
    if (g.C <= 3 && g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W && g.W % 4 == 0 && g.W >= KB &&
        ctx->reduce_scratch) {
        // few input channels, rows of whole groups of four pixels: dy streamed once through the matrix cores, then the ordered split sum
        const int mtiles = (g.K + 63) / 64;
        const size_t out_bytes = (size_t)M * N * sizeof(float);
        long splits = 3l * ctx->num_cu / mtiles;
        const long by_len = Kred / (4 * WSC_SLICE), by_mem = (long)(ctx->reduce_scratch_bytes / out_bytes);
        if (splits > by_len) splits = by_len;
        if (splits > by_mem) splits = by_mem;
        if (splits < 1) splits = 1;
        long kchunk = (Kred + splits - 1) / splits;
        kchunk = (kchunk + WSC_SLICE - 1) / WSC_SLICE * WSC_SLICE;
        splits = (Kred + kchunk - 1) / kchunk;
        const long nspan = kchunk / PQ + 2;
        if (PQ >= WSC_SLICE && nspan * g.K * PQ * (long)sizeof(E) < (long)MAX_SUM_RANGE && nspan * g.C * PQ * (long)sizeof(E) < (long)MAX_SUM_RANGE) {
            const bool with_bias = bias && bias->wanted() && bias_parts_fit(ctx, g.K, splits);
            const WgradSmallC geo{dy, x, g.N, g.K, g.H, g.W, ctx->reduce_scratch, (int)kchunk, with_bias ? ctx->bias_scratch : nullptr, (int)splits};
            {
                ProfScope prof(ctx, st, "conv_bwd_filter_smallc", 2.0 * (double)M * N * (double)Kred, 0.0);
                const dim3 grid((unsigned)(mtiles * splits));
                switch (g.C) {
                case 1: hipLaunchKernelGGL((wgrad_smallc3x3_mfma_kernel<1, E>), grid, dim3(NT), 0, st, geo); break;
                case 2: hipLaunchKernelGGL((wgrad_smallc3x3_mfma_kernel<2, E>), grid, dim3(NT), 0, st, geo); break;
                default: hipLaunchKernelGGL((wgrad_smallc3x3_mfma_kernel<3, E>), grid, dim3(NT), 0, st, geo); break;
                }
                VDNN_LAUNCH_CHECK();
            }
            if (with_bias) {
                const int rcb = launch_bias_grad_final(ctx, st, ctx->bias_scratch, bias->out, g.K, (int)splits, bias->alpha, bias->accumulate);
                if (rcb != VDNN_OK) return rcb;
                bias->done = true;
            }
            return launch_reduce_splits(ctx, st, w, ctx->reduce_scratch, (size_t)M * N, (int)splits, alpha, accumulate, nullptr, 0);
        }
    }
    if (g.C <= 4 && g.R == 3 && g.S == 3 && g.K % 4 == 0 && ctx->reduce_scratch) {
        // few input channels: vector-ALU kernel over chunks of output pixels, then the ordered chunk sum
        const long total = Kred;
        const size_t out_bytes = (size_t)M * N * sizeof(float);
        long chunks = (total + 256 * 96 - 1) / (256 * 96);
        const long by_mem = (long)(ctx->reduce_scratch_bytes / out_bytes);
        if (chunks > by_mem) chunks = by_mem;
        if (chunks < 1) chunks = 1;
        long per = (total + chunks - 1) / chunks;
        per = (per + 255) / 256 * 256;
        chunks = (total + per - 1) / per;
        const long blocks = chunks * (g.K / 4);
        VDNN_REQUIRE(blocks < (1l << 31), "grid too large");
        const PixelStep step{256 / PQ, (256 % PQ) / g.Q, (256 % PQ) % g.Q};
        float* staging = ctx->reduce_scratch;
        {
            ProfScope prof(ctx, st, "conv_bwd_filter_smallc", 2.0 * (double)M * N * (double)Kred, 0.0);
            switch (g.C) {
            case 1: hipLaunchKernelGGL((conv_bwd_filter_smallc3x3_kernel<1, 4, E>), dim3((unsigned)blocks), dim3(256), 0, st, dy, x, staging, g, per, step); break;
            case 2: hipLaunchKernelGGL((conv_bwd_filter_smallc3x3_kernel<2, 4, E>), dim3((unsigned)blocks), dim3(256), 0, st, dy, x, staging, g, per, step); break;
            case 3: hipLaunchKernelGGL((conv_bwd_filter_smallc3x3_kernel<3, 4, E>), dim3((unsigned)blocks), dim3(256), 0, st, dy, x, staging, g, per, step); break;
            default: hipLaunchKernelGGL((conv_bwd_filter_smallc3x3_kernel<4, 4, E>), dim3((unsigned)blocks), dim3(256), 0, st, dy, x, staging, g, per, step); break;
            }
            VDNN_LAUNCH_CHECK();
        }
        return launch_reduce_splits(ctx, st, w, staging, (size_t)M * N, (int)chunks, alpha, accumulate, nullptr, 0);
    }
    // Split the (n,p,q) reduction so the grid fills the chip; partial sums go to a staging area and
    // are added in split order by a second kernel (no floating-point atomics).
    const bool narrow = M <= 64;
    const int TM = narrow ? 64 : 128, TN = narrow ? 256 : 128;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    float* staging = ctx->reduce_scratch;
    size_t staging_bytes = ctx->reduce_scratch_bytes;
    if (workspace && workspace_bytes > staging_bytes) { staging = (float*)workspace; staging_bytes = workspace_bytes; }
    const size_t out_bytes = (size_t)M * N * sizeof(float);
    long cap = (Kred + 4 * KB - 1) / (4 * KB); // at least four slices per split
    const long by_mem = staging ? (long)(staging_bytes / out_bytes) : 1;
    if (cap > by_mem) cap = by_mem;
    const int want = choose_splits(tiles, Kred, cap, ctx->num_cu, out_bytes, 2.0 * TM * TN * KB);
    GemmDims d = make_dims(M, N, (int)Kred, TM, TN, want);
    // one split's samples of dy and of x are addressed through one descriptor with summed offsets
    const long nspan = d.kchunk / PQ + 2;
    VDNN_REQUIRE(nspan * g.K * PQ * (long)sizeof(E) < (long)MAX_SUM_RANGE && nspan * g.C * g.H * g.W * (long)sizeof(E) < (long)MAX_SUM_RANGE,
                 "samples of one reduction split too large for one descriptor");
    StoreDense<float> ep{w, staging, nullptr, (long)N, (long)M * N, alpha, accumulate};
    const FastDiv dRS = FastDiv::make(RS), dS = FastDiv::make(g.S), dQ = FastDiv::make(g.Q), dPQ = FastDiv::make(PQ);
    const bool vec = PQ % 4 == 0 && aligned16(dy); // bf16: four elements are 8 bytes, covered by the same test
    // tap-major column order when the tile's columns fall into whole groups of channels with one tap each
    const int tile_n = narrow ? 256 : 128;
    const int ntap = g.C % tile_n == 0 ? 1 : (g.C % (tile_n / 2) == 0 ? 2 : (g.C % (tile_n / 4) == 0 ? 4 : 0));
    if constexpr (sizeof(E) == 2) {
        // bfloat16 activations: both factors of every product are bfloat16 already
        if (wgrad3x3_ok(g)) { // loads of eight pixels take any alignment of the tensors
            bool taken = false;
            const int rcw = launch_wgrad3x3(ctx, st, g, x, dy, w, alpha, accumulate, staging, staging_bytes, &taken, bias);
            if (taken || rcw != VDNN_OK) return rcw;
        }
        if (vec && ntap != 0 && PQ >= KH && 3 * g.Q >= KH && g.Q % 2 == 0 && ((uintptr_t)x & 3) == 0 && staging) {
            long caph = (Kred + 4 * KH - 1) / (4 * KH);
            if (caph > by_mem) caph = by_mem;
            const int wanth = choose_splits(tiles, Kred, caph, ctx->num_cu, out_bytes, 2.0 * TM * TN * KB);
            GemmDims dh = make_dims(M, N, (int)Kred, TM, TN, wanth, KH);
            const long nspanh = dh.kchunk / PQ + 2;
            if (nspanh * g.K * PQ * 2 < (long)MAX_SUM_RANGE && nspanh * g.C * g.H * g.W * 2 < (long)MAX_SUM_RANGE) {
                const FastDiv dC = FastDiv::make(g.C);
                StoreFilterTap ept{w, staging, g.C, RS, (long)M * N, alpha, accumulate, dC};
                LoadDyRedIncH al{dy, g.N, g.K, PQ, dh.kchunk, dh.K};
                int rch;
                // 3x3, stride 1, padding 1, channel counts the kernel above does not take: a tap's im2col operand is the plane
                // shifted by a constant, fetched in groups of four pixels when the image rows are whole groups
                const int vg = g.W % 4 == 0 ? 4 : 0;
                const int tap_cols = tile_n / ntap; // columns of the tile that share a tap
                if (g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W && PQ % 8 == 0 &&
                    vg != 0 && tap_cols % (8 * vg) == 0 && (long)g.C * g.H * g.W * 2 < (long)MAX_SUM_RANGE) {
                    LoadDyRedVecH<8> alv{dy, g.N, g.K, PQ, dh.kchunk, dh.K};
                    LoadIm2colRedTapVecH<1, 4> geo{x, g.N, g.C, g.H, g.W, N, dh.kchunk, dh.K, dC};
                    rch = narrow ? launch_wgrad_vec<64, 256>(ctx, st, kBwdFilterHalfNames.t64, alv, geo, ept, dh, ntap, vg)
                                 : launch_wgrad_vec<128, 128>(ctx, st, kBwdFilterHalfNames.t128, alv, geo, ept, dh, ntap, vg);
                    if (rch != VDNN_OK) return rch;
                    if (dh.splits > 1) return launch_reduce_splits_tap(ctx, st, w, staging, (size_t)M * N, dh.splits, alpha, accumulate, g.C, RS);
                    return VDNN_OK;
                }
#define VDNN_WGRAD_TAP_H(NTAP)                                                                                              \
                do {                                                                                                        \
                    if (g.sw == 1) {                                                                                        \
                        LoadIm2colRedTapH<NTAP, true> bl{x, g.N, g.C, g.H, g.W, g.R, g.S, g.P, g.Q, g.ph, g.pw, g.sh, g.sw, N, dh.kchunk, dh.K, dC, dS}; \
                        rch = narrow ? launch_igemm<64, 256, LoadDyRedIncH, LoadIm2colRedTapH<NTAP, true>, StoreFilterTap, true>(ctx, st, kBwdFilterHalfNames.t64, al, bl, ept, dh) \
                                     : launch_igemm<128, 128, LoadDyRedIncH, LoadIm2colRedTapH<NTAP, true>, StoreFilterTap, true>(ctx, st, kBwdFilterHalfNames.t128, al, bl, ept, dh); \
                        break;                                                                                              \
                    }                                                                                                       \
                    LoadIm2colRedTapH<NTAP> bl{x, g.N, g.C, g.H, g.W, g.R, g.S, g.P, g.Q, g.ph, g.pw, g.sh, g.sw, N, dh.kchunk, dh.K, dC, dS}; \
                    rch = narrow ? launch_igemm<64, 256, LoadDyRedIncH, LoadIm2colRedTapH<NTAP>, StoreFilterTap, true>(ctx, st, kBwdFilterHalfNames.t64, al, bl, ept, dh) \
                                 : launch_igemm<128, 128, LoadDyRedIncH, LoadIm2colRedTapH<NTAP>, StoreFilterTap, true>(ctx, st, kBwdFilterHalfNames.t128, al, bl, ept, dh); \
                } while (0)
                if (ntap == 1) VDNN_WGRAD_TAP_H(1);
                else if (ntap == 2) VDNN_WGRAD_TAP_H(2);
                else VDNN_WGRAD_TAP_H(4);
#undef VDNN_WGRAD_TAP_H
                if (rch != VDNN_OK) return rch;
                if (dh.splits > 1) return launch_reduce_splits_tap(ctx, st, w, staging, (size_t)M * N, dh.splits, alpha, accumulate, g.C, RS);
                return VDNN_OK;
            }
        }
    }
    if constexpr (sizeof(E) == 4) {
        // 3x3, stride 1, padding 1: one filter row and 64 input channels per workgroup, one fetch for three taps
        if (wgrad3x3_f32_ok(g)) { // loads of four pixels take any alignment of the tensors
            bool taken = false;
            const int rcw = launch_wgrad3x3_f32(ctx, st, g, x, dy, w, alpha, accumulate, staging, staging_bytes, &taken, bias);
            if (taken || rcw != VDNN_OK) return rcw;
        }
    }
    if (vec && ntap != 0 && PQ >= KB && 2 * g.Q >= KB) {
        const FastDiv dC = FastDiv::make(g.C);
        StoreFilterTap ept{w, staging, g.C, RS, (long)M * N, alpha, accumulate, dC};
        LoadDyRedInc<E> al{dy, g.N, g.K, PQ, d.kchunk, d.K};
        int rc2;
#define VDNN_WGRAD_TAP(NTAP)                                                                                                \
        do {                                                                                                                \
            LoadIm2colRedTap<NTAP, E> bl{x, g.N, g.C, g.H, g.W, g.R, g.S, g.P, g.Q, g.ph, g.pw, g.sh, g.sw, N, d.kchunk, d.K, dC, dS}; \
            rc2 = narrow ? launch_igemm<64, 256>(ctx, st, kBwdFilterNames.t64, al, bl, ept, d)                               \
                         : launch_igemm<128, 128>(ctx, st, kBwdFilterNames.t128, al, bl, ept, d);                            \
        } while (0)
        if (ntap == 1) VDNN_WGRAD_TAP(1);
        else if (ntap == 2) VDNN_WGRAD_TAP(2);
        else VDNN_WGRAD_TAP(4);
#undef VDNN_WGRAD_TAP
        if (rc2 != VDNN_OK) return rc2;
        if (d.splits > 1) return launch_reduce_splits_tap(ctx, st, w, staging, (size_t)M * N, d.splits, alpha, accumulate, g.C, RS);
        return VDNN_OK;
    }
    const bool big = RS > 32;
    int rc;
#define VDNN_WGRAD(VEC, BIG)                                                                                              \
    do {                                                                                                                  \
        LoadDyRed<VEC, E> al{dy, g.N, g.K, PQ, d.kchunk, d.K, dPQ};                                                               \
        LoadIm2colRed<BIG, E> bl{x, g.N, g.C, g.H, g.W, g.R, g.S, g.P, g.Q, g.ph, g.pw, g.sh, g.sw, N, d.kchunk, d.K, dRS, dS, dQ, dPQ}; \
        rc = conv_wgrad_with(ctx, st, al, bl, ep, d, narrow);                                                             \
    } while (0)
    if (vec && !big) VDNN_WGRAD(true, false);
    else if (vec && big) VDNN_WGRAD(true, true);
    else if (!vec && !big) VDNN_WGRAD(false, false);
    else VDNN_WGRAD(false, true);
#undef VDNN_WGRAD
    if (rc != VDNN_OK) return rc;
    if (d.splits > 1) return launch_reduce_splits(ctx, st, w, staging, (size_t)M * N, d.splits, alpha, accumulate, nullptr, 0);
    return VDNN_OK;
}

// Backward filter, and with `bias` the bias gradient as well: inside the filter-gradient kernel where the shape's kernel
// can, otherwise by the kernels of vdnn_conv_bwd_bias[_sgd] behind it on the same stream.
template <class E>
static int conv_bwd_filter_impl(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                                const E* x, const E* dy, float* w, float alpha, int accumulate,
                                void* workspace, size_t workspace_bytes, BiasOut* bias = nullptr) {
    const int rc = conv_bwd_filter_core<E>(ctx, stream, shape, algo_mode, x, dy, w, alpha, accumulate, workspace, workspace_bytes, bias);
    if (rc != VDNN_OK || !bias || !bias->wanted() || bias->done || ctx->plan_only) return rc;
    return bias->accumulate ? vdnn_conv_bwd_bias_sgd(ctx, stream, shape, dy, bias->out, bias->alpha)
                            : vdnn_conv_bwd_bias(ctx, stream, shape, dy, bias->out);
}

// Does backward filter of this shape add up the bias gradient inside its own kernel? (The shapes' dispatch above: the
// Winograd variant - float activations only -, the first-layer kernel, the filter-row kernels.)
static bool bwd_filter_sums_bias(const ConvGeo& g, int algo_mode, int dtype) {
    if (is_dense(g)) return false;
    const bool f32 = dtype == VDNN_DTYPE_F32;
    if (f32 && algo_mode == 1 && wino_wgrad_ok(g) && wino_wgrad_plan_ok(wino_wgrad_plan(g), g)) return true;
    if (g.C <= 3 && g.R == 3 && g.S == 3 && g.ph == 1 && g.pw == 1 && g.sh == 1 && g.sw == 1 && g.P == g.H && g.Q == g.W && g.W % 4 == 0 && g.W >= KB &&
        g.P * g.Q >= WSC_SLICE)
        return true;
    return g.C > 4 && (f32 ? wgrad3x3_f32_ok(g) : wgrad3x3_ok(g));
}

extern "C" {

int vdnn_conv_bwd_filter_sums_bias(const vdnn_shape_t* shape, int algo_mode, int dtype) {
    ConvGeo g;
    return shape && geo_from_shape(shape, g) && bwd_filter_sums_bias(g, algo_mode, dtype);
}

int vdnn_conv_bwd_filter_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                                  const void* x, const void* dy, float* w, float* bias, float alpha,
                                  void* workspace, size_t workspace_bytes) {
    VDNN_REQUIRE(bias != nullptr, "null bias");
    BiasOut b; b.out = bias; b.alpha = alpha; b.accumulate = 1;
    return VDNN_BY_ACT(ctx, conv_bwd_filter_impl<float>(ctx, stream, shape, algo_mode, (const float*)x, (const float*)dy, w, alpha, 1, workspace, workspace_bytes, &b),
                       conv_bwd_filter_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)x, (const bf16_t*)dy, w, alpha, 1, workspace, workspace_bytes, &b));
}

int vdnn_conv_bwd_filter_bias(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                              const void* x, const void* dy, float* dw, float* db, void* workspace, size_t workspace_bytes) {
    VDNN_REQUIRE(db != nullptr, "null bias gradient");
    BiasOut b; b.out = db; b.alpha = 1.0f; b.accumulate = 0;
    return VDNN_BY_ACT(ctx, conv_bwd_filter_impl<float>(ctx, stream, shape, algo_mode, (const float*)x, (const float*)dy, dw, 1.0f, 0, workspace, workspace_bytes, &b),
                       conv_bwd_filter_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)x, (const bf16_t*)dy, dw, 1.0f, 0, workspace, workspace_bytes, &b));
}

int vdnn_conv_bwd_filter_then_bias_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                                       const void* x, const void* dy, float* dw, float* bias, float alpha,
                                       void* workspace, size_t workspace_bytes) {
    VDNN_REQUIRE(bias != nullptr, "null bias");
    BiasOut b; b.out = bias; b.alpha = alpha; b.accumulate = 1;
    return VDNN_BY_ACT(ctx, conv_bwd_filter_impl<float>(ctx, stream, shape, algo_mode, (const float*)x, (const float*)dy, dw, 1.0f, 0, workspace, workspace_bytes, &b),
                       conv_bwd_filter_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)x, (const bf16_t*)dy, dw, 1.0f, 0, workspace, workspace_bytes, &b));
}

size_t vdnn_conv_winograd_chunk_bytes(size_t bytes) {
    const size_t before = g_wino_chunk_bytes;
    g_wino_chunk_bytes = bytes ? bytes : kWinoChunkBytesDefault;
    return before;
}

int vdnn_conv_perf_variant(int variant) {
    const int before = g_perf_variant;
    if (variant == 0 || variant == 1) g_perf_variant = variant;
    return before;
}

size_t vdnn_conv_workspace_bytes(const vdnn_shape_t* shape, int algo_mode, int pass) {
    return vdnn_conv_workspace_bytes_dtype(shape, algo_mode, pass, VDNN_DTYPE_F32);
}

size_t vdnn_conv_workspace_bytes_dtype(const vdnn_shape_t* shape, int algo_mode, int pass, int dtype) {
    ConvGeo g;
    if (!shape || !geo_from_shape(shape, g)) return 0;
    if (algo_mode == 0 /* VDNN_MEMORY_OPT_ALGO */ || is_dense(g)) return 0;
    // Perf-optimal mode, float activations: forward and backward data on the bfloat16 matrix cores take the filter bank
    // split into bfloat16 parts (the filter's bytes); under the Winograd variant, and for backward filter where the default
    // has no kernel, wide 3x3 layers take the transformed filter, input and output of a chunk of samples; other layers
    // re-lay the filter bank out for 128-bit operand loads; backward filter otherwise takes a staging area large enough
    // for the split count that fills the chip.
    const int RS = g.R * g.S;
    const size_t filter_bytes = (size_t)g.K * g.C * RS * sizeof(float);
    if (dtype == VDNN_DTYPE_F32 && pass != 2 && g_perf_variant == 0 && (split3x3_ok(g, pass) || split_general_ok(g, pass))) return filter_bytes;
    if (dtype == VDNN_DTYPE_F32 && pass != 2 && wino_ok(g, pass == 1)) {
        const WinoPlan p = wino_plan(g, pass == 1);
        if (wino_plan_ok(p)) return p.total;
    }
    const bool split_wgrad = dtype == VDNN_DTYPE_F32 && pass == 2 && g_perf_variant == 0 && wgrad3x3_ok(g);
    if (dtype == VDNN_DTYPE_F32 && pass == 2 && !split_wgrad && wino_wgrad_ok(g)) {
        const WinoWgradPlan p = wino_wgrad_plan(g);
        if (wino_wgrad_plan_ok(p, g)) return p.total;
    }
    if (pass == 0) return packed_fwd_ok(g) ? filter_bytes : 0;
    if (pass == 1) return packed_bwd_data_ok(g) ? filter_bytes : 0;
    const int M = g.K, N = g.C * RS;
    const bool narrow = M <= 64;
    const int TM = narrow ? 64 : 128, TN = narrow ? 256 : 128;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    long cap = ((long)g.N * g.P * g.Q + 4 * KB - 1) / (4 * KB);
    const long by_mem = (long)(kMaxWgradWorkspace / filter_bytes);
    if (cap > by_mem) cap = by_mem;
    const int want = choose_splits(tiles, (long)g.N * g.P * g.Q, cap, kPlanningCUs, filter_bytes, 2.0 * TM * TN * KB);
    if (want <= 1) return 0;
    const size_t need = (size_t)want * filter_bytes;
    if (need <= kDefaultStagingBytes) return 0; // the context's own staging area already holds it
    return need;
}

int vdnn_conv_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                  const void* x, const float* w, const float* bias, void* y,
                  void* workspace, size_t workspace_bytes) {
    return VDNN_BY_ACT(ctx, conv_fwd_impl<float>(ctx, stream, shape, algo_mode, (const float*)x, w, bias, (float*)y, workspace, workspace_bytes, 0),
                       conv_fwd_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)x, w, bias, (bf16_t*)y, workspace, workspace_bytes, 0));
}

int vdnn_conv_fwd_relu(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                       const void* x, const float* w, const float* bias, void* y,
                       void* workspace, size_t workspace_bytes) {
    return VDNN_BY_ACT(ctx, conv_fwd_impl<float>(ctx, stream, shape, algo_mode, (const float*)x, w, bias, (float*)y, workspace, workspace_bytes, 1),
                       conv_fwd_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)x, w, bias, (bf16_t*)y, workspace, workspace_bytes, 1));
}

int vdnn_conv_bwd_data(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                       const void* dy, const float* w, void* dx,
                       void* workspace, size_t workspace_bytes) {
    return VDNN_BY_ACT(ctx, conv_bwd_data_impl<float>(ctx, stream, shape, algo_mode, (const float*)dy, w, (float*)dx, workspace, workspace_bytes, nullptr),
                       conv_bwd_data_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)dy, w, (bf16_t*)dx, workspace, workspace_bytes, nullptr));
}

int vdnn_conv_bwd_data_in_place_ok(const vdnn_shape_t* shape) {
    ConvGeo g;
    return shape && geo_from_shape(shape, g) && conv_bwd_data_in_place_ok(g);
}

int vdnn_conv_bwd_data_relu(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                            const void* dy, const float* w, const void* x, void* dx,
                            void* workspace, size_t workspace_bytes) {
    VDNN_REQUIRE(x != nullptr, "null input tensor");
    return VDNN_BY_ACT(ctx, conv_bwd_data_impl<float>(ctx, stream, shape, algo_mode, (const float*)dy, w, (float*)dx, workspace, workspace_bytes, (const float*)x),
                       conv_bwd_data_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)dy, w, (bf16_t*)dx, workspace, workspace_bytes, (const bf16_t*)x));
}

int vdnn_conv_bwd_filter_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                             const void* x, const void* dy, float* w, float alpha,
                             void* workspace, size_t workspace_bytes) {
    return VDNN_BY_ACT(ctx, conv_bwd_filter_impl<float>(ctx, stream, shape, algo_mode, (const float*)x, (const float*)dy, w, alpha, 1, workspace, workspace_bytes),
                       conv_bwd_filter_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)x, (const bf16_t*)dy, w, alpha, 1, workspace, workspace_bytes));
}

int vdnn_conv_bwd_filter(vdnn_ctx* ctx, vdnn_stream_t stream, const vdnn_shape_t* shape, int algo_mode,
                         const void* x, const void* dy, float* dw, void* workspace, size_t workspace_bytes) {
    return VDNN_BY_ACT(ctx, conv_bwd_filter_impl<float>(ctx, stream, shape, algo_mode, (const float*)x, (const float*)dy, dw, 1.0f, 0, workspace, workspace_bytes),
                       conv_bwd_filter_impl<bf16_t>(ctx, stream, shape, algo_mode, (const bf16_t*)x, (const bf16_t*)dy, dw, 1.0f, 0, workspace, workspace_bytes));
}

} // extern "C"
