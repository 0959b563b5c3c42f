// Fully connected layers as fp32 MFMA GEMMs. Replaces the cublasSgemm calls of layer.cu:667-764.
// The filter is [c_out][c_in] row-major, activations are [n][c] row-major.
#include "backend_internal.h"
#include "mfma_gemm.h"
#include "fc_bf16.h"

namespace vdnn {

int launch_reduce_splits(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count,
                         int splits, float alpha, int accumulate, const float* bias_j, int ncols, int relu, const float* gate);
int launch_reduce_splits(vdnn_ctx* ctx, hipStream_t stream, bf16_t* out, const float* partial, size_t count,
                         int splits, float alpha, int accumulate, const float* bias_j, int ncols, int relu, const bf16_t* gate);

static inline bool fc_aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// The filter operand of forward and backward data: as stored for float activations; rounded to bfloat16 on
// its way into LDS when the activations are bfloat16 (the products then have two bfloat16 factors).
template <class L, class E> struct FilterOperand { struct type : L {}; };
template <class L> struct FilterOperand<L, bf16_t> { typedef RoundedToBf16<L> type; };

// Out[M][N] (dense, row stride N) = alpha * A*B (+ Out) (+ bias per column); the reduction is split into
// ordered partial sums when the tile grid alone cannot fill the chip.
template <class AL, class BL, class EO>
static int fc_gemm(vdnn_ctx* ctx, hipStream_t st, const char* name, const AL& al, const BL& bl, int M, int N, int K,
                   EO* out, float alpha, int accumulate, const float* bias_j, int relu = 0, const EO* gate = nullptr) {
    const int TM = M <= 64 ? 64 : 128, TN = M <= 64 ? 256 : 128;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    long cap = ((long)K + 8 * KB - 1) / (8 * KB); // at least eight slices per split
    const long by_mem = (long)(ctx->reduce_scratch_bytes / ((size_t)M * N * sizeof(float)));
    if (cap > by_mem) cap = by_mem;
    const long want = choose_splits(tiles, K, cap, ctx->num_cu, (size_t)M * N * sizeof(float), 2.0 * TM * TN * KB);
    GemmDims d;
    d.M = M; d.N = N; d.K = K;
    d.mtiles = (M + TM - 1) / TM; d.ntiles = (N + TN - 1) / TN;
    int kchunk = (int)((K + want - 1) / want);
    kchunk = (kchunk + KB - 1) / KB * KB;
    d.kchunk = kchunk;
    d.splits = (K + kchunk - 1) / kchunk;
    d.full_tiles = 0;
    StoreDense<EO> ep{out, ctx->reduce_scratch, d.splits > 1 ? nullptr : bias_j, (long)N, (long)M * N, alpha, accumulate, relu, gate};
    const long blocks = (long)d.mtiles * d.ntiles * d.splits;
    ProfScope prof(ctx, st, name, 2.0 * M * (double)N * K, 0.0);
    if (TM == 64) hipLaunchKernelGGL((igemm_kernel<64, 256, AL, BL, StoreDense<EO>>), dim3((unsigned)blocks), dim3(NT), 0, st, al, bl, ep, d);
    else hipLaunchKernelGGL((igemm_kernel<128, 128, AL, BL, StoreDense<EO>>), dim3((unsigned)blocks), dim3(NT), 0, st, al, bl, ep, d);
    VDNN_LAUNCH_CHECK();
    if (d.splits > 1) return launch_reduce_splits(ctx, st, out, ctx->reduce_scratch, (size_t)M * N, d.splits, alpha, accumulate, bias_j, N, relu, gate);
    return VDNN_OK;
}

// The same product on the bfloat16 matrix cores (operands of fc_bf16.h). The multiplications are no longer what
// bounds it, the filter's trip through memory is: the reduction is split until about two workgroups per compute
// unit are in flight, each with at least eight slices.
// The update's result is the filter itself: column tiles fastest, so that the workgroups at work together write runs of rows.
template <class E> struct StoreDenseRuns : StoreDense<E> {};
template <class E> struct TileOrder<StoreDenseRuns<E>> { static constexpr bool COLUMNS_FASTEST = true; };

template <template <class> class EPT = StoreDense, class AL, class BL, class EO>
static int fc_gemm_bf16(vdnn_ctx* ctx, hipStream_t st, const char* name, const AL& al, const BL& bl, int M, int N, int K,
                        EO* out, float alpha, int accumulate, const float* bias_j, int relu = 0, const EO* gate = nullptr) {
    const int TM = M <= 64 ? 64 : 128, TN = M <= 64 ? 256 : 128;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    long want = (2l * ctx->num_cu + tiles - 1) / tiles;
    const long by_depth = ((long)K + 8 * KH - 1) / (8 * KH);
    const long by_mem = (long)(ctx->reduce_scratch_bytes / ((size_t)M * N * sizeof(float)));
    if (want > by_depth) want = by_depth;
    if (want > by_mem) want = by_mem;
    if (want < 1) want = 1;
    GemmDims d;
    d.M = M; d.N = N; d.K = K;
    d.mtiles = (M + TM - 1) / TM; d.ntiles = (N + TN - 1) / TN;
    int kchunk = (int)((K + want - 1) / want);
    kchunk = (kchunk + KH - 1) / KH * KH;
    d.kchunk = kchunk;
    d.splits = (K + kchunk - 1) / kchunk;
    d.full_tiles = 0;
    const StoreDense<EO> fields{out, ctx->reduce_scratch, d.splits > 1 ? nullptr : bias_j, (long)N, (long)M * N, alpha, accumulate, relu, gate};
    EPT<EO> ep;
    static_cast<StoreDense<EO>&>(ep) = fields;
    const long blocks = (long)d.mtiles * d.ntiles * d.splits;
    ProfScope prof(ctx, st, name, 2.0 * M * (double)N * K, 0.0);
    if (TM == 64) hipLaunchKernelGGL((igemm_bf16_kernel<64, 256, AL, BL, EPT<EO>>), dim3((unsigned)blocks), dim3(NT), 0, st, al, bl, ep, d);
    else hipLaunchKernelGGL((igemm_bf16_kernel<128, 128, AL, BL, EPT<EO>>), dim3((unsigned)blocks), dim3(NT), 0, st, al, bl, ep, d);
    VDNN_LAUNCH_CHECK();
    if (d.splits > 1) return launch_reduce_splits(ctx, st, out, ctx->reduce_scratch, (size_t)M * N, d.splits, alpha, accumulate, bias_j, N, relu, gate);
    return VDNN_OK;
}

template <class E> struct IsBf16 { static constexpr bool V = false; };
template <> struct IsBf16<bf16_t> { static constexpr bool V = true; };

} // namespace vdnn

using namespace vdnn;

#define FC_REQUIRE_SMALL(elems) VDNN_REQUIRE((long)(elems) * 4 < 0x7FFF0000l, "matrix of 2 GiB or more")

// y[n][o] = sum_i x[n][i] * w[o][i] + bias[o]        (Sgemm(T,N) + bias broadcast, layer.cu:677-706)
template <class E>
static int fc_fwd_impl(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                       const E* x, const float* w, const float* bias, E* y, int relu) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(x && w && y && n > 0 && c_in > 0 && c_out > 0, "bad argument");
    FC_REQUIRE_SMALL((long)n * c_in); FC_REQUIRE_SMALL((long)c_out * c_in);
    const unsigned xb = (unsigned)((long)n * c_in * sizeof(E)), wb = (unsigned)((long)c_out * c_in * 4);
    hipStream_t st = stream_of(ctx, stream);
    if constexpr (IsBf16<E>::V) {
        if (c_in % 8 == 0 && fc_aligned16(x) && fc_aligned16(w)) {
            LoadRedAsH<bf16_t> al{x, (long)c_in, n, xb};
            LoadRedAsH<float> bl{w, (long)c_in, c_out, wb};
            return fc_gemm_bf16(ctx, st, "fc_fwd", al, bl, n, c_out, c_in, y, 1.0f, 0, bias, relu);
        }
    }
    if (c_in % 4 == 0 && fc_aligned16(x) && fc_aligned16(w)) {
        LoadDenseRed<true, E> al{x, (long)c_in, n, xb};
        typename FilterOperand<LoadDenseRed<true>, E>::type bl{{w, (long)c_in, c_out, wb}};
        return fc_gemm(ctx, st, "fc_fwd", al, bl, n, c_out, c_in, y, 1.0f, 0, bias, relu);
    }
    LoadDenseRed<false, E> al{x, (long)c_in, n, xb};
    typename FilterOperand<LoadDenseRed<false>, E>::type bl{{w, (long)c_in, c_out, wb}};
    return fc_gemm(ctx, st, "fc_fwd", al, bl, n, c_out, c_in, y, 1.0f, 0, bias, relu);
}

// dx[n][i] = sum_o dy[n][o] * w[o][i]                 (Sgemm(N,N), layer.cu:725-733)
template <class E>
static int fc_bwd_data_impl(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                            const E* dy, const float* w, E* dx, const E* gate) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(dy && w && dx && n > 0 && c_in > 0 && c_out > 0, "bad argument");
    FC_REQUIRE_SMALL((long)n * c_out); FC_REQUIRE_SMALL((long)c_out * c_in);
    const unsigned db = (unsigned)((long)n * c_out * sizeof(E)), wb = (unsigned)((long)c_out * c_in * 4);
    hipStream_t st = stream_of(ctx, stream);
    if constexpr (IsBf16<E>::V) {
        if (c_out % 8 == 0 && fc_aligned16(dy)) {
            LoadRedAsH<bf16_t> al{dy, (long)c_out, n, db};
            LoadRowAsH<float> bl{w, (long)c_in, c_in, wb};
            return fc_gemm_bf16(ctx, st, "fc_bwd_data", al, bl, n, c_in, c_out, dx, 1.0f, 0, nullptr, 0, gate);
        }
    }
    typename FilterOperand<LoadDenseRow<float>, E>::type bl{{w, (long)c_in, c_in, wb}};
    if (c_out % 4 == 0 && fc_aligned16(dy)) {
        LoadDenseRed<true, E> al{dy, (long)c_out, n, db};
        return fc_gemm(ctx, st, "fc_bwd_data", al, bl, n, c_in, c_out, dx, 1.0f, 0, nullptr, 0, gate);
    }
    LoadDenseRed<false, E> al{dy, (long)c_out, n, db};
    return fc_gemm(ctx, st, "fc_bwd_data", al, bl, n, c_in, c_out, dx, 1.0f, 0, nullptr, 0, gate);
}

// out[o][i] = (accumulate ? out : 0) + alpha * sum_n dy[n][o] * x[n][i]   (Sgemm(N,T), layer.cu:736-744)
template <class E>
static int fc_bwd_weight_impl(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                              const E* x, const E* dy, float* w, float alpha, int accumulate) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(x && dy && w && n > 0 && c_in > 0 && c_out > 0, "bad argument");
    FC_REQUIRE_SMALL((long)n * c_out); FC_REQUIRE_SMALL((long)n * c_in);
    if constexpr (IsBf16<E>::V) {
        if (n % 8 == 0) {
            LoadRowAsH<bf16_t> al{dy, (long)c_out, c_out, (unsigned)((long)n * c_out * sizeof(E))};
            LoadRowAsH<bf16_t> bl{x, (long)c_in, c_in, (unsigned)((long)n * c_in * sizeof(E))};
            return fc_gemm_bf16<StoreDenseRuns>(ctx, stream_of(ctx, stream), "fc_bwd_weight", al, bl, c_out, c_in, n, w, alpha, accumulate, nullptr);
        }
    }
    LoadDenseRow<E> al{dy, (long)c_out, c_out, (unsigned)((long)n * c_out * sizeof(E))};
    LoadDenseRow<E> bl{x, (long)c_in, c_in, (unsigned)((long)n * c_in * sizeof(E))};
    return fc_gemm(ctx, stream_of(ctx, stream), "fc_bwd_weight", al, bl, c_out, c_in, n, w, alpha, accumulate, nullptr);
}

extern "C" {

int vdnn_fc_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                const void* x, const float* w, const float* bias, void* y) {
    return VDNN_BY_ACT(ctx, fc_fwd_impl<float>(ctx, stream, n, c_in, c_out, (const float*)x, w, bias, (float*)y, 0),
                       fc_fwd_impl<bf16_t>(ctx, stream, n, c_in, c_out, (const bf16_t*)x, w, bias, (bf16_t*)y, 0));
}

int vdnn_fc_fwd_relu(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                     const void* x, const float* w, const float* bias, void* y) {
    return VDNN_BY_ACT(ctx, fc_fwd_impl<float>(ctx, stream, n, c_in, c_out, (const float*)x, w, bias, (float*)y, 1),
                       fc_fwd_impl<bf16_t>(ctx, stream, n, c_in, c_out, (const bf16_t*)x, w, bias, (bf16_t*)y, 1));
}

int vdnn_fc_bwd_data(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                     const void* dy, const float* w, void* dx) {
    return VDNN_BY_ACT(ctx, fc_bwd_data_impl<float>(ctx, stream, n, c_in, c_out, (const float*)dy, w, (float*)dx, nullptr),
                       fc_bwd_data_impl<bf16_t>(ctx, stream, n, c_in, c_out, (const bf16_t*)dy, w, (bf16_t*)dx, nullptr));
}

int vdnn_fc_bwd_data_relu(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                          const void* dy, const float* w, const void* x, void* dx) {
    VDNN_REQUIRE(x != nullptr, "null input tensor");
    return VDNN_BY_ACT(ctx, fc_bwd_data_impl<float>(ctx, stream, n, c_in, c_out, (const float*)dy, w, (float*)dx, (const float*)x),
                       fc_bwd_data_impl<bf16_t>(ctx, stream, n, c_in, c_out, (const bf16_t*)dy, w, (bf16_t*)dx, (const bf16_t*)x));
}

int vdnn_fc_bwd_weight_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                           const void* x, const void* dy, float* w, float alpha) {
    return VDNN_BY_ACT(ctx, fc_bwd_weight_impl<float>(ctx, stream, n, c_in, c_out, (const float*)x, (const float*)dy, w, alpha, 1),
                       fc_bwd_weight_impl<bf16_t>(ctx, stream, n, c_in, c_out, (const bf16_t*)x, (const bf16_t*)dy, w, alpha, 1));
}

int vdnn_fc_bwd_weight(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                       const void* x, const void* dy, float* dw) {
    return VDNN_BY_ACT(ctx, fc_bwd_weight_impl<float>(ctx, stream, n, c_in, c_out, (const float*)x, (const float*)dy, dw, 1.0f, 0),
                       fc_bwd_weight_impl<bf16_t>(ctx, stream, n, c_in, c_out, (const bf16_t*)x, (const bf16_t*)dy, dw, 1.0f, 0));
}

} // extern "C"
