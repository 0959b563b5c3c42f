// Fully connected layers as fp32 MFMA GEMMs. Replaces the cublasSgemm calls of layer.cu:667-764.
// The filter is [c_out][c_in] row-major, activations are [n][c] row-major.
#include "backend_internal.h"
#include "mfma_gemm.h"

namespace vdnn {

int launch_reduce_splits(vdnn_ctx* ctx, hipStream_t stream, float* out, const float* partial, size_t count,
                         int splits, float alpha, int accumulate, const float* bias_j, int ncols);

// Out[M][N] (row stride ld_out) = alpha * A*B (+ Out) (+ bias per column); reduction split into
// ordered partial sums when the tile grid alone cannot fill the chip.
template <class AL, class BL>
static int fc_gemm(vdnn_ctx* ctx, hipStream_t st, const char* name, const AL& al, const BL& bl, int M, int N, int K,
                   float* out, long ld_out, float alpha, int accumulate, const float* bias_j) {
    if (ld_out != N) { set_error("fc_gemm: output must be dense"); return VDNN_EINVAL; }
    const int TM = M <= 64 ? 64 : 128, TN = M <= 64 ? 256 : 128;
    const long tiles = (long)((M + TM - 1) / TM) * ((N + TN - 1) / TN);
    long want = (4l * ctx->num_cu + tiles - 1) / tiles;
    const long by_depth = ((long)K + 8 * KB - 1) / (8 * KB);
    if (want > by_depth) want = by_depth;
    const long by_mem = (long)(ctx->reduce_scratch_bytes / ((size_t)M * N * sizeof(float)));
    if (want > by_mem) want = by_mem;
    if (want < 1) want = 1;
    GemmDims d;
    d.M = M; d.N = N; d.K = K;
    d.mtiles = (M + TM - 1) / TM; d.ntiles = (N + TN - 1) / TN;
    int kchunk = (int)((K + want - 1) / want);
    kchunk = (kchunk + KB - 1) / KB * KB;
    d.kchunk = kchunk;
    d.splits = (K + kchunk - 1) / kchunk;
    StoreDense ep{out, ctx->reduce_scratch, d.splits > 1 ? nullptr : bias_j, ld_out, (long)M * N, alpha, accumulate};
    const long blocks = (long)d.mtiles * d.ntiles * d.splits;
    ProfScope prof(ctx, st, name, 2.0 * M * (double)N * K, 0.0);
    if (TM == 64) hipLaunchKernelGGL((igemm_kernel<64, 256, AL, BL, StoreDense>), dim3((unsigned)blocks), dim3(NT), 0, st, al, bl, ep, d);
    else hipLaunchKernelGGL((igemm_kernel<128, 128, AL, BL, StoreDense>), dim3((unsigned)blocks), dim3(NT), 0, st, al, bl, ep, d);
    VDNN_LAUNCH_CHECK();
    if (d.splits > 1) return launch_reduce_splits(ctx, st, out, ctx->reduce_scratch, (size_t)M * N, d.splits, alpha, accumulate, bias_j, N);
    return VDNN_OK;
}

} // namespace vdnn

using namespace vdnn;

extern "C" {

// y[n][o] = sum_i x[n][i] * w[o][i] + bias[o]        (Sgemm(T,N) + bias broadcast, layer.cu:677-706)
int vdnn_fc_fwd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                const float* x, const float* w, const float* bias, float* y) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(x && w && y && n > 0 && c_in > 0 && c_out > 0, "bad argument");
    LoadDense<true> al{x, (long)c_in, 1, n, ctx->zeros};
    LoadDense<true> bl{w, (long)c_in, 1, c_out, ctx->zeros};
    return fc_gemm(ctx, stream_of(ctx, stream), "fc_fwd", al, bl, n, c_out, c_in, y, c_out, 1.0f, 0, bias);
}

// dx[n][i] = sum_o dy[n][o] * w[o][i]                 (Sgemm(N,N), layer.cu:725-733)
int vdnn_fc_bwd_data(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                     const float* dy, const float* w, float* dx) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(dy && w && dx && n > 0 && c_in > 0 && c_out > 0, "bad argument");
    LoadDense<true> al{dy, (long)c_out, 1, n, ctx->zeros};
    LoadDense<false> bl{w, 1, (long)c_in, c_in, ctx->zeros};
    return fc_gemm(ctx, stream_of(ctx, stream), "fc_bwd_data", al, bl, n, c_in, c_out, dx, c_in, 1.0f, 0, nullptr);
}

// w[o][i] += alpha * sum_n dy[n][o] * x[n][i]         (Sgemm(N,T) alpha=-lr beta=1, layer.cu:736-744)
int vdnn_fc_bwd_weight_sgd(vdnn_ctx* ctx, vdnn_stream_t stream, int n, int c_in, int c_out,
                           const float* x, const float* dy, float* w, float alpha) {
    VDNN_KERNEL_PROLOGUE(ctx);
    VDNN_REQUIRE(x && dy && w && n > 0 && c_in > 0 && c_out > 0, "bad argument");
    LoadDense<false> al{dy, 1, (long)c_out, c_out, ctx->zeros};
    LoadDense<false> bl{x, 1, (long)c_in, c_in, ctx->zeros};
    return fc_gemm(ctx, stream_of(ctx, stream), "fc_bwd_weight", al, bl, c_out, c_in, n, w, c_in, alpha, 1, nullptr);
}

} // extern "C"
