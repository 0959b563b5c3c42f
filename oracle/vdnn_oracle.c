/* TEST INFRASTRUCTURE — CPU restatement of the reference's layer math (see vdnn_oracle.h).
 * Plain C + OpenMP. Each function cites the reference call site whose semantics it restates. */
#include "vdnn_oracle.h"

#include <float.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_acc_double = 0;
static int g_blocked = 0; /* stride-1 convolutions through the blocked SGEMM of vdnn_oracle_gemm.c (float accumulation only) */
static int g_threads = 0;

void orc_set_accumulate_double(int on) { g_acc_double = on ? 1 : 0; }
int  orc_get_accumulate_double(void) { return g_acc_double; }
void orc_set_blocked_gemm(int on) { g_blocked = on ? 1 : 0; }
int  orc_get_blocked_gemm(void) { return g_blocked; }
void orc_set_threads(int n) {
    g_threads = n;
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#endif
}
int orc_get_threads(void) {
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

/* layer.cu:208-216 (conv), 432-439 (pool): cuDNN's output extent */
int orc_out_dim(int in, int pad, int window, int stride) {
    if (stride <= 0) return 0;
    return (in + 2 * pad - window) / stride + 1;
}

/* valid q range for a filter tap s: 0 <= q*sw - pw + s < W */
static void q_range(int Q, int W, int sw, int pw, int s, int* q_lo, int* q_hi) {
    int lo = 0, hi = Q; /* [lo, hi) */
    /* q*sw >= pw - s */
    int t = pw - s;
    if (t > 0) lo = (t + sw - 1) / sw;
    /* q*sw <= W - 1 + pw - s */
    int u = W - 1 + pw - s;
    if (u < 0) hi = 0;
    else {
        int m = u / sw + 1;
        if (m < hi) hi = m;
    }
    if (lo > hi) lo = hi;
    *q_lo = lo; *q_hi = hi;
}

/* ---------------------------------------------------------------------------------------------
 * Convolution forward: cudnnConvolutionForward (alpha 1, beta 0) then cudnnAddTensor
 * (layer.cu:560-582). y[n,k,p,q] = sum_{c,r,s} x[n,c,p*sh-ph+r,q*sw-pw+s] * w[k,c,r,s] + b[k].
 * Per (n,k) plane, taps are applied as row updates in (c,r,s) order, so every output element sums
 * its terms in (c,r,s) order.
 * ------------------------------------------------------------------------------------------- */
#define DEFINE_CONV_FWD(NAME, ACC)                                                                   \
static void NAME(const orc_shape* g, const float* x, const float* w, const float* bias, float* y) { \
    const int N = g->n, C = g->c, H = g->h, W = g->w, K = g->k, R = g->r, S = g->s;                  \
    const int ph = g->pad_h, pw = g->pad_w, sh = g->stride_h, sw = g->stride_w;                      \
    const int P = orc_out_dim(H, ph, R, sh), Q = orc_out_dim(W, pw, S, sw);                          \
    const long planes = (long)N * K;                                                                 \
    _Pragma("omp parallel")                                                                          \
    {                                                                                                \
        ACC* acc = (ACC*)malloc(sizeof(ACC) * (size_t)P * Q);                                        \
        _Pragma("omp for schedule(dynamic, 1)")                                                      \
        for (long nk = 0; nk < planes; nk++) {                                                       \
            const int n = (int)(nk / K), k = (int)(nk % K);                                          \
            for (long i = 0; i < (long)P * Q; i++) acc[i] = 0;                                       \
            for (int c = 0; c < C; c++) {                                                            \
                const float* xp = x + ((size_t)n * C + c) * H * W;                                   \
                for (int r = 0; r < R; r++)                                                          \
                    for (int s = 0; s < S; s++) {                                                    \
                        const ACC wv = w[(((size_t)k * C + c) * R + r) * S + s];                     \
                        int q_lo, q_hi;                                                              \
                        q_range(Q, W, sw, pw, s, &q_lo, &q_hi);                                      \
                        for (int p = 0; p < P; p++) {                                                \
                            const int ih = p * sh - ph + r;                                          \
                            if (ih < 0 || ih >= H) continue;                                         \
                            const float* xr = xp + (size_t)ih * W - pw + s;                          \
                            ACC* ar = acc + (size_t)p * Q;                                           \
                            if (sw == 1) {                                                           \
                                for (int q = q_lo; q < q_hi; q++) ar[q] += wv * (ACC)xr[q];          \
                            } else {                                                                 \
                                for (int q = q_lo; q < q_hi; q++) ar[q] += wv * (ACC)xr[q * sw];     \
                            }                                                                        \
                        }                                                                            \
                    }                                                                                \
            }                                                                                        \
            float* yp = y + ((size_t)n * K + k) * P * Q;                                             \
            const float b = bias ? bias[k] : 0.0f;                                                   \
            for (long i = 0; i < (long)P * Q; i++) {                                                 \
                const float v = (float)acc[i];                                                       \
                yp[i] = bias ? v + b : v;                                                            \
            }                                                                                        \
        }                                                                                            \
        free(acc);                                                                                   \
    }                                                                                                \
}
DEFINE_CONV_FWD(conv_fwd_f32, float)
DEFINE_CONV_FWD(conv_fwd_f64, double)

void orc_conv_fwd(const orc_shape* g, const float* x, const float* w, const float* bias, float* y) {
    if (g_blocked && !g_acc_double && orc_blocked_conv_ok(g)) { orc_blocked_conv_fwd(g, x, w, bias, y); return; }
    if (g_acc_double) conv_fwd_f64(g, x, w, bias, y);
    else conv_fwd_f32(g, x, w, bias, y);
}

/* ---------------------------------------------------------------------------------------------
 * Backward data: cudnnConvolutionBackwardData, alpha 1, beta 0 (layer.cu:616-625).
 * dx[n,c,h,w] = sum_{k,r,s} dy[n,k,p,q] * w[k,c,r,s] over the (p,q) with p*sh-ph+r == h,
 * q*sw-pw+s == w. Scatter form per (n,c) plane.
 * ------------------------------------------------------------------------------------------- */
#define DEFINE_CONV_BWD_DATA(NAME, ACC)                                                              \
static void NAME(const orc_shape* g, const float* dy, const float* w, float* dx) {                   \
    const int N = g->n, C = g->c, H = g->h, W = g->w, K = g->k, R = g->r, S = g->s;                  \
    const int ph = g->pad_h, pw = g->pad_w, sh = g->stride_h, sw = g->stride_w;                      \
    const int P = orc_out_dim(H, ph, R, sh), Q = orc_out_dim(W, pw, S, sw);                          \
    const long planes = (long)N * C;                                                                 \
    _Pragma("omp parallel")                                                                          \
    {                                                                                                \
        ACC* acc = (ACC*)malloc(sizeof(ACC) * (size_t)H * W);                                        \
        _Pragma("omp for schedule(dynamic, 1)")                                                      \
        for (long nc = 0; nc < planes; nc++) {                                                       \
            const int n = (int)(nc / C), c = (int)(nc % C);                                          \
            for (long i = 0; i < (long)H * W; i++) acc[i] = 0;                                       \
            for (int k = 0; k < K; k++) {                                                            \
                const float* dyp = dy + ((size_t)n * K + k) * P * Q;                                 \
                for (int r = 0; r < R; r++)                                                          \
                    for (int s = 0; s < S; s++) {                                                    \
                        const ACC wv = w[(((size_t)k * C + c) * R + r) * S + s];                     \
                        int q_lo, q_hi;                                                              \
                        q_range(Q, W, sw, pw, s, &q_lo, &q_hi);                                      \
                        for (int p = 0; p < P; p++) {                                                \
                            const int ih = p * sh - ph + r;                                          \
                            if (ih < 0 || ih >= H) continue;                                         \
                            ACC* ar = acc + (size_t)ih * W - pw + s;                                 \
                            const float* dr = dyp + (size_t)p * Q;                                   \
                            if (sw == 1) {                                                           \
                                for (int q = q_lo; q < q_hi; q++) ar[q] += wv * (ACC)dr[q];          \
                            } else {                                                                 \
                                for (int q = q_lo; q < q_hi; q++) ar[q * sw] += wv * (ACC)dr[q];     \
                            }                                                                        \
                        }                                                                            \
                    }                                                                                \
            }                                                                                        \
            float* dxp = dx + ((size_t)n * C + c) * H * W;                                           \
            for (long i = 0; i < (long)H * W; i++) dxp[i] = (float)acc[i];                           \
        }                                                                                            \
        free(acc);                                                                                   \
    }                                                                                                \
}
DEFINE_CONV_BWD_DATA(conv_bwd_data_f32, float)
DEFINE_CONV_BWD_DATA(conv_bwd_data_f64, double)

void orc_conv_bwd_data(const orc_shape* g, const float* dy, const float* w, float* dx) {
    if (g_blocked && !g_acc_double && orc_blocked_conv_ok(g)) { orc_blocked_conv_bwd_data(g, dy, w, dx); return; }
    if (g_acc_double) conv_bwd_data_f64(g, dy, w, dx);
    else conv_bwd_data_f32(g, dy, w, dx);
}

/* cudnnConvolutionBackwardBias alpha=-lr beta=1 (layer.cu:631-637) */
void orc_conv_bwd_bias_sgd(const orc_shape* g, const float* dy, float* bias, float alpha) {
    const int N = g->n, K = g->k;
    const int P = orc_out_dim(g->h, g->pad_h, g->r, g->stride_h);
    const int Q = orc_out_dim(g->w, g->pad_w, g->s, g->stride_w);
    const size_t PQ = (size_t)P * Q;
#pragma omp parallel for schedule(static)
    for (int k = 0; k < K; k++) {
        double acc = 0.0; /* double: the bias sum is a long, cancellation-prone reduction */
        for (int n = 0; n < N; n++) {
            const float* d = dy + ((size_t)n * K + k) * PQ;
            for (size_t i = 0; i < PQ; i++) acc += d[i];
        }
        bias[k] = bias[k] + alpha * (float)acc;
    }
}

/* ---------------------------------------------------------------------------------------------
 * Backward filter: cudnnConvolutionBackwardFilter alpha=-lr beta=1 (layer.cu:651-660).
 * w[k,c,r,s] = w + alpha * sum_{n,p,q} dy[n,k,p,q] * x[n,c,p*sh-ph+r,q*sw-pw+s].
 * ------------------------------------------------------------------------------------------- */
#define DEFINE_CONV_BWD_FILTER(NAME, ACC)                                                            \
static void NAME(const orc_shape* g, const float* x, const float* dy, float* w, float alpha) {       \
    const int N = g->n, C = g->c, H = g->h, W = g->w, K = g->k, R = g->r, S = g->s;                  \
    const int ph = g->pad_h, pw = g->pad_w, sh = g->stride_h, sw = g->stride_w;                      \
    const int P = orc_out_dim(H, ph, R, sh), Q = orc_out_dim(W, pw, S, sw);                          \
    const long pairs = (long)K * C;                                                                  \
    _Pragma("omp parallel for schedule(dynamic, 4)")                                                 \
    for (long kc = 0; kc < pairs; kc++) {                                                            \
        const int k = (int)(kc / C), c = (int)(kc % C);                                              \
        for (int r = 0; r < R; r++)                                                                  \
            for (int s = 0; s < S; s++) {                                                            \
                int q_lo, q_hi;                                                                      \
                q_range(Q, W, sw, pw, s, &q_lo, &q_hi);                                              \
                ACC acc = 0;                                                                         \
                for (int n = 0; n < N; n++) {                                                        \
                    const float* xp = x + ((size_t)n * C + c) * H * W;                               \
                    const float* dyp = dy + ((size_t)n * K + k) * P * Q;                             \
                    for (int p = 0; p < P; p++) {                                                    \
                        const int ih = p * sh - ph + r;                                              \
                        if (ih < 0 || ih >= H) continue;                                             \
                        const float* xr = xp + (size_t)ih * W - pw + s;                              \
                        const float* dr = dyp + (size_t)p * Q;                                       \
                        ACC row = 0;                                                                 \
                        if (sw == 1) {                                                               \
                            _Pragma("omp simd reduction(+:row)")                                     \
                            for (int q = q_lo; q < q_hi; q++) row += (ACC)dr[q] * (ACC)xr[q];        \
                        } else {                                                                     \
                            for (int q = q_lo; q < q_hi; q++) row += (ACC)dr[q] * (ACC)xr[q * sw];   \
                        }                                                                            \
                        acc += row;                                                                  \
                    }                                                                                \
                }                                                                                    \
                float* wp = w + (((size_t)k * C + c) * R + r) * S + s;                               \
                *wp = *wp + alpha * (float)acc;                                                      \
            }                                                                                        \
    }                                                                                                \
}
DEFINE_CONV_BWD_FILTER(conv_bwd_filter_f32, float)
DEFINE_CONV_BWD_FILTER(conv_bwd_filter_f64, double)

void orc_conv_bwd_filter_sgd(const orc_shape* g, const float* x, const float* dy, float* w, float alpha) {
    if (g_blocked && !g_acc_double && orc_blocked_conv_ok(g)) { orc_blocked_conv_bwd_filter_sgd(g, x, dy, w, alpha); return; }
    if (g_acc_double) conv_bwd_filter_f64(g, x, dy, w, alpha);
    else conv_bwd_filter_f32(g, x, dy, w, alpha);
}

/* ---- brute-force forms: one loop per index, double accumulation ------------------------------ */
void orc_conv_fwd_brute(const orc_shape* g, const float* x, const float* w, const float* bias, float* y) {
    const int N = g->n, C = g->c, H = g->h, W = g->w, K = g->k, R = g->r, S = g->s;
    const int P = orc_out_dim(H, g->pad_h, R, g->stride_h), Q = orc_out_dim(W, g->pad_w, S, g->stride_w);
    for (int n = 0; n < N; n++) for (int k = 0; k < K; k++)
    for (int p = 0; p < P; p++) for (int q = 0; q < Q; q++) {
        double acc = 0.0;
        for (int c = 0; c < C; c++) for (int r = 0; r < R; r++) for (int s = 0; s < S; s++) {
            const int ih = p * g->stride_h - g->pad_h + r, iw = q * g->stride_w - g->pad_w + s;
            if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
            acc += (double)x[(((size_t)n * C + c) * H + ih) * W + iw] *
                   (double)w[(((size_t)k * C + c) * R + r) * S + s];
        }
        if (bias) acc += bias[k];
        y[(((size_t)n * K + k) * P + p) * Q + q] = (float)acc;
    }
}

void orc_conv_bwd_data_brute(const orc_shape* g, const float* dy, const float* w, float* dx) {
    const int N = g->n, C = g->c, H = g->h, W = g->w, K = g->k, R = g->r, S = g->s;
    const int P = orc_out_dim(H, g->pad_h, R, g->stride_h), Q = orc_out_dim(W, g->pad_w, S, g->stride_w);
    for (int n = 0; n < N; n++) for (int c = 0; c < C; c++)
    for (int h = 0; h < H; h++) for (int ww = 0; ww < W; ww++) {
        double acc = 0.0;
        for (int k = 0; k < K; k++) for (int r = 0; r < R; r++) for (int s = 0; s < S; s++) {
            const int tp = h + g->pad_h - r, tq = ww + g->pad_w - s;
            if (tp < 0 || tq < 0 || tp % g->stride_h || tq % g->stride_w) continue;
            const int p = tp / g->stride_h, q = tq / g->stride_w;
            if (p >= P || q >= Q) continue;
            acc += (double)dy[(((size_t)n * K + k) * P + p) * Q + q] *
                   (double)w[(((size_t)k * C + c) * R + r) * S + s];
        }
        dx[(((size_t)n * C + c) * H + h) * W + ww] = (float)acc;
    }
}

void orc_conv_bwd_filter_brute(const orc_shape* g, const float* x, const float* dy, float* dw) {
    const int N = g->n, C = g->c, H = g->h, W = g->w, K = g->k, R = g->r, S = g->s;
    const int P = orc_out_dim(H, g->pad_h, R, g->stride_h), Q = orc_out_dim(W, g->pad_w, S, g->stride_w);
    for (int k = 0; k < K; k++) for (int c = 0; c < C; c++)
    for (int r = 0; r < R; r++) for (int s = 0; s < S; s++) {
        double acc = 0.0;
        for (int n = 0; n < N; n++) for (int p = 0; p < P; p++) for (int q = 0; q < Q; q++) {
            const int ih = p * g->stride_h - g->pad_h + r, iw = q * g->stride_w - g->pad_w + s;
            if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
            acc += (double)dy[(((size_t)n * K + k) * P + p) * Q + q] *
                   (double)x[(((size_t)n * C + c) * H + ih) * W + iw];
        }
        dw[(((size_t)k * C + c) * R + r) * S + s] = (float)acc;
    }
}

/* ---------------------------------------------------------------------------------------------
 * Fully connected. w is [c_out][c_in] row-major (column-major c_in x c_out with ld c_in, which is
 * how the reference hands it to cuBLAS, layer.cu:677-685).
 * ------------------------------------------------------------------------------------------- */
/* Sgemm(T,N) then the rank-1 bias GEMM (layer.cu:677-706) */
void orc_fc_fwd(int n, int c_in, int c_out, const float* x, const float* w, const float* bias, float* y) {
    const int dbl = g_acc_double;
#pragma omp parallel for collapse(2) schedule(static)
    for (int i = 0; i < n; i++)
        for (int o = 0; o < c_out; o++) {
            const float* xr = x + (size_t)i * c_in;
            const float* wr = w + (size_t)o * c_in;
            float v;
            if (dbl) {
                double acc = 0.0;
                for (int j = 0; j < c_in; j++) acc += (double)wr[j] * (double)xr[j];
                v = (float)acc;
            } else {
                float acc = 0.0f;
#pragma omp simd reduction(+:acc)
                for (int j = 0; j < c_in; j++) acc += wr[j] * xr[j];
                v = acc;
            }
            y[(size_t)i * c_out + o] = bias ? v + bias[o] : v;
        }
}

/* Sgemm(N,N) (layer.cu:725-733): dx[n,i] = sum_o w[o,i] dy[n,o] */
void orc_fc_bwd_data(int n, int c_in, int c_out, const float* dy, const float* w, float* dx) {
    const int dbl = g_acc_double;
#pragma omp parallel
    {
        double* accd = dbl ? (double*)malloc(sizeof(double) * (size_t)c_in) : NULL;
#pragma omp for schedule(static)
        for (int i = 0; i < n; i++) {
            float* dr = dx + (size_t)i * c_in;
            if (dbl) {
                for (int j = 0; j < c_in; j++) accd[j] = 0.0;
                for (int o = 0; o < c_out; o++) {
                    const double d = dy[(size_t)i * c_out + o];
                    const float* wr = w + (size_t)o * c_in;
                    for (int j = 0; j < c_in; j++) accd[j] += d * (double)wr[j];
                }
                for (int j = 0; j < c_in; j++) dr[j] = (float)accd[j];
            } else {
                for (int j = 0; j < c_in; j++) dr[j] = 0.0f;
                for (int o = 0; o < c_out; o++) {
                    const float d = dy[(size_t)i * c_out + o];
                    const float* wr = w + (size_t)o * c_in;
                    for (int j = 0; j < c_in; j++) dr[j] += d * wr[j];
                }
            }
        }
        free(accd);
    }
}

/* Sgemm(N,T) alpha=-lr beta=1 (layer.cu:736-744): w[o,i] += alpha * sum_n x[n,i] dy[n,o] */
void orc_fc_bwd_weight_sgd(int n, int c_in, int c_out, const float* x, const float* dy, float* w, float alpha) {
    const int dbl = g_acc_double;
#pragma omp parallel
    {
        double* accd = dbl ? (double*)malloc(sizeof(double) * (size_t)c_in) : NULL;
        float* accf = dbl ? NULL : (float*)malloc(sizeof(float) * (size_t)c_in);
#pragma omp for schedule(static)
        for (int o = 0; o < c_out; o++) {
            float* wr = w + (size_t)o * c_in;
            if (dbl) {
                for (int j = 0; j < c_in; j++) accd[j] = 0.0;
                for (int i = 0; i < n; i++) {
                    const double d = dy[(size_t)i * c_out + o];
                    const float* xr = x + (size_t)i * c_in;
                    for (int j = 0; j < c_in; j++) accd[j] += d * (double)xr[j];
                }
                for (int j = 0; j < c_in; j++) wr[j] = wr[j] + alpha * (float)accd[j];
            } else {
                for (int j = 0; j < c_in; j++) accf[j] = 0.0f;
                for (int i = 0; i < n; i++) {
                    const float d = dy[(size_t)i * c_out + o];
                    const float* xr = x + (size_t)i * c_in;
                    for (int j = 0; j < c_in; j++) accf[j] += d * xr[j];
                }
                for (int j = 0; j < c_in; j++) wr[j] = wr[j] + alpha * accf[j];
            }
        }
        free(accd); free(accf);
    }
}

/* Sgemm with the ones vector, alpha=-lr beta=1 (layer.cu:747-761) */
void orc_fc_bwd_bias_sgd(int n, int c_out, const float* dy, float* bias, float alpha) {
    for (int o = 0; o < c_out; o++) {
        double acc = 0.0;
        for (int i = 0; i < n; i++) acc += dy[(size_t)i * c_out + o];
        bias[o] = bias[o] + alpha * (float)acc;
    }
}

/* ---------------------------------------------------------------------------------------------
 * ReLU: cudnnActivationForward/Backward, CUDNN_PROPAGATE_NAN, coef 0 (layer.cu:774-781, 802-811,
 * descriptor :380-385).
 * ------------------------------------------------------------------------------------------- */
void orc_relu_fwd(size_t count, const float* x, float* y) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        const float v = x[i];
        y[i] = (v > 0.0f) ? v : ((v != v) ? v : 0.0f);
    }
}

/* dx = dy where x > 0, else 0. x may be NULL: y > 0 selects the same elements. */
void orc_relu_bwd(size_t count, const float* x, const float* y, const float* dy, float* dx) {
    const float* t = x ? x : y;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) dx[i] = (t[i] > 0.0f) ? dy[i] : 0.0f;
}

/* ---------------------------------------------------------------------------------------------
 * bfloat16 storage (the reduced-precision configuration; the reference is float only, vdnn.h:11-12).
 * A bfloat16 value is the float whose low 16 bits are zero. Rounding a float to it: to nearest, ties
 * to even; infinities stay, NaN stays NaN (quiet). y[i] is x[i] rounded, still held as a float.
 * ------------------------------------------------------------------------------------------- */
void orc_round_bf16(size_t count, const float* x, float* y) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        uint32_t u;
        memcpy(&u, &x[i], 4);
        if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
            u = (u | 0x00400000u) & 0xFFFF0000u;
        } else {
            const uint32_t lower = u & 0xFFFFu, odd = (u >> 16) & 1u;
            u &= 0xFFFF0000u;
            if (lower > 0x8000u || (lower == 0x8000u && odd)) u += 0x10000u;
        }
        memcpy(&y[i], &u, 4);
    }
}

/* ---------------------------------------------------------------------------------------------
 * tanh and sigmoid: cudnnActivationForward/Backward with CUDNN_ACTIVATION_TANH / _SIGMOID, selected
 * by the layer type at layer.cu:362-369 and run through the same two call sites as ReLU
 * (layer.cu:774-781, 802-811). Backward uses the output only: tanh' = 1 - y^2, sigmoid' = y (1 - y).
 * Evaluated in double and rounded once.
 * ------------------------------------------------------------------------------------------- */
void orc_tanh_fwd(size_t count, const float* x, float* y) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) y[i] = (float)tanh((double)x[i]);
}

void orc_tanh_bwd(size_t count, const float* y, const float* dy, float* dx) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) dx[i] = (float)((double)dy[i] * (1.0 - (double)y[i] * (double)y[i]));
}

void orc_sigmoid_fwd(size_t count, const float* x, float* y) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) y[i] = (float)(1.0 / (1.0 + exp(-(double)x[i])));
}

void orc_sigmoid_bwd(size_t count, const float* y, const float* dy, float* dx) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) dx[i] = (float)((double)dy[i] * (double)y[i] * (1.0 - (double)y[i]));
}

/* ---------------------------------------------------------------------------------------------
 * Max pooling: CUDNN_POOLING_MAX, NOT_PROPAGATE_NAN (layer.cu:416-428, 875-882, 903-912).
 * Padding positions never win. Backward: dy of each window goes to the window's first maximum in
 * row-major order (PARITY UNPINNED tie rule, see header); windows are visited in row-major order
 * so overlapping contributions add in that order.
 * ------------------------------------------------------------------------------------------- */
void orc_maxpool_fwd(const orc_shape* g, const float* x, float* y) {
    const int N = g->n, C = g->c, H = g->h, W = g->w, R = g->r, S = g->s;
    const int P = orc_out_dim(H, g->pad_h, R, g->stride_h), Q = orc_out_dim(W, g->pad_w, S, g->stride_w);
#pragma omp parallel for schedule(static)
    for (long nc = 0; nc < (long)N * C; nc++) {
        const float* xp = x + (size_t)nc * H * W;
        float* yp = y + (size_t)nc * P * Q;
        for (int p = 0; p < P; p++) for (int q = 0; q < Q; q++) {
            float m = -FLT_MAX;
            for (int r = 0; r < R; r++) for (int s = 0; s < S; s++) {
                const int ih = p * g->stride_h - g->pad_h + r, iw = q * g->stride_w - g->pad_w + s;
                if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                const float v = xp[(size_t)ih * W + iw];
                if (v > m) m = v;
            }
            yp[(size_t)p * Q + q] = m;
        }
    }
}

void orc_maxpool_bwd(const orc_shape* g, const float* x, const float* y, const float* dy, float* dx) {
    const int N = g->n, C = g->c, H = g->h, W = g->w, R = g->r, S = g->s;
    const int P = orc_out_dim(H, g->pad_h, R, g->stride_h), Q = orc_out_dim(W, g->pad_w, S, g->stride_w);
    (void)y;
#pragma omp parallel for schedule(static)
    for (long nc = 0; nc < (long)N * C; nc++) {
        const float* xp = x + (size_t)nc * H * W;
        const float* dyp = dy + (size_t)nc * P * Q;
        float* dxp = dx + (size_t)nc * H * W;
        for (long i = 0; i < (long)H * W; i++) dxp[i] = 0.0f;
        for (int p = 0; p < P; p++) for (int q = 0; q < Q; q++) {
            float m = -FLT_MAX; long arg = -1;
            for (int r = 0; r < R; r++) for (int s = 0; s < S; s++) {
                const int ih = p * g->stride_h - g->pad_h + r, iw = q * g->stride_w - g->pad_w + s;
                if (ih < 0 || ih >= H || iw < 0 || iw >= W) continue;
                const float v = xp[(size_t)ih * W + iw];
                if (arg < 0) arg = (long)ih * W + iw; /* first valid position wins if nothing exceeds -FLT_MAX */
                if (v > m) { m = v; arg = (long)ih * W + iw; }
            }
            if (arg >= 0) dxp[arg] += dyp[(size_t)p * Q + q];
        }
    }
}

/* ---------------------------------------------------------------------------------------------
 * LRN across channels (no counterpart in the reference): window 5, alpha 1e-4, beta 0.75, k 2.
 * scale_c = k + (alpha/5) * sum_{c' in [c-2,c+2]} x_c'^2 ;  y_c = x_c * scale_c^-beta
 * dx_c = dy_c * scale_c^-beta - (2*alpha*beta/5) * x_c * sum_{c' in [c-2,c+2]} dy_c' * y_c' / scale_c'
 * ------------------------------------------------------------------------------------------- */
#define LRN_WIN 5
#define LRN_ALPHA 1e-4f
#define LRN_BETA 0.75f
#define LRN_K 2.0f

void orc_lrn_fwd(int n, int c, int hw, const float* x, float* y) {
#pragma omp parallel for schedule(static)
    for (long ni = 0; ni < (long)n * hw; ni++) {
        const int in = (int)(ni / hw), i = (int)(ni % hw);
        const float* xp = x + (size_t)in * c * hw + i;
        float* yp = y + (size_t)in * c * hw + i;
        for (int ch = 0; ch < c; ch++) {
            float ss = 0.0f;
            for (int d = -(LRN_WIN / 2); d <= LRN_WIN / 2; d++) {
                const int cc = ch + d;
                if (cc < 0 || cc >= c) continue;
                const float v = xp[(size_t)cc * hw];
                ss += v * v;
            }
            const float scale = LRN_K + (LRN_ALPHA / LRN_WIN) * ss;
            yp[(size_t)ch * hw] = xp[(size_t)ch * hw] * powf(scale, -LRN_BETA);
        }
    }
}

void orc_lrn_bwd(int n, int c, int hw, const float* x, const float* y, const float* dy, float* dx) {
#pragma omp parallel
    {
        float* scale = (float*)malloc(sizeof(float) * (size_t)c);
#pragma omp for schedule(static)
        for (long ni = 0; ni < (long)n * hw; ni++) {
            const int in = (int)(ni / hw), i = (int)(ni % hw);
            const size_t base = (size_t)in * c * hw + i;
            for (int ch = 0; ch < c; ch++) {
                float ss = 0.0f;
                for (int d = -(LRN_WIN / 2); d <= LRN_WIN / 2; d++) {
                    const int cc = ch + d;
                    if (cc < 0 || cc >= c) continue;
                    const float v = x[base + (size_t)cc * hw];
                    ss += v * v;
                }
                scale[ch] = LRN_K + (LRN_ALPHA / LRN_WIN) * ss;
            }
            for (int ch = 0; ch < c; ch++) {
                float t = 0.0f;
                for (int d = -(LRN_WIN / 2); d <= LRN_WIN / 2; d++) {
                    const int cc = ch + d;
                    if (cc < 0 || cc >= c) continue;
                    t += dy[base + (size_t)cc * hw] * y[base + (size_t)cc * hw] / scale[cc];
                }
                dx[base + (size_t)ch * hw] = dy[base + (size_t)ch * hw] * powf(scale[ch], -LRN_BETA)
                                             - (2.0f * LRN_ALPHA * LRN_BETA / LRN_WIN) * x[base + (size_t)ch * hw] * t;
            }
        }
        free(scale);
    }
}

/* ---------------------------------------------------------------------------------------------
 * Softmax: CUDNN_SOFTMAX_ACCURATE (max subtracted), per sample (layer.cu:824-832, 853-862).
 * ------------------------------------------------------------------------------------------- */
void orc_softmax_fwd(int n, int classes, const float* x, float* y) {
    for (int i = 0; i < n; i++) {
        const float* xr = x + (size_t)i * classes;
        float* yr = y + (size_t)i * classes;
        float m = xr[0];
        for (int j = 1; j < classes; j++) if (xr[j] > m) m = xr[j];
        double sum = 0.0;
        for (int j = 0; j < classes; j++) { yr[j] = expf(xr[j] - m); sum += yr[j]; }
        const float inv = (float)(1.0 / sum);
        for (int j = 0; j < classes; j++) yr[j] *= inv;
    }
}

void orc_softmax_bwd(int n, int classes, const float* y, const float* dy, float* dx) {
    for (int i = 0; i < n; i++) {
        const float* yr = y + (size_t)i * classes;
        const float* dr = dy + (size_t)i * classes;
        float* xr = dx + (size_t)i * classes;
        double dot = 0.0;
        for (int j = 0; j < classes; j++) dot += (double)dr[j] * (double)yr[j];
        const float d = (float)dot;
        for (int j = 0; j < classes; j++) xr[j] = yr[j] * (dr[j] - d);
    }
}

/* calculateDiffTensor (network.cu:3-8) */
void orc_sub(size_t count, const float* a, const float* b, float* r) {
    for (size_t i = 0; i < count; i++) r[i] = a[i] - b[i];
}

float orc_softmax_ce_fwd(int n, int classes, const float* logits, const int32_t* labels, float* prob) {
    orc_softmax_fwd(n, classes, logits, prob);
    double loss = 0.0;
    for (int i = 0; i < n; i++) {
        float p = prob[(size_t)i * classes + labels[i]];
        if (p < FLT_MIN) p = FLT_MIN;
        loss -= log((double)p);
    }
    return (float)(loss / n);
}

void orc_softmax_ce_bwd(int n, int classes, const float* prob, const int32_t* labels, float* dlogits) {
    const float inv = 1.0f / (float)n;
    for (int i = 0; i < n; i++)
        for (int j = 0; j < classes; j++) {
            const float t = (j == labels[i]) ? 1.0f : 0.0f;
            dlogits[(size_t)i * classes + j] = (prob[(size_t)i * classes + j] - t) * inv;
        }
}

float orc_cross_entropy_dense(int n, int classes, const float* prob, const float* target) {
    double loss = 0.0;
    for (int i = 0; i < n; i++)
        for (int j = 0; j < classes; j++) {
            const float t = target[(size_t)i * classes + j];
            if (t == 0.0f) continue;
            float p = prob[(size_t)i * classes + j];
            if (p < FLT_MIN) p = FLT_MIN;
            loss -= (double)t * log((double)p);
        }
    return (float)(loss / n);
}

/* ---------------------------------------------------------------------------------------------
 * Seeded synthetic data. The reference draws from an unseeded mt19937 (layer.cu:925-967,
 * network.cu:819-829); here every element is a pure function of (seed, stream, index):
 * splitmix64 finaliser over a per-stream key, Box-Muller in double for normals.
 * ------------------------------------------------------------------------------------------- */
static uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

uint64_t orc_rng_u64(uint64_t seed, uint64_t stream, uint64_t i) {
    const uint64_t key = mix64(seed ^ mix64(stream));
    return mix64(key + i * 0x9E3779B97F4A7C15ull);
}

static double u01(uint64_t r) { return ((double)(r >> 11) + 0.5) * (1.0 / 9007199254740992.0); }

void orc_fill_normal(float* p, size_t count, uint64_t seed, uint64_t stream, float mean, float std) {
    const double two_pi = 6.283185307179586476925286766559;
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < count; i++) {
        const double u1 = u01(orc_rng_u64(seed, stream, 2 * i));
        const double u2 = u01(orc_rng_u64(seed, stream, 2 * i + 1));
        const double z = sqrt(-2.0 * log(u1)) * cos(two_pi * u2);
        p[i] = (float)((double)mean + (double)std * z);
    }
}

void orc_fill_uniform(float* p, size_t count, uint64_t seed, uint64_t stream, float lo, float hi) {
    for (size_t i = 0; i < count; i++)
        p[i] = (float)((double)lo + ((double)hi - (double)lo) * u01(orc_rng_u64(seed, stream, i)));
}

void orc_fill_labels(int32_t* p, size_t count, uint64_t seed, uint64_t stream, int classes) {
    for (size_t i = 0; i < count; i++)
        p[i] = (int32_t)(((orc_rng_u64(seed, stream, i) >> 32) * (uint64_t)classes) >> 32);
}
