/* TEST INFRASTRUCTURE - the convolutions of the CPU checker as im2col + cache-blocked SGEMM.
 *
 * Same layer math as vdnn_oracle.c (layer.cu:560-569, 616-625, 651-660), arranged for speed: it is what the bench's
 * cpu_baseline times. The im2col matrix is never stored: the routine that packs a panel of the GEMM's B operand
 * gathers it from the tensor. Packed panels (BLIS order: A in strips of MR rows, B in strips of NR columns), a
 * 6 x 16 AVX2 / FMA micro-kernel, OpenMP over samples x pixel blocks. Float accumulation in a different order than
 * the direct loops, so results agree with them to rounding (tests/test_oracle_layers.py), not to the bit; the
 * parity tests of the GPU path use the direct loops (double accumulation), never this file.
 * Stride-1 convolutions only (every VGG16 layer); the callers fall back to the direct loops otherwise.
 */
#include <immintrin.h>
#include <omp.h>
#include <stdlib.h>
#include <string.h>

#include "vdnn_oracle.h"

enum { MR = 6, NR = 16, KC = 256, NC = 384 };

/* c[MR][NR] (row stride ldc) = (accumulate ? c : 0) + a_panel[kc][MR] * b_panel[kc][NR] */
static void micro_6x16(int kc, const float* restrict a, const float* restrict b, float* restrict c, long ldc, int accumulate) {
    __m256 acc[MR][2];
    for (int i = 0; i < MR; i++) {
        if (accumulate) { acc[i][0] = _mm256_loadu_ps(c + i * ldc); acc[i][1] = _mm256_loadu_ps(c + i * ldc + 8); }
        else { acc[i][0] = _mm256_setzero_ps(); acc[i][1] = _mm256_setzero_ps(); }
    }
    for (int p = 0; p < kc; p++) {
        const __m256 b0 = _mm256_load_ps(b + (long)p * NR), b1 = _mm256_load_ps(b + (long)p * NR + 8);
        for (int i = 0; i < MR; i++) {
            const __m256 av = _mm256_broadcast_ss(a + (long)p * MR + i);
            acc[i][0] = _mm256_fmadd_ps(av, b0, acc[i][0]);
            acc[i][1] = _mm256_fmadd_ps(av, b1, acc[i][1]);
        }
    }
    for (int i = 0; i < MR; i++) { _mm256_storeu_ps(c + i * ldc, acc[i][0]); _mm256_storeu_ps(c + i * ldc + 8, acc[i][1]); }
}

/* C[m][n] block (rows i0.., columns j0.. of a row-major matrix with row stride ldc) from packed panels; edge tiles go
 * through a full-size scratch tile */
static void macro_kernel(int mc, int nc, int kc, const float* Ap, const float* Bp, float* C, long ldc, int accumulate) {
    float tile[MR * NR] __attribute__((aligned(32)));
    for (int jr = 0; jr < nc; jr += NR) {
        const int nr = nc - jr < NR ? nc - jr : NR;
        for (int ir = 0; ir < mc; ir += MR) {
            const int mr = mc - ir < MR ? mc - ir : MR;
            const float* a = Ap + (long)(ir / MR) * kc * MR;
            const float* b = Bp + (long)(jr / NR) * kc * NR;
            float* c = C + (long)ir * ldc + jr;
            if (mr == MR && nr == NR) { micro_6x16(kc, a, b, c, ldc, accumulate); continue; }
            memset(tile, 0, sizeof(tile));
            if (accumulate) for (int i = 0; i < mr; i++) for (int j = 0; j < nr; j++) tile[i * NR + j] = c[i * ldc + j];
            micro_6x16(kc, a, b, tile, NR, accumulate);
            for (int i = 0; i < mr; i++) for (int j = 0; j < nr; j++) c[i * ldc + j] = tile[i * NR + j];
        }
    }
}

/* rows [0, M) x reduction [p0, p0+kc) of a row-major matrix A (row stride lda) -> strips of MR rows, zero padded */
static void pack_a_rows(const float* A, long lda, int M, int p0, int kc, float* Ap) {
    for (int i0 = 0; i0 < M; i0 += MR) {
        for (int p = 0; p < kc; p++)
            for (int i = 0; i < MR; i++) Ap[(long)(i0 / MR) * kc * MR + (long)p * MR + i] = i0 + i < M ? A[(long)(i0 + i) * lda + p0 + p] : 0.0f;
    }
}

static float* alloc32(size_t floats) {
    void* p = NULL;
    if (posix_memalign(&p, 64, floats * sizeof(float) + 64) != 0) abort();
    return (float*)p;
}

/* ---- forward and backward data (stride 1): Out[m][pix] = sum_kk Wm[m][kk] * gather(src, kk, pix) -------------------
 * kk = (ch, r, s). Forward: m = k, ch = c, the tap reads src[ch][p - ph + r][q - pw + s]. Backward data: m = c, ch = k,
 * the tap reads dy[ch][h + ph - r][w + pw - s] (the caller hands in Wm with rows and reduction already swapped). */
typedef struct { int flip; int CH, H, W, OH, OW, R, S, ph, pw; } gather_geo;

static void pack_b_gather(const gather_geo* g, const float* src_n, int kk0, int kc, int j0, int nc, float* Bp) {
    const int RS = g->R * g->S;
    for (int jr = 0; jr < nc; jr += NR) {
        float* bp = Bp + (long)(jr / NR) * kc * NR;
        int oh[NR], ow[NR];
        for (int j = 0; j < NR; j++) {
            const int pix = j0 + jr + j;
            if (jr + j < nc) { oh[j] = pix / g->OW; ow[j] = pix - oh[j] * g->OW; }
            else { oh[j] = -0x10000; ow[j] = -0x10000; } /* past the block: reads as outside the image */
        }
        /* sixteen pixels of one image row read sixteen consecutive input elements through any tap */
        const int one_row = jr + NR <= nc && oh[0] == oh[NR - 1];
        int kk = kk0, ch = kk0 / RS, tap = kk0 - ch * RS;
        for (int p = 0; p < kc; p++, kk++) {
            const int r = tap / g->S, s = tap - r * g->S;
            const int dh = g->flip ? g->ph - r : r - g->ph, dw = g->flip ? g->pw - s : s - g->pw;
            const float* plane = src_n + (long)ch * g->H * g->W;
            float* dst = bp + (long)p * NR;
            const int ih0 = oh[0] + dh, iw0 = ow[0] + dw;
            if (one_row && (unsigned)ih0 < (unsigned)g->H && iw0 >= 0 && iw0 + NR <= g->W) {
                memcpy(dst, plane + (long)ih0 * g->W + iw0, sizeof(float) * NR);
            } else if (one_row && !((unsigned)ih0 < (unsigned)g->H)) {
                memset(dst, 0, sizeof(float) * NR);
            } else {
                for (int j = 0; j < NR; j++) {
                    const int ih = oh[j] + dh, iw = ow[j] + dw;
                    dst[j] = ((unsigned)ih < (unsigned)g->H && (unsigned)iw < (unsigned)g->W) ? plane[(long)ih * g->W + iw] : 0.0f;
                }
            }
            if (++tap == RS) { tap = 0; ch++; }
        }
    }
}

/* Out[n][m][pix] = Wm[m][kk] x gather + bias[m] for every sample; Wm is M x KK row-major */
static void conv_gemm(const gather_geo* g, int N, int M, const float* Wm, const float* src, long src_sample, const float* bias, float* out) {
    const int KK = g->CH * g->R * g->S, OPIX = g->OH * g->OW;
    const int mstrips = (M + MR - 1) / MR;
    /* the whole filter matrix packed once, per reduction block: block b starts at Apack + b * mstrips * MR * KC */
    const int kblocks = (KK + KC - 1) / KC;
    float* Apack = alloc32((size_t)kblocks * mstrips * MR * KC);
    for (int b = 0; b < kblocks; b++) {
        const int kc = KK - b * KC < KC ? KK - b * KC : KC;
        pack_a_rows(Wm, KK, M, b * KC, kc, Apack + (size_t)b * mstrips * MR * KC);
    }
    const int jblocks = (OPIX + NC - 1) / NC;
    const long units = (long)N * jblocks;
#pragma omp parallel
    {
        float* Bp = alloc32((size_t)KC * NC);
#pragma omp for schedule(dynamic, 1)
        for (long u = 0; u < units; u++) {
            const int n = (int)(u / jblocks), j0 = (int)(u % jblocks) * NC;
            const int nc = OPIX - j0 < NC ? OPIX - j0 : NC;
            float* C = out + (long)n * M * OPIX + j0;
            for (int b = 0; b < kblocks; b++) {
                const int kc = KK - b * KC < KC ? KK - b * KC : KC;
                pack_b_gather(g, src + (long)n * src_sample, b * KC, kc, j0, nc, Bp);
                macro_kernel(M, nc, kc, Apack + (size_t)b * mstrips * MR * KC, Bp, C, OPIX, b > 0);
            }
            if (bias)
                for (int m = 0; m < M; m++) { float* row = C + (long)m * OPIX; for (int j = 0; j < nc; j++) row[j] += bias[m]; }
        }
        free(Bp);
    }
    free(Apack);
}

int orc_blocked_conv_ok(const orc_shape* g) { return g->stride_h == 1 && g->stride_w == 1; }

void orc_blocked_conv_fwd(const orc_shape* s, const float* x, const float* w, const float* bias, float* y) {
    const int P = orc_out_dim(s->h, s->pad_h, s->r, 1), Q = orc_out_dim(s->w, s->pad_w, s->s, 1);
    const gather_geo g = {0, s->c, s->h, s->w, P, Q, s->r, s->s, s->pad_h, s->pad_w};
    conv_gemm(&g, s->n, s->k, w, x, (long)s->c * s->h * s->w, bias, y); /* KCRS is K x (c,r,s) row-major already */
}

void orc_blocked_conv_bwd_data(const orc_shape* s, const float* dy, const float* w, float* dx) {
    const int P = orc_out_dim(s->h, s->pad_h, s->r, 1), Q = orc_out_dim(s->w, s->pad_w, s->s, 1);
    const int RS = s->r * s->s;
    /* Wt[c][(k, r, s)] = w[k][c][r][s] */
    float* Wt = alloc32((size_t)s->c * s->k * RS);
    for (int k = 0; k < s->k; k++)
        for (int c = 0; c < s->c; c++)
            memcpy(Wt + ((size_t)c * s->k + k) * RS, w + ((size_t)k * s->c + c) * RS, sizeof(float) * RS);
    const gather_geo g = {1, s->k, P, Q, s->h, s->w, s->r, s->s, s->pad_h, s->pad_w};
    conv_gemm(&g, s->n, s->c, Wt, dy, (long)s->k * P * Q, NULL, dx);
    free(Wt);
}

/* ---- backward filter: dW[k][(c,r,s)] = sum_n sum_pix dy[n][k][pix] * x[n][c][p - ph + r][q - pw + s] ------------------
 * Per sample a GEMM with the pixels as reduction; every thread sums its samples into a copy of its own, the copies are
 * added in thread order and the update w += alpha dW is applied once. */
static void pack_b_columns(const orc_shape* s, int P, int Q, const float* x_n, int pix0, int kc, int j0, int nc, float* Bp) {
    const int RS = s->r * s->s;
    for (int jr = 0; jr < nc; jr += NR) {
        float* bp = Bp + (long)(jr / NR) * kc * NR;
        int ch[NR], dh[NR], dw[NR];
        for (int j = 0; j < NR; j++) {
            const int col = j0 + jr + j;
            if (jr + j < nc) { ch[j] = col / RS; const int tap = col - ch[j] * RS; dh[j] = tap / s->s - s->pad_h; dw[j] = tap % s->s - s->pad_w; }
            else ch[j] = -1;
        }
        for (int p = 0; p < kc; p++) {
            const int pix = pix0 + p, oh = pix / Q, ow = pix - oh * Q;
            for (int j = 0; j < NR; j++) {
                float v = 0.0f;
                if (ch[j] >= 0) {
                    const int ih = oh + dh[j], iw = ow + dw[j];
                    if ((unsigned)ih < (unsigned)s->h && (unsigned)iw < (unsigned)s->w) v = x_n[((long)ch[j] * s->h + ih) * s->w + iw];
                }
                bp[(long)p * NR + j] = v;
            }
        }
    }
    (void)P;
}

void orc_blocked_conv_bwd_filter_sgd(const orc_shape* s, const float* x, const float* dy, float* w, float alpha) {
    const int P = orc_out_dim(s->h, s->pad_h, s->r, 1), Q = orc_out_dim(s->w, s->pad_w, s->s, 1);
    const int OPIX = P * Q, K = s->k, COLS = s->c * s->r * s->s;
    const int mstrips = (K + MR - 1) / MR;
    int threads = orc_get_threads();
    if (threads > s->n) threads = s->n;
    float* sums = alloc32((size_t)threads * K * COLS);
    memset(sums, 0, sizeof(float) * (size_t)threads * K * COLS);
#pragma omp parallel num_threads(threads)
    {
        const int t = omp_get_thread_num();
        float* mine = sums + (size_t)t * K * COLS;
        float* Ap = alloc32((size_t)mstrips * MR * KC);
        float* Bp = alloc32((size_t)KC * NC);
#pragma omp for schedule(static)
        for (int n = 0; n < s->n; n++) {
            const float* dy_n = dy + (long)n * K * OPIX;
            const float* x_n = x + (long)n * s->c * s->h * s->w;
            for (int pix0 = 0; pix0 < OPIX; pix0 += KC) {
                const int kc = OPIX - pix0 < KC ? OPIX - pix0 : KC;
                pack_a_rows(dy_n, OPIX, K, pix0, kc, Ap);
                for (int j0 = 0; j0 < COLS; j0 += NC) {
                    const int nc = COLS - j0 < NC ? COLS - j0 : NC;
                    pack_b_columns(s, P, Q, x_n, pix0, kc, j0, nc, Bp);
                    macro_kernel(K, nc, kc, Ap, Bp, mine + j0, COLS, 1);
                }
            }
        }
        free(Ap); free(Bp);
    }
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)K * COLS; i++) {
        float acc = 0.0f;
        for (int t = 0; t < threads; t++) acc += sums[(size_t)t * K * COLS + i];
        w[i] = w[i] + alpha * acc;
    }
    free(sums);
}
