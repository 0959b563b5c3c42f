// Forward of 3x3 / stride 1 / padding 1 layers with at most four input channels and at most 64 output channels (the
// first layer of VGG16). The pass writes 64 values per pixel and reads three: it is bound by its stores, and the
// reduction is 27 deep - a tile engine's per-tile set-up (two slices, then an epilogue) costs more than the tile.
// Here nothing is staged and nothing is shared: a wavefront owns 32 consecutive pixels at a time (lanes along the
// pixels, so every load and store of a wavefront covers one 128-byte run of a plane), keeps the whole filter bank in
// registers as the A operand of v_mfma_f32_32x32x2_f32 (14 steps of two reduction indices for 27), fetches the 14
// input values of its lane straight from memory (neighbouring taps hit the same lines), multiplies, adds the bias
// and stores - then moves on to the next 32 pixels of its run (a wavefront's 64 output rows are 64 sequential
// streams). The next 32 pixels' values are fetched before
// the current ones are multiplied. Activations float or bfloat16 (converted on the way in; products of two
// bfloat16 values are exact in float, as on the bfloat16 matrix cores).
#pragma once
#include "conv_loaders.h"

namespace vdnn {

template <class E> __device__ __forceinline__ void buf_store_e(__amdgpu_buffer_rsrc_t r, float v, int voff, int soff);
template <> __device__ __forceinline__ void buf_store_e<float>(__amdgpu_buffer_rsrc_t r, float v, int voff, int soff) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), r, voff, soff, 0);
}
template <> __device__ __forceinline__ void buf_store_e<bf16_t>(__amdgpu_buffer_rsrc_t r, float v, int voff, int soff) {
    __builtin_amdgcn_raw_buffer_store_b16((unsigned short)float_to_bf16_bits(v), r, voff, soff, 0);
}

// x and y below 2 GiB each (offsets are 32-bit), N*H*W below 2^31. UP = blocks of 32 pixels per unit: with two, the
// halves of the wavefront exchange what they hold of the two blocks (v_permlane32_swap), so that one store covers 64
// consecutive pixels of one output row instead of 32 pixels of two rows - whole 128-byte lines also with two-byte
// elements.
template <int CC, int RBLK, int UP, class E>
__global__ void __launch_bounds__(256) conv_fwd_smallc3x3_kernel(const E* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
                                                                  E* __restrict__ y, int N, int K, int H, int W, int relu) {
    static_assert(UP == 1 || UP == 2, "one block of 32 pixels per unit, or two");
    constexpr int KRED = 9 * CC, ES = ElemBytes<E>::V;
    // with an odd reduction length the bias rides in the unused last index (input value 1); otherwise it is added afterwards
    constexpr bool BIAS_SLOT = KRED % 2 == 1;
    constexpr int KS = (KRED + 1) / 2;
    const int lane = threadIdx.x & 63, l32 = lane & 31, lk = lane >> 5;
    const int PQ = H * W;
    const int total = N * PQ;
    const int nunits = (total + 32 * UP - 1) / (32 * UP);
    const int nwaves = (int)gridDim.x * 4;
    const int wave0 = (int)blockIdx.x * 4 + (int)(threadIdx.x >> 6);
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(x, clamp_range((long)N * CC * PQ * ES));
    const __amdgpu_buffer_rsrc_t ro = make_rsrc(y, clamp_range((long)N * K * PQ * ES));

    // A operand: step t multiplies reduction indices 2t (lanes 0-31) and 2t + 1 (lanes 32-63); index = (c, r, s) in the
    // filter's own order. The lane's input offset for each step, and its tap's place r*3 + s in the window (9: none),
    // four bits per step.
    float a[RBLK][KS];
    int koff[KS];
    unsigned long long ktap[2] = {0, 0};
#pragma unroll
    for (int t = 0; t < KS; t++) {
        const int k = 2 * t + lk;
        const bool live = k < KRED;
        const int kk = live ? k : 0;
        const int c = kk / 9, rs9 = kk % 9;
        koff[t] = (c * PQ + (rs9 / 3 - 1) * W + (rs9 % 3 - 1)) * ES;
        ktap[t / 16] |= (unsigned long long)(live ? rs9 : 9) << (4 * (t % 16));
#pragma unroll
        for (int i = 0; i < RBLK; i++) {
            const int m = 32 * i + l32;
            float v = (live && m < K) ? w[(long)m * KRED + k] : 0.0f;
            if (BIAS_SLOT && k == KRED && bias && m < K) v = bias[m];
            a[i][t] = v;
        }
    }
    static_assert(KS <= 32, "four bits per step in two 64-bit words");
    float bv[BIAS_SLOT ? 1 : RBLK][BIAS_SLOT ? 1 : 16];
    if (!BIAS_SLOT) {
#pragma unroll
        for (int i = 0; i < RBLK; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = 32 * i + 8 * (v / 4) + 4 * lk + (v % 4);
                bv[i][v] = (bias && m < K) ? bias[m] : 0.0f;
            }
    }

    // a wavefront walks a run of consecutive units (its 64 output rows are 64 sequential streams); the lane's pixel
    // of each block (sample, row, column) is carried from unit to unit
    const int per = (nunits + nwaves - 1) / nwaves;
    const int first = wave0 * per, last = first + per < nunits ? first + per : nunits;
    struct Pix { int px, n, p, q; };
    Pix pix[UP];
#pragma unroll
    for (int u = 0; u < UP; u++) {
        pix[u].px = (first * UP + u) * 32 + l32;
        const int pc = pix[u].px < total ? pix[u].px : 0;
        pix[u].n = pc / PQ;
        const int pq = pc - pix[u].n * PQ;
        pix[u].p = pq / W; pix[u].q = pq - pix[u].p * W;
    }
    // byte offset in y of the pixel's value in output channel 0 (UP == 2) or 4*lk (UP == 1), or out of range
    auto fetch = [&](bool in_run, Pix& px, float (&dst)[KS], int& out_base) {
        const bool inside = in_run && px.px < total;
        const int pq = px.p * W + px.q;
        const int base = (px.n * CC * PQ + pq) * ES;
        // the nine places of the window that lie inside the image, as bits r*3 + s
        const unsigned colok = (px.q > 0 ? 1u : 0u) | 2u | (px.q < W - 1 ? 4u : 0u);
        const unsigned win = inside ? ((px.p > 0 ? colok : 0u) | (colok << 3) | (px.p < H - 1 ? colok << 6 : 0u)) : 0u;
#pragma unroll
        for (int t = 0; t < KS; t++) {
            const unsigned tap = (unsigned)(ktap[t / 16] >> (4 * (t % 16))) & 15u;
            float v = buf_load_e<E>(rs, ((win >> tap) & 1u) ? base + koff[t] : OOB, 0);
            if (BIAS_SLOT && t == KS - 1) v = lk ? 1.0f : v; // reduction index KRED: the bias' factor
            dst[t] = v;
        }
        out_base = inside ? ((px.n * K + (UP == 1 ? 4 * lk : 0)) * PQ + pq) * ES : OOB;
        // one unit further
        px.px += 32 * UP; px.q += 32 * UP;
        while (px.q >= W) { px.q -= W; px.p += 1; }
        while (px.p >= H) { px.p -= H; px.n += 1; }
    };

    float b[UP][KS];
    int obase[UP];
#pragma unroll
    for (int u = 0; u < UP; u++) fetch(first < last, pix[u], b[u], obase[u]);
    for (int unit = first; unit < last; unit++) {
        float bn[UP][KS];
        int obase_next[UP];
#pragma unroll
        for (int u = 0; u < UP; u++) fetch(unit + 1 < last, pix[u], bn[u], obase_next[u]);
        floatx16 acc[UP][RBLK];
#pragma unroll
        for (int u = 0; u < UP; u++)
#pragma unroll
            for (int i = 0; i < RBLK; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[u][i][v] = 0.0f;
#pragma unroll
        for (int t = 0; t < KS; t++)
#pragma unroll
            for (int u = 0; u < UP; u++)
#pragma unroll
                for (int i = 0; i < RBLK; i++) acc[u][i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][t], b[u][t], acc[u][i], 0, 0, 0);
        // the lane's store address with two blocks: lanes 0-31 write the first block's pixels, lanes 32-63 the second's
        const int obase2 = UP == 2 ? (lk ? obase[UP - 1] : obase[0]) : 0;
#pragma unroll
        for (int i = 0; i < RBLK; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int mrow = 32 * i + 8 * (v / 4) + (v % 4); // the lane holds row mrow + 4*lk
                float r[UP];
#pragma unroll
                for (int u = 0; u < UP; u++) {
                    r[u] = acc[u][i][v];
                    if (!BIAS_SLOT && bias) r[u] += bv[i][v];
                    if (relu) r[u] = relu_value(r[u]);
                }
                // rows past K (the last block of a layer with fewer channels) are sent out of range
                if constexpr (UP == 1) {
                    // the lane's offset carries the 4*lk rows
                    const int soff = __builtin_amdgcn_readfirstlane(mrow * PQ * ES);
                    buf_store_e<E>(ro, r[0], (mrow + 4 * lk < K) ? obase[0] : OOB, soff);
                } else {
                    // [first block: rows mrow | mrow + 4] x [second block: rows mrow | mrow + 4]  ->
                    // row mrow of both blocks, row mrow + 4 of both blocks (the builtin's result is read through a
                    // 64-bit integer: subscripts of the two-element vector both gave its first element)
                    const unsigned long long sw = __builtin_bit_cast(unsigned long long,
                        __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(unsigned, r[0]), __builtin_bit_cast(unsigned, r[UP - 1]), false, false));
                    const int soff0 = __builtin_amdgcn_readfirstlane(mrow * PQ * ES), soff1 = __builtin_amdgcn_readfirstlane((mrow + 4) * PQ * ES);
                    buf_store_e<E>(ro, __builtin_bit_cast(float, (unsigned)sw), (mrow < K) ? obase2 : OOB, soff0);
                    buf_store_e<E>(ro, __builtin_bit_cast(float, (unsigned)(sw >> 32)), (mrow + 4 < K) ? obase2 : OOB, soff1);
                }
            }
#pragma unroll
        for (int u = 0; u < UP; u++) {
#pragma unroll
            for (int t = 0; t < KS; t++) b[u][t] = bn[u][t];
            obase[u] = obase_next[u];
        }
    }
}

} // namespace vdnn

namespace vdnn {

// Backward filter of 3x3 / stride 1 / padding 1 layers with at most three input channels (9*C <= 32 columns), rows of
// whole groups of four pixels (W % 4 == 0, W >= 16). The pass reads dy once and is bound by that; the reduction runs
// over pixels, contiguous in dy and x, so - as in wgrad3x3_f32_kernel - a slice of pixels is fetched with 128-bit loads
// along the pixels into reduction-major LDS rows: 64 rows of dy, and one row of x per (channel, filter row) shifted by
// (r-1)*W, plus the element before and after each run. Slices are 64 pixels long: with 16 the barrier and the latency
// of a fetch (one slice ahead) cost more than the slice's four multiplies per wavefront. Column n = (c, r, s) of the
// product takes row (c, r) of x one place left / in place / one place right by s: every lane forms the three variants
// from one 128-bit read and picks its own. Four wavefronts share a slice's multiplies: 32 output channels x half of the
// slice's pixels each; the halves are added through LDS at the end. Partial sums of a reduction split go to the
// staging area as [split][K][C][3][3], which reduce_splits adds in split order.
struct WgradSmallC {
    const void* dy;
    const void* x;
    int N, K, H, W;
    float* partial; // [split][K][9*C]
    int kchunk;     // pixels per split, a multiple of WSC_SLICE
    // optional: the bias gradient's partial sums, [K][bias_splits] (split ks of channel m at m * bias_splits + ks). The
    // product has 32 columns of which 9*C are taken: column 9*C multiplies dy by one, so its sums are those of dy.
    float* bias_partial;
    int bias_splits;
};
constexpr int WSC_SLICE = 64;            // pixels per slice
constexpr int WSC_STRIDE = WSC_SLICE + 4; // LDS row stride in floats: 128-bit reads of 16 consecutive rows hit 16 different bank groups

template <int CC, class E>
__global__ void __launch_bounds__(NT) wgrad_smallc3x3_mfma_kernel(const WgradSmallC g) {
    constexpr int ROWS = 3 * CC, NCOL = 9 * CC, ES = ElemBytes<E>::V;
    constexpr int SL = WSC_SLICE, GPS = SL / 4; // groups of four pixels per slice
    static_assert(NCOL <= 32, "one block of 32 columns");
    static_assert(ROWS * GPS <= NT && 2 * ROWS <= 64, "one x group per thread");
    __shared__ __attribute__((aligned(16))) float As[2][64 * WSC_STRIDE];
    __shared__ __attribute__((aligned(16))) float Bs[2][ROWS * WSC_STRIDE];
    __shared__ float Hs[2][2][ROWS];
    __shared__ float Red[2][64][17]; // the second half's sums, [row block][lane][value]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int H = g.H, W = g.W, PQ = H * W;
    const int Kred = g.N * PQ;
    const int mtiles = (g.K + 63) / 64;
    const int mt = blockIdx.x % mtiles, ks = blockIdx.x / mtiles;
    const int m0 = mt * 64;
    const int k_begin = ks * g.kchunk;
    const int k_end = min(Kred, k_begin + g.kchunk);
    const E* dy = (const E*)g.dy;
    const E* x = (const E*)g.x;

    const int n_first = k_begin / PQ;
    const int n_last = k_end > k_begin ? (k_end - 1) / PQ : n_first;
    const __amdgpu_buffer_rsrc_t rsA = make_rsrc(dy + (long)n_first * g.K * PQ, clamp_range((long)(n_last - n_first + 1) * g.K * PQ * ES));
    const __amdgpu_buffer_rsrc_t rsB = make_rsrc(x + (long)n_first * CC * PQ, clamp_range((long)(n_last - n_first + 1) * CC * PQ * ES));

    // loaders: thread t fetches pixel group t % 16 of the dy rows t / 16 + 16 i; threads below 16*ROWS also that group
    // of x row t / 16 = (channel, filter row); lanes of wavefront 3 below 2*ROWS the element before / after the run of
    // row lane / 2
    const int pg = tid & (GPS - 1), rl = tid / GPS;
    int mrow[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { const int m = m0 + rl + 16 * i; mrow[i] = m < g.K ? m * PQ * ES : SENT; }
    int pqA, offA;
    {
        const int kk = k_begin + 4 * pg;
        const int n = kk / PQ, pq = kk - n * PQ;
        pqA = pq;
        offA = (n - n_first) * g.K * PQ * ES + pq * ES;
    }
    struct Cursor { int p, q, pos; };
    auto cursor_at = [&](int kk) {
        const int n = kk / PQ, pq = kk - n * PQ;
        Cursor c;
        c.p = pq / W; c.q = pq - c.p * W;
        c.pos = ((n - n_first) * CC * PQ + pq) * ES;
        return c;
    };
    auto advance = [&](Cursor& c) { // one slice further: several image rows when they are short, at most one sample
        c.q += SL; c.pos += SL * ES;
        while (c.q >= W) { c.q -= W; c.p += 1; }
        const bool next = c.p >= H;
        c.p -= next ? H : 0; c.pos += next ? (CC - 1) * PQ * ES : 0;
    };
    const bool loads_b = rl < ROWS;
    const int rB = rl % 3;
    const int colB = loads_b ? ((rl / 3) * PQ + (rB - 1) * W) * ES : SENT;
    Cursor cb = cursor_at(k_begin + 4 * pg);
    const bool loads_h = wave == 3 && lane < 2 * ROWS;
    const int side = lane & 1, rowH = (lane >> 1) % ROWS, rH = rowH % 3;
    const int colH = loads_h ? ((rowH / 3) * PQ + (rH - 1) * W) * ES + (side ? 4 * ES : -ES) : SENT;
    Cursor ch = cursor_at(k_begin + (side ? SL - 4 : 0));

    // what a slice's fetch leaves in registers; two slices are in flight (the pass is bound by the latency of dy)
    struct Fetched { floatx4 ra[4], rb; float rh; };
    Fetched fa, fb;
    fa.rh = 0.0f; fb.rh = 0.0f;
    auto fetch = [&](Fetched& f) {
#pragma unroll
        for (int i = 0; i < 4; i++) f.ra[i] = buf_load4_e<E>(rsA, mrow[i] + offA, 0);
        pqA += SL;
        const bool wrapA = pqA >= PQ; // H*W >= 64: one sample at most
        pqA -= wrapA ? PQ : 0;
        offA += wrapA ? (SL + (g.K - 1) * PQ) * ES : SL * ES;
        if (tid < ROWS * GPS) {
            const bool row_ok = (unsigned)(cb.p + rB - 1) < (unsigned)H;
            f.rb = buf_load4_e<E>(rsB, row_ok ? cb.pos + colB : OOB, 0);
        }
        advance(cb);
        if (wave == 3) {
            const bool used = (unsigned)(ch.p + rH - 1) < (unsigned)H && ch.q != (side ? W - 4 : 0);
            f.rh = buf_load_e<E>(rsB, used ? ch.pos + colH : OOB, 0);
            advance(ch);
        }
    };
    auto stash = [&](int buf, const Fetched& f) {
#pragma unroll
        for (int i = 0; i < 4; i++) *(floatx4*)(As[buf] + (rl + 16 * i) * WSC_STRIDE + 4 * pg) = f.ra[i];
        if (loads_b) *(floatx4*)(Bs[buf] + rl * WSC_STRIDE + 4 * pg) = f.rb;
        if (loads_h) Hs[buf][side][rowH] = f.rh;
    };

    floatx16 acc;
#pragma unroll
    for (int v = 0; v < 16; v++) acc[v] = 0.0f;
    const int rowblk = wave & 1, hf = wave >> 1; // this wavefront: 32 output channels, pixels 32*hf .. 32*hf + 31 of every slice
    // this lane's column (c, r, s): its row of x in LDS and which neighbour it takes
    const bool col_live = l32 < NCOL;
    const float idle = (g.bias_partial != nullptr && l32 == NCOL) ? 1.0f : 0.0f; // what a lane beyond the filter's columns multiplies by
    const int bro = col_live ? l32 / 3 : 0, sB = col_live ? l32 % 3 : 1;
    int qs = k_begin % W;

    const int nslices = (k_end - k_begin + SL - 1) / SL;
    // slice s is multiplied from LDS buffer s % 2; `f` holds slice s + 1 (fetched two slices ago): it is written to the
    // other buffer behind the multiplies, and the registers then take the fetch of slice s + 3
    fetch(fa);
    stash(0, fa);
    fetch(fb);
    fetch(fa);
    __syncthreads();
    auto slice_body = [&](int s, Fetched& f) {
        const int cur = s & 1;
        const float* arow = As[cur] + (32 * rowblk + l32) * WSC_STRIDE + 32 * hf + 4 * lk;
        const float* brow = Bs[cur] + bro * WSC_STRIDE + 32 * hf + 4 * lk;
#pragma unroll
        for (int gq = 0; gq < 4; gq++) { // eight pixels: four per half of the lanes
            const floatx4 a = *(const floatx4*)(arow + 8 * gq);
            const floatx4 v = *(const floatx4*)(brow + 8 * gq);
            const float* pp = (hf == 0 && gq == 0 && lk == 0) ? &Hs[cur][0][bro] : brow + 8 * gq - 1;
            const float* np = (hf == 1 && gq == 3 && lk == 1) ? &Hs[cur][1][bro] : brow + 8 * gq + 4;
            float prev = *pp, next = *np;
            int qg = qs + 32 * hf + 8 * gq + 4 * lk;
            while (qg >= W) qg -= W;
            prev = qg == 0 ? 0.0f : prev;     // left of the image
            next = qg == W - 4 ? 0.0f : next; // right of the image
            const float b0 = !col_live ? idle : sB == 0 ? prev : sB == 1 ? v.x : v.y;
            const float b1 = !col_live ? idle : sB == 0 ? v.x : sB == 1 ? v.y : v.z;
            const float b2 = !col_live ? idle : sB == 0 ? v.y : sB == 1 ? v.z : v.w;
            const float b3 = !col_live ? idle : sB == 0 ? v.z : sB == 1 ? v.w : next;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b0, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b1, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b2, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b3, acc, 0, 0, 0);
        }
        qs += SL;
        while (qs >= W) qs -= W;
        stash(cur ^ 1, f);
        __syncthreads();
        fetch(f);
    };
    for (int s = 0; s < nslices; s += 2) {
        slice_body(s, fb);
        if (s + 1 < nslices) slice_body(s + 1, fa);
    }

    // the two halves of the slices: wavefronts 2 and 3 hand their sums to 0 and 1 (fixed order: first half + second half)
    if (hf == 1) {
#pragma unroll
        for (int v = 0; v < 16; v++) Red[rowblk][lane][v] = acc[v];
    }
    __syncthreads();
    if (hf == 0 && col_live) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = m0 + 32 * rowblk + 8 * (v / 4) + 4 * lk + (v % 4);
            if (m >= g.K) continue;
            g.partial[((long)ks * g.K + m) * NCOL + l32] = acc[v] + Red[rowblk][lane][v];
        }
    }
    if (hf == 0 && g.bias_partial != nullptr && l32 == NCOL) {
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const int m = m0 + 32 * rowblk + 8 * (v / 4) + 4 * lk + (v % 4);
            if (m >= g.K) continue;
            g.bias_partial[(long)m * g.bias_splits + ks] = acc[v] + Red[rowblk][lane][v];
        }
    }
}

} // namespace vdnn

namespace vdnn {

// Backward data of 3x3 / stride 1 / padding 1 layers with at most three input channels and at most 64 output channels
// (the first layer). dx has three rows per pixel, far too few for a matrix tile, and the vector-ALU kernel read dy
// nine times per pixel. Here the products are formed once, on the matrix cores, as a 1x1 convolution with 9*C <= 32
// output rows over dy, one image row at a time:
//     T_j[(c,r,s)][q] = sum over k of w[k][c][r][s] * dy[k][j][q]
// (A = the transposed filter bank in registers, 32 steps of two output channels; B = dy fetched straight from memory,
// lanes along q), and a workgroup that walks down a strip of image rows, 126 columns wide, keeps the last three T rows
// (128 columns: one more on either side) in LDS and emits
//     dx[c][ih][iw] = sum over (r,s) of T_(ih-r+1)[(c,r,s)][iw-s+1]
// for the row above the one just computed (nine LDS reads per value; rows outside the image are skipped, columns
// outside it hold zero because nothing was fetched for them). Each of the four wavefronts owns 32 of the 128 columns;
// the next row's values are fetched before the barrier and the emission of the current one. dy is read once, plus two
// rows per strip and two columns per 126.
constexpr int BDS_COLS = 128;          // T columns of a workgroup
constexpr int BDS_EMIT = BDS_COLS - 2; // dx columns of a workgroup
template <int CC, class E>
__global__ void __launch_bounds__(256) conv_bwd_data_smallc3x3_mfma_kernel(const E* __restrict__ dy, const float* __restrict__ w, E* __restrict__ dx,
                                                                            int N, int K, int H, int W, int strip_rows) {
    constexpr int NROW = 9 * CC, ES = ElemBytes<E>::V, KS = 32; // up to 64 output channels
    constexpr int WP = BDS_COLS + 1, TROW = NROW * WP;          // odd row stride: the nine reads of a value fall on different banks
    static_assert(NROW <= 32, "one block of 32 rows");
    __shared__ float T[3 * TROW];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int PQ = H * W;
    const int strips = (H + strip_rows - 1) / strip_rows, cblocks = (W + BDS_EMIT - 1) / BDS_EMIT;
    const int cbk = blockIdx.x % cblocks, sid = (blockIdx.x / cblocks) % strips, n = blockIdx.x / (cblocks * strips);
    const int p0 = sid * strip_rows, p1 = p0 + strip_rows < H ? p0 + strip_rows : H;
    const int e0 = cbk * BDS_EMIT, e1 = e0 + BDS_EMIT < W ? e0 + BDS_EMIT : W; // dx columns of this workgroup
    const __amdgpu_buffer_rsrc_t rs = make_rsrc(dy + (long)n * K * PQ, clamp_range((long)K * PQ * ES));

    float a[KS];
    int koff[KS];
#pragma unroll
    for (int t = 0; t < KS; t++) {
        const int k = 2 * t + lk;
        a[t] = (l32 < NROW && k < K) ? w[(long)k * NROW + l32] : 0.0f;
        koff[t] = k < K ? k * PQ * ES : SENT;
    }
    // this lane's T column: image column e0 - 1 + 32*wave + l32, LDS column 32*wave + l32
    const int tc = 32 * wave + l32, q = e0 - 1 + tc;
    const bool q_in = q >= 0 && q < W;
    float b[KS];
    auto fetch = [&](int j) {
        const int base = (q_in && j >= 0 && j < H) ? (j * W + q) * ES : SENT;
#pragma unroll
        for (int t = 0; t < KS; t++) b[t] = buf_load_e<E>(rs, base + koff[t], 0);
    };

    fetch(p0 - 1);
    for (int j = p0 - 1; j <= p1; j++) {
        if (j >= 0 && j < H) { // (a row outside the image is never read below)
            floatx16 acc;
#pragma unroll
            for (int v = 0; v < 16; v++) acc[v] = 0.0f;
#pragma unroll
            for (int t = 0; t < KS; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc, 0, 0, 0);
            float* Tj = T + (j % 3) * TROW;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = 8 * (v / 4) + 4 * lk + (v % 4);
                if (m < NROW) Tj[m * WP + tc] = acc[v];
            }
        }
        if (j < p1) fetch(j + 1);
        __syncthreads();
        const int ih = j - 1;
        if (ih >= p0 && ih < p1) {
            for (int o = tid; o < CC * (e1 - e0); o += 256) {
                const int c = o / (e1 - e0), ew = o - c * (e1 - e0); // dx column e0 + ew: T columns ew, ew + 1, ew + 2 by s = 2, 1, 0
                float sum = 0.0f;
#pragma unroll
                for (int r = 0; r < 3; r++) {
                    const int jj = ih - r + 1;
                    if (jj < 0 || jj >= H) continue;
                    const float* row = T + (jj % 3) * TROW + (c * 9 + r * 3) * WP + ew + 2;
#pragma unroll
                    for (int s = 0; s < 3; s++) sum += row[s * WP - s];
                }
                store_elem(dx + ((long)n * CC + c) * PQ + (long)ih * W + e0 + ew, sum);
            }
        }
        __syncthreads();
    }
}

} // namespace vdnn
