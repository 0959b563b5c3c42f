// Backward filter of 3x3 / stride 1 / padding 1 layers with float activations whose image rows are whole groups of
// two pixels and whose planes are whole groups of four (W % 2 == 0, W >= 14, H*W % 4 == 0, C % 64 == 0). The float
// counterpart of wgrad3x3_bf16_kernel:
//
//   dW[k][c][r][s] = sum over (n,p,q) of dy[n,k,p,q] * x[n,c,p+r-1,q+s-1]
//
// Through tap (r, s) pixel j of a sample meets element j + (r-1)*W + (s-1) of the input plane. A workgroup owns one
// filter row r, 64 input channels and TM output channels; per 16-pixel slice it fetches dy (TM rows) and one run of x
// (64 rows, shifted by (r-1)*W) with 128-bit loads, four pixels per lane, into reduction-major LDS rows, plus the
// element before and the one after the run. A lane's four values of the centre tap are one 128-bit LDS read; the left
// and right tap take the same registers one place apart, the value that enters at the end comes from the neighbouring
// group (or the two extra elements) and is zero where the tap reads the padding beside the image. Rows of the image
// outside the input are not fetched and stay zero. One fetch of dy and of x serves three taps (the tile-per-tap
// engine fetches both again for every tap), which halves the requests to L2 per multiply.
// When W is not a multiple of four (HALFROW) a group of four pixels can hold the last two of one image row and the
// first two of the next: the halves are in or outside the input separately (masked when the group is stored), and
// the padding is met in the middle of a lane's four values as well.
// Accumulators: WR/32 x 3 blocks of 32x32. Partial sums of a reduction split go to the staging area in the
// tap-major order that reduce_splits_tap sums.
#pragma once
#include "mfma_gemm.h"

#include <type_traits>

namespace vdnn {

constexpr int WG3F_CH = 64; // input channels of a workgroup's tile

struct Wgrad3x3F {
    const float* dy;
    const float* x;
    int N, K, C, H, W;
    float* out;          // filter gradient target [K][C][3][3]
    float* partial;      // staging area: [split][K][9*C], column = tap*C + c
    long partial_stride; // K*9*C
    float alpha;
    int accumulate;
    // optional: the bias gradient's partial sums, [K][bias_splits] (split ks of channel m at m * bias_splits + ks). The
    // workgroups add up the dy values they multiply; those of the centre filter row and the first block of input
    // channels write the sums.
    float* bias_partial;
    int bias_splits;
};

// d.M = K, d.N = 9*C, d.K = N*H*W; d.mtiles tiles of 2*WR output channels, d.ntiles = 3 * C/64 (filter row
// fastest), d.splits reduction splits of d.kchunk pixels (a multiple of 16).
template <int WR, bool HALFROW>
__global__ void __launch_bounds__(NT, 2) wgrad3x3_f32_kernel(const Wgrad3x3F g, const GemmDims d) {
    constexpr int TM = 2 * WR, RB = WR / 32, AL = TM / 64;
    __shared__ __attribute__((aligned(16))) float As[2][TM * RED_STRIDE];
    __shared__ __attribute__((aligned(16))) float Bs[2][WG3F_CH * RED_STRIDE];
    __shared__ float Hs[2][2][WG3F_CH]; // [buffer][before / after the run][channel]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int ntiles_all = d.mtiles * d.ntiles;
    const int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int tile = bid % ntiles_all, ks = bid / ntiles_all;
    const int mt = tile % d.mtiles, nt = tile / d.mtiles;
    const int r = nt % 3, c0 = (nt / 3) * WG3F_CH;
    const int m0 = mt * TM;
    const int k_begin = ks * d.kchunk;
    const int k_end = min(d.K, k_begin + d.kchunk);
    const int H = g.H, W = g.W, PQ = H * W;

    const int n_first = k_begin / PQ;
    const int n_last = k_end > k_begin ? (k_end - 1) / PQ : n_first;
    const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.dy + (long)n_first * g.K * PQ, clamp_range((long)(n_last - n_first + 1) * g.K * PQ * 4));
    const __amdgpu_buffer_rsrc_t rsB = make_rsrc(g.x + (long)n_first * g.C * PQ, clamp_range((long)(n_last - n_first + 1) * g.C * PQ * 4));

    // loader state: this thread's pixel group of the slice (four pixels) and its row of the operands
    const int pg = tid & 3, rl = tid >> 2;
    int mrow[AL];
#pragma unroll
    for (int i = 0; i < AL; i++) { const int m = m0 + rl + 64 * i; mrow[i] = m < g.K ? m * PQ * 4 : SENT; }
    int pqA, offA, pB, qB, posB;
    {
        const int kk = k_begin + 4 * pg;
        const int n = kk / PQ, pq = kk - n * PQ;
        pqA = pq;
        offA = (int)(((long)(n - n_first) * g.K * PQ + pq) * 4);
        pB = pq / W; qB = pq - pB * W;
        posB = (int)(((long)(n - n_first) * g.C * PQ + pq) * 4);
    }
    const int colB = ((c0 + rl) * PQ + (r - 1) * W) * 4; // the channel's plane and the filter row's shift
    // wavefronts 0 and 1 also fetch the element before (after) the slice's run, one channel per lane
    const int side = wave & 1;
    int pH, qH, posH;
    {
        const int kk = k_begin + (side ? 12 : 0); // the group the element is the neighbour of
        const int n = kk / PQ, pq = kk - n * PQ;
        pH = pq / W; qH = pq - pH * W;
        posH = (int)(((long)(n - n_first) * g.C * PQ + pq) * 4);
    }
    const int colH = ((c0 + lane) * PQ + (r - 1) * W) * 4 + (side ? 16 : -4);

    floatx4 ra[AL], rb;
    float rh = 0.0f;
    bool keep_lo = true, keep_hi = true;
    // a group's image row / column / byte offset one slice further: one row wrap when W >= 16, else two; at most one sample
    auto advance = [&](int& p, int& q, int& pos) {
        q += KB; pos += KB * 4;
#pragma unroll
        for (int t = 0; t < (HALFROW ? 2 : 1); t++) {
            const bool wrap = q >= W;
            q -= wrap ? W : 0; p += wrap ? 1 : 0;
        }
        const bool next = p >= H;
        p -= next ? H : 0; pos += next ? (g.C - 1) * PQ * 4 : 0;
    };
    auto fetch = [&]() {
#pragma unroll
        for (int i = 0; i < AL; i++) ra[i] = buf_load4(rsA, mrow[i] + offA, 0);
        pqA += KB;
        const bool wrapA = pqA >= PQ;
        pqA -= wrapA ? PQ : 0;
        offA += wrapA ? (KB + (g.K - 1) * PQ) * 4 : KB * 4;

        {
            const bool lo_ok = (unsigned)(pB + r - 1) < (unsigned)H;                               // the row of the group's first pixel
            const bool hi_ok = (HALFROW && qB == W - 2) ? (unsigned)(pB + r) < (unsigned)H : lo_ok; // its last two may be in the next row
            // only the last two inside (the image's first row through the upper filter row): fetched from there on, so that the
            // load does not begin below the first element of the plane - and of the descriptor, where all of it reads zero
            const bool late = hi_ok & !lo_ok;
            rb = buf_load4(rsB, (lo_ok | hi_ok) ? posB + colB + (late ? 8 : 0) : OOB, 0);
            keep_lo = lo_ok; keep_hi = hi_ok;
        }
        advance(pB, qB, posB);

        if (wave < 2) {
            // not fetched where the tap reads the padding (the element would belong to another image row)
            const int prow = pH + r - 1 + ((HALFROW && side && qH == W - 2) ? 1 : 0);
            const bool used = (unsigned)prow < (unsigned)H && qH != (side ? W - 4 : 0);
            rh = buf_load(rsB, used ? posH + colH : OOB, 0);
            advance(pH, qH, posH);
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < AL; i++) *(floatx4*)(As[buf] + (rl + 64 * i) * RED_STRIDE + 4 * pg) = ra[i];
        floatx4 v = rb; // a group outside the input was not fetched: zero
        if (HALFROW) {
            const bool late = keep_hi & !keep_lo;
            v.x = keep_lo ? rb.x : 0.0f; v.y = keep_lo ? rb.y : 0.0f;
            v.z = keep_hi ? (late ? rb.x : rb.z) : 0.0f; v.w = keep_hi ? (late ? rb.y : rb.w) : 0.0f;
        }
        *(floatx4*)(Bs[buf] + rl * RED_STRIDE + 4 * pg) = v;
        if (wave < 2) Hs[buf][side][lane] = rh;
    };

    floatx16 acc[RB][3];
#pragma unroll
    for (int i = 0; i < RB; i++)
#pragma unroll
        for (int s = 0; s < 3; s++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][s][v] = 0.0f;

    const int wm0 = (wave & 1) * WR, wc0 = (wave >> 1) * 32; // this wavefront's rows of dy and channels
    int qs = k_begin % W;                                      // image column of the slice's first pixel

    // fragments of half hf (pixels 8 hf .. 8 hf + 7) of the slice in buffer `buf` whose first pixel has image column q0:
    // a lane holds pixels 8 hf + 4 lk .. + 3 of its row / channel, and the elements before and after them
    struct Frag { floatx4 a[RB]; floatx4 v; float prev, next; bool mid; };
    auto read = [&](int buf, int hf, int q0, Frag& f) {
        const float* arow = As[buf] + (wm0 + l32) * RED_STRIDE + 8 * hf + 4 * lk;
        const float* brow = Bs[buf] + (wc0 + l32) * RED_STRIDE + 8 * hf + 4 * lk;
#pragma unroll
        for (int i = 0; i < RB; i++) f.a[i] = *(const floatx4*)(arow + i * 32 * RED_STRIDE);
        f.v = *(const floatx4*)brow;
        const float* pp = (hf == 0 && lk == 0) ? &Hs[buf][0][wc0 + l32] : brow - 1;
        const float* np = (hf == 1 && lk == 1) ? &Hs[buf][1][wc0 + l32] : brow + 4;
        const float prev = *pp, next = *np;
        int qg = q0 + 8 * hf + 4 * lk;
        qg -= qg >= W ? W : 0;
        f.prev = qg == 0 ? 0.0f : prev;     // left of the image
        f.next = qg == W - 4 ? 0.0f : next; // right of the image
        f.mid = HALFROW && qg == W - 2;     // pixels 2.. of the four begin an image row
    };
    // A launch that also sums dy runs a copy of the loop of its own (chosen once, before the loop), so that the loop of
    // a launch without stays one basic block. Wavefronts 0 and 1 (input channels 0-31) cover the tile's rows of dy.
    // Every workgroup of such a launch runs that copy, though only those of the centre filter row and the first block of
    // input channels write their sums: the workgroups of one reduction split read the same dy (and the three filter
    // rows of a channel block the same run of x) through L2 at the same time, and one that runs a longer loop falls
    // behind the others until its lines are gone (conv1_2 at batch 128: 8.8 GB fetched per launch against 5.2 with all alike).
    const bool bias_loop = g.bias_partial != nullptr && wave < 2;
    const bool sums_bias = bias_loop && nt == 1;
    float bsum[RB];
#pragma unroll
    for (int i = 0; i < RB; i++) bsum[i] = 0.0f;
    auto multiply = [&](const Frag& f, auto with_bias) {
        if constexpr (decltype(with_bias)::value) {
#pragma unroll
            for (int i = 0; i < RB; i++) bsum[i] += (f.a[i][0] + f.a[i][1]) + (f.a[i][2] + f.a[i][3]);
        }
        // pixel 2 reads left of the image through the left tap, pixel 1 right of it through the right tap, where a row begins inside
        const float up[4] = {f.prev, f.v.x, (HALFROW && f.mid) ? 0.0f : f.v.y, f.v.z};
        const float ce[4] = {f.v.x, f.v.y, f.v.z, f.v.w};
        const float dn[4] = {f.v.y, (HALFROW && f.mid) ? 0.0f : f.v.z, f.v.w, f.next};
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int i = 0; i < RB; i++) {
                acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[i][e], up[e], acc[i][0], 0, 0, 0);
                acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[i][e], ce[e], acc[i][1], 0, 0, 0);
                acc[i][2] = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[i][e], dn[e], acc[i][2], 0, 0, 0);
            }
    };

    // Software pipeline of the tile engine: one barrier per slice, in the middle of it; each half's fragments are read
    // while the half before is multiplied; a slice's fetch has a full slice of multiplies to return.
    const int nslices = (k_end - k_begin + KB - 1) / KB;
    fetch();
    stash(0);
    fetch();
    __syncthreads();
    Frag f0, f1;
    read(0, 0, qs, f0);
    auto run = [&](auto with_bias) {
        for (int s = 0; s < nslices; s++) {
            const int cur = s & 1, nxt = cur ^ 1;
            read(cur, 1, qs, f1);
            multiply(f0, with_bias);
            stash(nxt);
#pragma unroll
            for (int i = 0; i < 12 * RB; i++) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x300, 1, 0); }
            __syncthreads();
            fetch();
            qs += KB;
            qs -= qs >= W ? W : 0;
            if (HALFROW) qs -= qs >= W ? W : 0;
            read(nxt, 0, qs, f0);
            multiply(f1, with_bias);
#pragma unroll
            for (int i = 0; i < 12 * RB; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        }
    };
    if (bias_loop) run(std::true_type{});
    else run(std::false_type{});

    if (sums_bias) {
        // a lane summed pixels 4 lk .. 4 lk + 3 of every group of eight of its row: the two halves of the wavefront together
#pragma unroll
        for (int i = 0; i < RB; i++) {
            const float whole = bsum[i] + __shfl_xor(bsum[i], 32);
            const int m = m0 + wm0 + 32 * i + l32;
            if (lk == 0 && m < g.K) g.bias_partial[(long)m * g.bias_splits + ks] = whole;
        }
    }

    // acc[i][s][v]: output channel m0 + wm0 + 32*i + 8*(v/4) + 4*lk + v%4, input channel c0 + wc0 + l32, tap (r, s)
    const int c = c0 + wc0 + l32;
    const int ncols = 9 * g.C;
    const bool to_partial = d.splits > 1;
#pragma unroll
    for (int i = 0; i < RB; i++)
#pragma unroll
        for (int s = 0; s < 3; s++) {
            const int tap = 3 * r + s;
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int m = m0 + wm0 + 32 * i + 8 * (v / 4) + 4 * lk + (v % 4);
                if (m >= g.K || c >= g.C) continue;
                const float a = acc[i][s][v];
                if (to_partial) g.partial[(long)ks * g.partial_stride + (long)m * ncols + (long)tap * g.C + c] = a;
                else {
                    const long idx = (long)m * ncols + (long)c * 9 + tap;
                    g.out[idx] = g.accumulate ? __fmaf_rn(g.alpha, a, g.out[idx]) : g.alpha * a;
                }
            }
        }
}

} // namespace vdnn
