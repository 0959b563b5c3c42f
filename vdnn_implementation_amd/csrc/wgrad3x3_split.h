// Backward filter of 3x3 / stride 1 / padding 1 layers with float activations on the bfloat16 matrix cores: the
// perf-optimal mode's kernel (W % 4 == 0, W >= 16, H*W % 8 == 0, C % 64 == 0).
//
//   dW[k][c][r][s] = sum over (n,p,q) of dy[n,k,p,q] * x[n,c,p+r-1,q+s-1]
//
// The scheme of wgrad3x3_bf16.h - a workgroup owns one filter row r, 64 input channels and TM output channels, the
// pixel reduction runs in slices whose x fragment is read from LDS once for the centre tap and moved one element
// left / right in registers for the other two - with every float operand as two bfloat16 parts, hi = bf16(v) and
// lo = bf16(v - hi), and a product taken as hi*hi + hi*lo + lo*hi accumulated in float (see conv3x3_bf16.h for the
// error: about 2^-16 per product, averaged down by random signs). A slice is 16 pixels; an LDS row holds
// [hi of 16 pixels | lo of 16 pixels], so the address arithmetic of the bfloat16 kernel's half slices serves the two
// parts. The operands are fetched as floats (two 128-bit loads of four pixels per lane and row: a group of four
// pixels never leaves its image row, so each load is inside the input or not fetched at all) and split when they
// are written to LDS, two slices after their fetch. Per slice and wavefront: 6 + 4 LDS reads, 18 matrix
// instructions (3 taps x 2 row blocks x 3 products), one barrier.
// The bias gradient, where asked for, is the sum of the float dy values as fetched: every loading thread adds up its
// row's pixels slice by slice, the two threads of a row are added at the end (a fixed order).
#pragma once
#include "wgrad3x3_bf16.h"
#include "conv3x3_bf16.h"

namespace vdnn {

constexpr int WG3S_SLICE = 16; // pixels of a slice

struct Wgrad3x3S {
    const float* dy;
    const float* x;
    int N, K, C, H, W;
    float* out;          // filter gradient target [K][C][3][3]
    float* partial;      // staging area: [split][K][9*C], column = tap*C + c
    long partial_stride; // K*9*C
    float alpha;
    int accumulate;
    float* bias_partial; // optional: [K][bias_splits], written by the workgroups of the centre filter row and the first channel block
    int bias_splits;
};

typedef float floatx4 __attribute__((ext_vector_type(4)));

// d.M = K, d.N = 9*C, d.K = N*H*W; d.mtiles tiles of 2*WR output channels, d.ntiles = 3 * C/64 (filter row fastest),
// d.splits reduction splits of d.kchunk pixels (a multiple of 16).
// HALFROW: W not a multiple of eight - a group of eight pixels may hold the end of one image row and the start of the next.
template <int WR, bool HALFROW>
__global__ void __launch_bounds__(NT, 2) wgrad3x3_split_kernel(const Wgrad3x3S g, const GemmDims d) {
    constexpr int TM = 2 * WR, RB = WR / 32, SL = WG3S_SLICE;
    __shared__ __attribute__((aligned(16))) unsigned short As[2][TM * HSTRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short Bs[2][WG3_CH * HSTRIDE];
    __shared__ unsigned short Hs[2][2][2][WG3_CH]; // [buffer][before / after the run][hi / lo][channel]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l32 = lane & 31, lk = lane >> 5;
    const int ntiles_all = d.mtiles * d.ntiles;
    const int bid = xcd_remap(blockIdx.x, gridDim.x);
    const int tile = bid % ntiles_all, ks = bid / ntiles_all;
    const int mt = tile % d.mtiles, nt = tile / d.mtiles;
    const int r = nt % 3, c0 = (nt / 3) * WG3_CH;
    const int m0 = mt * TM;
    const int k_begin = ks * d.kchunk;
    const int k_end = min(d.K, k_begin + d.kchunk);
    const int H = g.H, W = g.W, PQ = H * W;

    const int n_first = k_begin / PQ;
    const int n_last = k_end > k_begin ? (k_end - 1) / PQ : n_first;
    const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.dy + (long)n_first * g.K * PQ, clamp_range((long)(n_last - n_first + 1) * g.K * PQ * 4));
    const __amdgpu_buffer_rsrc_t rsB = make_rsrc(g.x + (long)n_first * g.C * PQ, clamp_range((long)(n_last - n_first + 1) * g.C * PQ * 4));

    // loader state: this thread's group of eight pixels of the slice and its row of the operands. TM = 128: rows of dy by
    // all threads, rows of x by wavefronts 0 and 1, the two neighbouring elements by wavefronts 2 and 3. TM = 64: rows
    // of dy by wavefronts 0 and 1, rows of x by wavefronts 2 and 3 (so that every wavefront splits one operand), the
    // neighbouring elements by wavefronts 0 and 1.
    const int pg = tid & 1, rl = rows_by_two_lanes(tid), rlb = rl & 63; // (that order of the rows: no LDS bank conflicts in the stores)
    const bool loads_a = rl < TM, loads_b = TM == 64 ? wave >= 2 : wave < 2;
    const int mrow = (loads_a && m0 + rl < g.K) ? (m0 + rl) * PQ * 4 : SENT;
    int pqA, offA, pB, qB, posB;
    {
        const int kk = k_begin + 8 * pg;
        const int n = kk / PQ, pq = kk - n * PQ;
        pqA = pq;
        offA = (int)(((long)(n - n_first) * g.K * PQ + pq) * 4);
        pB = pq / W; qB = pq - pB * W;
        posB = (int)(((long)(n - n_first) * g.C * PQ + pq) * 4);
    }
    const int colB = ((c0 + rlb) * PQ + (r - 1) * W) * 4; // the channel's plane and the filter row's shift
    // the element before (after) the slice's run, one channel per lane
    const bool loads_h = TM == 64 ? wave < 2 : wave >= 2;
    const int side = wave & 1;
    int pH, qH, posH;
    {
        const int kk = k_begin + (side ? SL - 8 : 0); // the group the element is the neighbour of
        const int n = kk / PQ, pq = kk - n * PQ;
        pH = pq / W; qH = pq - pH * W;
        posH = (int)(((long)(n - n_first) * g.C * PQ + pq) * 4);
    }
    const int colH = ((c0 + lane) * PQ + (r - 1) * W) * 4 + (side ? 32 : -4);

    // what a slice's fetch leaves in registers; two slices are in flight
    struct Fetched { floatx4 ra[2], rb[2]; float rh; };
    Fetched fa, fb;
    fa.rh = 0.0f; fb.rh = 0.0f;
    // a group's image row / column / byte offset one slice further: at most one image row (W >= 16), at most one sample
    auto advance = [&](int& p, int& q, int& pos) {
        q += SL; pos += SL * 4;
        const bool wrap = q >= W;
        q -= wrap ? W : 0; p += wrap ? 1 : 0;
        const bool next = p >= H;
        p -= next ? H : 0; pos += next ? (g.C - 1) * PQ * 4 : 0;
    };
    auto fetch = [&](Fetched& f) {
        if (loads_a) {
            f.ra[0] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsA, mrow + offA, 0, 0));
            f.ra[1] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsA, mrow + offA + 16, 0, 0));
        }
        pqA += SL;
        const bool wrapA = pqA >= PQ;
        pqA -= wrapA ? PQ : 0;
        offA += wrapA ? (SL + (g.K - 1) * PQ) * 4 : SL * 4;
        if (loads_b) {
            const bool lo_ok = (unsigned)(pB + r - 1) < (unsigned)H;                 // the row of the group's first four pixels
            const bool hi_ok = (HALFROW && qB == W - 4) ? (unsigned)(pB + r) < (unsigned)H : lo_ok; // its last four may be in the next row
            f.rb[0] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsB, lo_ok ? posB + colB : OOB, 0, 0));
            f.rb[1] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(rsB, hi_ok ? posB + colB + 16 : OOB, 0, 0));
            advance(pB, qB, posB);
        }
        if (loads_h) {
            // the neighbour of the slice's first (last) group, in the image row of that group's first (last) pixel; not
            // fetched where the tap reads the padding there
            const int prow = pH + r - 1 + ((HALFROW && side && qH == W - 4) ? 1 : 0);
            const bool used = (unsigned)prow < (unsigned)H && qH != (side ? W - 8 : 0);
            f.rh = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsB, used ? posH + colH : OOB, 0, 0));
            advance(pH, qH, posH);
        }
    };
    float bias_sum = 0.0f; // of this thread's pixels of its dy row
    auto split8 = [](const floatx4 (&v)[2], uintx4& hi, uintx4& lo) {
        unsigned h[4], l[4];
        split_pair(v[0].x, v[0].y, h[0], l[0]); split_pair(v[0].z, v[0].w, h[1], l[1]);
        split_pair(v[1].x, v[1].y, h[2], l[2]); split_pair(v[1].z, v[1].w, h[3], l[3]);
        hi.x = h[0]; hi.y = h[1]; hi.z = h[2]; hi.w = h[3];
        lo.x = l[0]; lo.y = l[1]; lo.z = l[2]; lo.w = l[3];
    };
    // `real`: the slice lies inside the range (the fetch runs two slices ahead of the multiplies and past the end)
    auto stash = [&](int buf, const Fetched& f, bool real, auto with_bias) {
        if (loads_a) {
            uintx4 hi, lo;
            split8(f.ra, hi, lo);
            unsigned short* at = As[buf] + rl * HSTRIDE + 8 * pg;
            *(uintx4*)at = hi; *(uintx4*)(at + 16) = lo;
            if constexpr (decltype(with_bias)::value) {
                const float s = ((f.ra[0].x + f.ra[0].y) + (f.ra[0].z + f.ra[0].w)) + ((f.ra[1].x + f.ra[1].y) + (f.ra[1].z + f.ra[1].w));
                bias_sum += real ? s : 0.0f;
            }
        }
        if (loads_b) {
            uintx4 hi, lo;
            split8(f.rb, hi, lo);
            unsigned short* at = Bs[buf] + rlb * HSTRIDE + 8 * pg;
            *(uintx4*)at = hi; *(uintx4*)(at + 16) = lo;
        }
        if (loads_h) {
            unsigned hi, lo;
            split_pair(f.rh, 0.0f, hi, lo);
            Hs[buf][side][0][lane] = (unsigned short)hi; Hs[buf][side][1][lane] = (unsigned short)lo;
        }
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

    // What a wavefront reads from LDS for one part (hi or lo) of a slice: its rows of dy, the centre tap's fragment of x
    // and the element before / after this lane's eight (in the row, unless the lane holds the slice's first / last group).
    struct Frag { bf16x8 a[RB]; uintx4 v; unsigned prev, next; };
    auto read_frag = [&](int buf, int part, Frag& fr) {
        const unsigned short* arow = As[buf] + (wm0 + l32) * HSTRIDE + 8 * lk + 16 * part;
        const unsigned short* brow = Bs[buf] + (wc0 + l32) * HSTRIDE + 8 * lk + 16 * part;
#pragma unroll
        for (int i = 0; i < RB; i++) fr.a[i] = *(const bf16x8*)(arow + i * 32 * HSTRIDE);
        fr.v = *(const uintx4*)brow;
        const unsigned short* pp = lk == 0 ? &Hs[buf][0][part][wc0 + l32] : brow - 1;
        const unsigned short* np = lk == 1 ? &Hs[buf][1][part][wc0 + l32] : brow + 8;
        fr.prev = *pp; fr.next = *np;
    };
    // the fragment moved one pixel up (the left tap), as it is (centre), one pixel down (right); zero enters at the image's edges
    auto taps = [&](const Frag& fr, bf16x8 (&b)[3]) {
        const uintx4 v = fr.v;
        unsigned prev = fr.prev, next = fr.next;
        int qg = qs + 8 * lk;
        qg -= qg >= W ? W : 0;
        prev = qg == 0 ? 0u : prev;     // left of the image
        next = qg == W - 8 ? 0u : next; // right of the image
        const bool mid = HALFROW && qg == W - 4; // pixels 4.. of the eight begin an image row
        const unsigned t1 = __builtin_amdgcn_alignbit(v.y, v.x, 16u), t2 = __builtin_amdgcn_alignbit(v.z, v.y, 16u),
                       t3 = __builtin_amdgcn_alignbit(v.w, v.z, 16u);
        uintx4 up, dn;
        up.x = (v.x << 16) | prev; up.y = t1; up.z = t2; up.w = t3;
        dn.x = t1; dn.y = t2; dn.z = t3; dn.w = (next << 16) | (v.w >> 16);
        if (HALFROW) {
            up.z &= mid ? 0xFFFF0000u : ~0u; // pixel 4 reads left of the image through the left tap
            dn.y &= mid ? 0x0000FFFFu : ~0u; // pixel 3 reads right of the image through the right tap
        }
        b[0] = __builtin_bit_cast(bf16x8, up); b[1] = __builtin_bit_cast(bf16x8, v); b[2] = __builtin_bit_cast(bf16x8, dn);
    };
    auto multiply = [&](const bf16x8 (&a)[RB], const bf16x8 (&b)[3]) {
#pragma unroll
        for (int i = 0; i < RB; i++)
#pragma unroll
            for (int s = 0; s < 3; s++) acc[i][s] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[s], acc[i][s], 0, 0, 0);
    };

    const int nslices = (k_end - k_begin + SL - 1) / SL;
    // Slice s (LDS buffer s % 2): read its lo parts; multiply hi x hi; write slice s + 1 (fetched two slices ago) to the
    // other buffer; barrier; fetch slice s + 3; read the hi parts of slice s + 1 from the buffer just completed; multiply
    // hi x lo and lo x hi. All reads of a buffer precede the barrier after which it is written again; the hi parts
    // of consecutive slices take turns in two sets of registers.
    auto run = [&](auto with_bias) {
        fetch(fa);
        stash(0, fa, nslices > 0, with_bias);
        fetch(fb);
        fetch(fa);
        __syncthreads();
        Frag hi[2], lo;
        read_frag(0, 0, hi[0]);
        auto slice_body = [&](auto parity, int s, Fetched& f) {
            constexpr int cur = decltype(parity)::value;
            bf16x8 bh[3], bl[3];
            read_frag(cur, 1, lo);
            taps(hi[cur], bh);
            multiply(hi[cur].a, bh);
            stash(cur ^ 1, f, s + 1 < nslices, with_bias);
            __syncthreads();
            fetch(f);
            read_frag(cur ^ 1, 0, hi[cur ^ 1]);
            taps(lo, bl);
            multiply(hi[cur].a, bl);
            multiply(lo.a, bh);
            qs += SL;
            qs -= qs >= W ? W : 0;
        };
        for (int s = 0; s < nslices; s += 2) {
            slice_body(std::integral_constant<int, 0>{}, s, fb);
            if (s + 1 < nslices) slice_body(std::integral_constant<int, 1>{}, s + 1, fa);
        }
    };
    // every workgroup of a launch that wants the bias gradient runs the summing loop (workgroups that share dy and x
    // through L2 keep pace that way); those of the centre filter row and the first block of input channels write the sums
    if (g.bias_partial) run(std::true_type{});
    else run(std::false_type{});
    if (g.bias_partial && nt == 1 && loads_a) {
        const float whole = bias_sum + __shfl_xor(bias_sum, 1); // the row's two pixel groups
        const int m = m0 + rl;
        if (pg == 0 && m < g.K) g.bias_partial[(long)m * g.bias_splits + ks] = whole;
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
