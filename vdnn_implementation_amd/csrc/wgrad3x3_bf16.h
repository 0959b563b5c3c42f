// Backward filter of 3x3 / stride 1 / padding 1 layers with bfloat16 activations whose image rows are whole
// groups of four pixels and whose planes are whole groups of eight (W % 4 == 0, W >= 16, H*W % 8 == 0, C % 64 == 0).
//
//   dW[k][c][r][s] = sum over (n,p,q) of dy[n,k,p,q] * x[n,c,p+r-1,q+s-1]
//
// The reduction runs over output pixels; dy and x both have it contiguous in memory, and through tap (r, s)
// pixel j of a sample meets element j + (r-1)*W + (s-1) of the input plane: the three taps of a filter row read
// the same run of the plane one element apart. The general engine gives every (tap, 128 channels) a tile of
// its own, which fetches dy and its shifted copy of x again - it is bound by the number of global loads. Here a
// workgroup owns one filter row r, 64 input channels and TM output channels:
//   * per 32-pixel slice it fetches dy (TM rows) and x (64 rows, the run shifted by (r-1)*W) with aligned
//     128-bit loads, eight pixels per lane, straight into reduction-major LDS rows - and two more elements per
//     channel, the one before and the one after the run (rows of the image outside the input are not fetched
//     and stay zero);
//   * a wavefront multiplies its WR x 32 block of dy with 32 channels: the fragment of the centre tap is read
//     from LDS once, the fragments of the left and right tap are that fragment moved by one element in
//     registers (three funnel shifts shared by both, the element that enters comes from the neighbouring group
//     or the two extra elements; it is zero where the tap reads the padding left or right of the image).
// A group of eight pixels never leaves its sample; when W is not a multiple of eight it can hold the last four
// pixels of one image row and the first four of the next: the two halves are then in or outside the input
// separately (masked when the group is stored), and the padding is met in the middle of the fragment as well.
// One LDS fragment and a third of the global loads serve three taps. Accumulators: WR/32 x 3 blocks of 32x32.
// Partial sums of a reduction split go to the staging area in the tap-major order that reduce_splits_tap sums.
#pragma once
#include "mfma_bf16.h"

#include <type_traits>

namespace vdnn {

constexpr int WG3_CH = 64; // input channels of a workgroup's tile

struct Wgrad3x3 {
    const bf16_t* dy;
    const bf16_t* x;
    int N, K, C, H, W;
    float* out;          // filter gradient target [K][C][3][3]
    float* partial;      // staging area: [split][K][9*C], column = tap*C + c
    long partial_stride; // K*9*C
    float alpha;
    int accumulate;
    // optional: the bias gradient's partial sums, [K][bias_splits] (split ks of channel m at m * bias_splits + ks). The
    // workgroups add up the dy values they multiply; those of the centre filter row and the first block of input channels
    // write the sums.
    float* bias_partial;
    int bias_splits;
};

// d.M = K, d.N = 9*C, d.K = N*H*W; d.mtiles tiles of 2*WR output channels, d.ntiles = 3 * C/64 (filter row
// fastest), d.splits reduction splits of d.kchunk pixels (a multiple of 32).
// HALFROW: the general variant - W not a multiple of eight (groups that hold the end of one image row and the start of
// the next) or shorter than a slice (two row wraps per slice); without it W % 8 == 0 and W >= 32.
template <int WR, bool HALFROW>
__global__ void __launch_bounds__(NT, 2) wgrad3x3_bf16_kernel(const Wgrad3x3 g, const GemmDims d) {
    constexpr int TM = 2 * WR, RB = WR / 32, AL = TM / 64;
    __shared__ __attribute__((aligned(16))) unsigned short As[2][TM * HSTRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short Bs[2][WG3_CH * HSTRIDE];
    __shared__ unsigned short Hs[2][2][WG3_CH]; // [buffer][before / after the run][channel]

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
    const __amdgpu_buffer_rsrc_t rsA = make_rsrc(g.dy + (long)n_first * g.K * PQ, clamp_range((long)(n_last - n_first + 1) * g.K * PQ * 2));
    const __amdgpu_buffer_rsrc_t rsB = make_rsrc(g.x + (long)n_first * g.C * PQ, clamp_range((long)(n_last - n_first + 1) * g.C * PQ * 2));

    // loader state: this thread's pixel group of the slice (eight pixels) and its row of the operands
    const int pg = tid & 3, rl = rows_by_four_lanes(tid); // (the order of the rows over the lanes: no LDS bank conflicts in the stores)
    int mrow[AL];
#pragma unroll
    for (int i = 0; i < AL; i++) { const int m = m0 + rl + 64 * i; mrow[i] = m < g.K ? m * PQ * 2 : SENT; }
    int pqA, offA, pB, qB, posB;
    {
        const int kk = k_begin + 8 * pg;
        const int n = kk / PQ, pq = kk - n * PQ;
        pqA = pq;
        offA = (int)(((long)(n - n_first) * g.K * PQ + pq) * 2);
        pB = pq / W; qB = pq - pB * W;
        posB = (int)(((long)(n - n_first) * g.C * PQ + pq) * 2);
    }
    const int colB = ((c0 + rl) * PQ + (r - 1) * W) * 2; // the channel's plane and the filter row's shift
    // wavefronts 0 and 1 also fetch the element before (after) the slice's run, one channel per lane
    const int side = wave & 1;
    int pH, qH, posH;
    {
        const int kk = k_begin + (side ? 24 : 0); // the group the element is the neighbour of
        const int n = kk / PQ, pq = kk - n * PQ;
        pH = pq / W; qH = pq - pH * W;
        posH = (int)(((long)(n - n_first) * g.C * PQ + pq) * 2);
    }
    const int colH = ((c0 + lane) * PQ + (r - 1) * W) * 2 + (side ? 16 : -2);

    // what a slice's fetch leaves in registers; two slices are in flight
    struct Fetched { uintx4 ra[AL], rb; unsigned rh, keep_lo, keep_hi; };
    Fetched fa, fb;
    fa.rh = 0; fb.rh = 0;
    // a group's image row / column / byte offset one slice further: up to two image rows, at most one sample
    auto advance = [&](int& p, int& q, int& pos) {
        q += KH; pos += KH * 2;
#pragma unroll
        for (int t = 0; t < (HALFROW ? 2 : 1); t++) { // W >= 32 when it is a multiple of eight: one wrap
            const bool wrap = q >= W;
            q -= wrap ? W : 0; p += wrap ? 1 : 0;
        }
        const bool next = p >= H;
        p -= next ? H : 0; pos += next ? (g.C - 1) * PQ * 2 : 0;
    };
    auto fetch = [&](Fetched& f) {
#pragma unroll
        for (int i = 0; i < AL; i++) f.ra[i] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(rsA, mrow[i] + offA, 0, 0));
        pqA += KH;
        const bool wrapA = pqA >= PQ;
        pqA -= wrapA ? PQ : 0;
        offA += wrapA ? (KH + (g.K - 1) * PQ) * 2 : KH * 2;

        {
            const bool lo_ok = (unsigned)(pB + r - 1) < (unsigned)H;                 // the row of the group's first pixel
            const bool hi_ok = (HALFROW && qB == W - 4) ? (unsigned)(pB + r) < (unsigned)H : lo_ok; // its last four may be in the next row
            // only the last four inside (the image's first row through the upper filter row): fetched from there on, so that
            // the load does not begin below the first element of the plane - and of the descriptor, where all of it reads zero
            const bool late = hi_ok & !lo_ok;
            f.rb = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(rsB, (lo_ok | hi_ok) ? posB + colB + (late ? 8 : 0) : OOB, 0, 0));
            f.keep_lo = lo_ok ? ~0u : 0u; f.keep_hi = hi_ok ? ~0u : 0u;
        }
        advance(pB, qB, posB);

        if (wave < 2) {
            // the neighbour of the slice's first (last) group, in the image row of that group's first (last) pixel; not
            // fetched where the tap reads the padding there
            const int prow = pH + r - 1 + ((HALFROW && side && qH == W - 4) ? 1 : 0);
            const bool used = (unsigned)prow < (unsigned)H && qH != (side ? W - 8 : 0);
            f.rh = (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rsB, used ? posH + colH : OOB, 0, 0);
            advance(pH, qH, posH);
        }
    };
    auto stash = [&](int buf, const Fetched& f) {
#pragma unroll
        for (int i = 0; i < AL; i++) *(uintx4*)(As[buf] + (rl + 64 * i) * HSTRIDE + 8 * pg) = f.ra[i];
        uintx4 v = f.rb; // a group outside the input was not fetched: zero
        if (HALFROW) {
            const bool late = (f.keep_hi & ~f.keep_lo) != 0u;
            v.x = f.rb.x & f.keep_lo; v.y = f.rb.y & f.keep_lo;
            v.z = (late ? f.rb.x : f.rb.z) & f.keep_hi; v.w = (late ? f.rb.y : f.rb.w) & f.keep_hi;
        }
        *(uintx4*)(Bs[buf] + rl * HSTRIDE + 8 * pg) = v;
        if (wave < 2) Hs[buf][side][lane] = (unsigned short)f.rh;
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

    const int nslices = (k_end - k_begin + KH - 1) / KH;
    // slice s is multiplied from LDS buffer s % 2; `f` holds slice s + 1 (fetched two slices ago): it is written to the
    // other buffer behind the multiplies, and the registers then take the fetch of slice s + 3
    fetch(fa);
    stash(0, fa);
    fetch(fb);
    fetch(fa);
    __syncthreads();
    // A launch that also sums dy runs a copy of the loop of its own, chosen once, so that the loop of a launch without
    // is unchanged: wavefronts 0 and 1 (input channels 0-31, all of the tile's rows of dy) add the eight values of every
    // dy fragment to a running sum of the lane's row, two per v_dot2c_f32_bf16 with a pair of ones. With up to 128 input
    // channels every workgroup of such a launch does, though only those of the centre filter row and the first block of
    // input channels write their sums: the few workgroups of a reduction split read the same dy and x through L2 at the
    // same time, and one with a longer loop falls behind until its lines are gone (the sums as one more MFMA per fragment
    // in those workgroups alone: conv1_2 at batch 128 0.96 ms and 2.7 GB fetched against 0.85 ms and 1.8 GB without the
    // sums; now 0.80 ms and 1.8 GB). With more channels a split has 24 workgroups and more, the straggler's share of the
    // fetches is small, and the sixteen extra instructions per slice in all of them cost more (256 channels: + 5 %).
    const bool bias_loop = g.bias_partial != nullptr && wave < 2 && (g.C <= 128 || nt == 1);
    const bool sums_bias = bias_loop && nt == 1;
    float bsum[RB];
#pragma unroll
    for (int i = 0; i < RB; i++) bsum[i] = 0.0f;
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 ones = __builtin_bit_cast(bf16x2, 0x3F803F80u);
    // What a wavefront reads from LDS for half a slice (16 pixels): its rows of dy, the centre tap's fragment of x and
    // the element before / after this lane's eight (in the row, unless the lane holds the slice's first / last group).
    struct Frag { bf16x8 a[RB]; uintx4 v; unsigned prev, next; };
    auto read_frag = [&](int buf, int h, Frag& fr) {
        const unsigned short* arow = As[buf] + (wm0 + l32) * HSTRIDE + 8 * lk + 16 * h;
        const unsigned short* brow = Bs[buf] + (wc0 + l32) * HSTRIDE + 8 * lk + 16 * h;
#pragma unroll
        for (int i = 0; i < RB; i++) fr.a[i] = *(const bf16x8*)(arow + i * 32 * HSTRIDE);
        fr.v = *(const uintx4*)brow;
        const unsigned short* pp = (h == 0 && lk == 0) ? &Hs[buf][0][wc0 + l32] : brow - 1;
        const unsigned short* np = (h == 1 && lk == 1) ? &Hs[buf][1][wc0 + l32] : brow + 8;
        fr.prev = *pp; fr.next = *np;
    };
    auto multiply = [&](const Frag& fr, int h, auto with_bias) {
        const uintx4 v = fr.v;
        unsigned prev = fr.prev, next = fr.next;
        int qg = qs + 16 * h + 8 * lk;
        qg -= qg >= W ? W : 0;
        if (HALFROW) qg -= qg >= W ? W : 0;
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
        const bf16x8 b0 = __builtin_bit_cast(bf16x8, up), b1 = __builtin_bit_cast(bf16x8, v), b2 = __builtin_bit_cast(bf16x8, dn);
#pragma unroll
        for (int i = 0; i < RB; i++) {
            acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr.a[i], b0, acc[i][0], 0, 0, 0);
            acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr.a[i], b1, acc[i][1], 0, 0, 0);
            acc[i][2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fr.a[i], b2, acc[i][2], 0, 0, 0);
            if constexpr (decltype(with_bias)::value) {
                // (pairs taken with shufflevector: bit casts of the elements of a 4 x 32-bit view all read the first one)
                bsum[i] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(fr.a[i], fr.a[i], 0, 1), ones, bsum[i], false);
                bsum[i] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(fr.a[i], fr.a[i], 2, 3), ones, bsum[i], false);
                bsum[i] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(fr.a[i], fr.a[i], 4, 5), ones, bsum[i], false);
                bsum[i] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(fr.a[i], fr.a[i], 6, 7), ones, bsum[i], false);
            }
        }
    };
    // Slice s (LDS buffer `cur`), as two halves of 16 pixels with the barrier between them; every half's fragments are
    // read while the half before it is multiplied:
    //   read (s, 1); multiply (s, 0); write slice s + 1 to the other buffer; barrier;
    //   fetch slice s + 3; read (s + 1, 0) from the buffer just completed; multiply (s, 1).
    // All reads of a buffer precede the barrier after which it is written again.
    Frag f0, f1;
    read_frag(0, 0, f0);
    auto slice_body = [&](auto parity, Fetched& f, auto with_bias) {
        constexpr int cur = decltype(parity)::value;
        read_frag(cur, 1, f1);
        multiply(f0, 0, with_bias);
        stash(cur ^ 1, f);
        __syncthreads();
        fetch(f);
        read_frag(cur ^ 1, 0, f0);
        multiply(f1, 1, with_bias);
        qs += KH;
        qs -= qs >= W ? W : 0;
        if (HALFROW) qs -= qs >= W ? W : 0;
    };
    auto run = [&](auto with_bias) {
        for (int s = 0; s < nslices; s += 2) {
            slice_body(std::integral_constant<int, 0>{}, fb, with_bias);
            if (s + 1 < nslices) slice_body(std::integral_constant<int, 1>{}, fa, with_bias);
        }
    };
    if (bias_loop) run(std::true_type{});
    else run(std::false_type{});
    if (sums_bias) {
        // a lane summed pixels 8 lk .. 8 lk + 7 of every 16 of its row: the two halves of the wavefront together
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
