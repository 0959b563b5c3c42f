// 3x3, stride 1, padding 1 convolutions of bfloat16 layers - forward and backward data - on the bfloat16
// matrix cores, with the im2col operand formed in LDS from one staged window per filter row.
//
// The general bfloat16 engine (mfma_bf16.h) fetches the im2col tile of every tap from memory: nine times the
// same input elements per channel block, two elements per load instruction, and it is bound by the number of
// those loads. Here the reduction runs in the same blocked tap-major order (32 channels of one tap per slice),
// but the three taps of a filter row share one *window*: for the tile's 256 consecutive output pixels j (an
// even number of them per image row, so pixel pairs never straddle a row) the element "one filter row away",
// x[c][pix(j) + (r-1) W], for 32 channels, plus one element to the left of the first pixel and one to the right
// of the last. Tap s of that row reads the window shifted by s - 1 pixels. A pixel whose tap falls outside the
// image reads zero: a row outside the image is never fetched (the lane's offset is sent out of the descriptor's
// range), a column outside is read from a row of zeros kept behind the window (the window holds the neighbouring
// image row's element there): a lane's fragment address is fixed per tap shift, chosen once per tile, and the
// loop carries no masking arithmetic. So the im2col side costs a third of the loads and LDS stores per tap; the tile is
// 64 x 256, the fragments of each half slice are read from LDS while the half before is multiplied, and the filter
// operand is the packed bank of the general engine (pack_filter_tap_bf16_kernel).
//
// Same results as the general engine up to the order of summation inside the matrix cores (none: both sum a
// slice's 32 products in the instruction and the slices in the same order), same epilogues, same split and
// tail modes (the reduction is cut at multiples of one filter row: 96).
//
// Float layers (E = float), the perf-optimal mode's kernel: every float operand is the sum of two bfloat16 values up to
// 2^-17 of itself - hi = bf16(v), lo = bf16(v - hi), both rounded to nearest - and a product is taken as
// hi*hi + hi*lo + lo*hi on the bfloat16 matrix cores, accumulated in float: three instructions of the 16x faster kind
// for one of the float kind, with a relative error of about 2^-16 per product (the dropped lo*lo term and the two
// remainders), which random signs average down like the rounding of the float instruction's own sums. A slice is then
// 16 channels of one tap, an LDS row holds [hi of 16 channels | lo of 16 channels] where the bfloat16 layers hold 32
// channels, the filter bank comes split the same way (pack_filter_split_kernel) and the "halves" of a slice are its
// hi and lo parts: same pipeline, same LDS traffic and barriers per step, twelve matrix instructions per step
// instead of eight. The window is fetched as 64-bit pixel pairs and split when it is written to LDS, two row
// steps after its fetch. An infinite input gives NaN (inf - inf in lo) where the float kernels give an infinity.
#pragma once
#include <type_traits>
#include "mfma_bf16.h"

namespace vdnn {

constexpr int W3_TM = 64;             // output rows (channels) per tile
constexpr int W3_TN = 256;            // pixels per tile
constexpr int W3_ROWS = W3_TN + 2;    // window positions: one to the left, the tile, one to the right
constexpr int W3_DEPTH = 3 * KH;      // reduction indices of one filter row of one channel block

// MODE 0: forward, src = x, the window of filter row r lies (r - 1) rows below the pixel, tap s reads one column
// further right per s. MODE 1: backward data, src = dy, filter row r lies (1 - r) rows away and tap s reads one
// column further left per s.
template <class E>
struct Win3x3T {
    const E* src;
    int H, W;            // extent of a plane (input and output planes agree)
    long sample_elems;   // reduced channels * H * W
    long total_elems;    // samples * sample_elems
    int nsamples;
};
typedef Win3x3T<bf16_t> Win3x3;

template <int MODE, class E = bf16_t, int RESIDENT = 3>
__global__ void __launch_bounds__(NT, RESIDENT) conv3x3_bf16_kernel(const LoadPackedH al, const Win3x3T<E> geo, const StoreNCHW<E> ep, const GemmDims d) {
    constexpr bool SPLIT = std::is_same<E, float>::value;
    constexpr int EB = (int)sizeof(E);
    constexpr int CH = SPLIT ? 16 : KH;  // channels of a slice
    // 64 rows x 256 pixels per workgroup, a 64 x 64 tile per wavefront: 64 accumulator registers, three workgroups
    // resident per compute unit. (A 128 x 256 tile with 64 x 128 per wavefront - three LDS fragment reads per four
    // MFMAs instead of four, half the window traffic and barriers per MFMA, two workgroups per compute unit - measured
    // the same on the large layers and 20 % slower on 14 x 14 planes.)
    constexpr int TM = W3_TM;
    constexpr int WM = 1;                // wavefronts along the rows
    constexpr int CW = W3_TN / 4;        // columns of a wavefront
    constexpr int NJ = CW / 32;          // 32-column blocks of a wavefront
    __shared__ __attribute__((aligned(16))) unsigned short As[2][TM * HSTRIDE];
    __shared__ __attribute__((aligned(16))) unsigned short Bw[2][(W3_ROWS + 1) * HSTRIDE]; // the window and a row of zeros

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int ntiles_all = d.mtiles * d.ntiles;
    int tile, ks;
    bool whole;
    if ((int)blockIdx.x < d.full_tiles) {
        tile = xcd_remap(blockIdx.x, d.full_tiles); ks = 0; whole = true;
    } else if (d.full_tiles > 0) {
        const int r = blockIdx.x - d.full_tiles, tl = ntiles_all - d.full_tiles;
        tile = d.full_tiles + r % tl; ks = r / tl; whole = false;
    } else {
        const int bid = xcd_remap(blockIdx.x, gridDim.x);
        tile = bid % ntiles_all; ks = bid / ntiles_all; whole = d.splits == 1;
    }
    const int mt = tile % d.mtiles, nt = tile / d.mtiles;
    const int m0 = mt * TM, j0 = nt * W3_TN;
    const int k_begin = whole ? 0 : ks * d.kchunk;
    const int k_end = whole ? d.K : min(d.K, k_begin + d.kchunk);
    const int row_begin = k_begin / W3_DEPTH, row_end = (k_end + W3_DEPTH - 1) / W3_DEPTH; // (channel block, filter row) steps

    const int W = geo.W, plane = geo.H * geo.W;
    const int n_first = j0 / plane;
    int n_last = (j0 + W3_TN - 1) / plane;
    if (n_last > geo.nsamples - 1) n_last = geo.nsamples - 1;
    // the descriptor starts W + 2 elements ahead of the first sample (a four-byte boundary: W is even) so that
    // every offset below is non-negative, and ends with the last sample the tile touches
    const long first = (long)n_first * geo.sample_elems;
    const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(geo.src + first - (W + 2), clamp_range(((long)(n_last - n_first + 1) * geo.sample_elems + (W + 2)) * EB));

    // ---- filter operand: rows tid/4 + 64 i, eight reduction values at 8 (tid%4) ------------------------
    // Two filter tiles are in flight: the one of step g + 2, about to be written to LDS, and the one of step g + 3,
    // fetched a whole step before it is needed (fetched only half a step ahead the wavefront waited for memory before
    // every LDS store: 860 -> 1120 TFLOP/s on 512 -> 512 channels at 28 x 28 with this alone).
    typename LoadPackedH::template State<TM> sa;
    typename LoadPackedH::template Regs<TM> ra[2];
    al.template init<TM>(sa, m0, tid, d.M, k_begin);

    // ---- window: thread = (pixel pair tid % 128, channel groups tid / 128 and tid / 128 + 2 of eight channels) ----
    int voff;                 // byte offset of the pair's first pixel in its sample's first plane, or out of range
    unsigned rowinv;          // bit r: filter row r of this pair's image row lies outside the image
    {
        const int j = j0 + 2 * (tid & 127);
        const bool valid = j < d.N;
        const int jj = valid ? j : j0;
        const int n = jj / plane, pix = jj - n * plane;
        const int p = pix / W;
        voff = valid ? (int)(((long)(n - n_first) * geo.sample_elems + pix) * EB) : OOB;
        rowinv = 0;
#pragma unroll
        for (int r = 0; r < 3; r++) {
            const int ih = MODE == 0 ? p + r - 1 : p + 1 - r;
            if (!((unsigned)ih < (unsigned)geo.H)) rowinv |= 1u << r;
        }
    }
    // the two elements beside the tile, for the slice's channels: lanes of wavefront 0, side = lane / CH, channel = lane % CH.
    // The left one is needed (and inside the image row) when the tile's first pixel is not the first of its row,
    // the right one when the tile's last pixel is not the last of its row.
    int hoff = OOB;
    unsigned hrowinv = 0;
    const bool halo_lane = wave == 0 && lane < 2 * CH;
    if (halo_lane) {
        const int side = lane / CH, ch = lane % CH;
        const int j = side ? j0 + W3_TN - 1 : j0;
        if (j < d.N) {
            const int n = j / plane, pix = j - n * plane;
            const int p = pix / W, q = pix - p * W;
            const bool needed = side ? q < W - 1 : q > 0;
            if (needed) hoff = (int)(((long)(n - n_first) * geo.sample_elems + (long)ch * plane + pix + (side ? 1 : -1)) * EB);
#pragma unroll
            for (int r = 0; r < 3; r++) {
                const int ih = MODE == 0 ? p + r - 1 : p + 1 - r;
                if (!((unsigned)ih < (unsigned)geo.H)) hrowinv |= 1u << r;
            }
        }
    }
    // where this lane's fragment of column block jt lies in a window buffer when the tap reads the window `shift`
    // positions on (16-bit units): window row column + shift - or the row of zeros, when the column is the first of
    // its image row and the tap reads its left neighbour (shift 0), or the last and the tap reads its right one (shift 2)
    const int wm0 = (wave % WM) * 64, wn0 = (wave / WM) * CW;
    const int l32 = lane & 31, lk = lane >> 5;
    int frag[NJ][3];
#pragma unroll
    for (int jt = 0; jt < NJ; jt++) {
        const int j = j0 + wn0 + jt * 32 + l32;
        const int pix = j % plane, q = pix % W;
#pragma unroll
        for (int shift = 0; shift < 3; shift++) {
            const bool outside = (shift == 0 && q == 0) || (shift == 2 && q == W - 1);
            frag[jt][shift] = (outside ? W3_ROWS : wn0 + jt * 32 + l32 + shift) * HSTRIDE + 8 * lk;
        }
    }
    if (tid < HSTRIDE) { Bw[0][W3_ROWS * HSTRIDE + tid] = 0; Bw[1][W3_ROWS * HSTRIDE + tid] = 0; }

    // Two windows are in flight: the one fetched for the row step after the next, and the one for the step after
    // that. [item][pixel of the pair]: eight channels each, ready for LDS; the halo element of this lane (wavefront 0).
    // Float layers: one item, [channel][pixel of the pair] as fetched, split when it is stored.
    struct FetchedH { uintx4 wr[2][2]; unsigned hr; };
    struct FetchedF { floatx2 raw[8]; float hr; };
    typedef typename std::conditional<SPLIT, FetchedF, FetchedH>::type Fetched;
    Fetched fa, fb;
    fa.hr = 0; fb.hr = 0;
    const int g0 = __builtin_amdgcn_readfirstlane(tid >> 7); // channel group of the thread's first item: uniform per wavefront
    const int swapped = (tid >> 2) & 1;                      // this lane stores its second pixel first
    const unsigned sel_first = swapped ? 0x07060302u : 0x05040100u, sel_second = swapped ? 0x05040100u : 0x07060302u;

    auto load_window = [&](int row_step, Fetched& f) {
        const int cb = row_step / 3, r = row_step - cb * 3;
        const int rowoff = MODE == 0 ? (r - 1) * W : (1 - r) * W;
        const int vo = voff | bit_to_all_ones(rowinv, r);
        if constexpr (SPLIT) {
            const int ch = cb * CH + 8 * g0;
            const int soff = (ch * plane + rowoff + W + 2) * 4, step = plane * 4;
#pragma unroll
            for (int e = 0; e < 8; e++) f.raw[e] = __builtin_bit_cast(floatx2, __builtin_amdgcn_raw_buffer_load_b64(rsrc, vo, soff + e * step, 0));
            if (halo_lane) f.hr = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, hoff | bit_to_all_ones(hrowinv, r), (cb * CH * plane + rowoff + W + 2) * 4, 0));
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int ch = cb * KH + 8 * (g0 + 2 * i);
                const int soff = (ch * plane + rowoff + W + 2) * 2, step = plane * 2;
                unsigned c[8];
#pragma unroll
                for (int e = 0; e < 8; e++) c[e] = (unsigned)__builtin_amdgcn_raw_buffer_load_b32(rsrc, vo, soff + e * step, 0);
                // 2 x 8 transpose of 16-bit values: the low halves are the first pixel's channels, the high halves the second's.
                // wr[i][0] is the pixel this lane stores first: its first pixel in lanes 0-3 of every eight, its second in
                // lanes 4-7 (store_window)
                f.wr[i][0].x = __builtin_amdgcn_perm(c[1], c[0], sel_first); f.wr[i][0].y = __builtin_amdgcn_perm(c[3], c[2], sel_first);
                f.wr[i][0].z = __builtin_amdgcn_perm(c[5], c[4], sel_first); f.wr[i][0].w = __builtin_amdgcn_perm(c[7], c[6], sel_first);
                f.wr[i][1].x = __builtin_amdgcn_perm(c[1], c[0], sel_second); f.wr[i][1].y = __builtin_amdgcn_perm(c[3], c[2], sel_second);
                f.wr[i][1].z = __builtin_amdgcn_perm(c[5], c[4], sel_second); f.wr[i][1].w = __builtin_amdgcn_perm(c[7], c[6], sel_second);
            }
            if (wave == 0) {
                const int soff = (cb * KH * plane + rowoff + W + 2) * 2;
                f.hr = (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(rsrc, hoff | bit_to_all_ones(hrowinv, r), soff, 0);
            }
        }
    };
    // A lane's two pixels are neighbouring LDS rows, lane after lane two rows on (160 bytes = 40 words): the eight lanes
    // that LDS takes together (rows_by_four_lanes in mfma_bf16.h) would meet on banks 0, 8, 16, 24 twice each. Lanes 4-7 of
    // every eight therefore store their second pixel first: odd rows, 20 words on, the other four groups of banks
    // (a 128-bit store of a wavefront: 8 cycles instead of 16, measured on the pattern alone).
    auto store_window = [&](unsigned short* lds, const Fetched& f) {
        if constexpr (SPLIT) {
#pragma unroll
            for (int e = 0; e < 2; e++) {
                // the pixel stored by instruction e: the lane's pixel e ^ swapped
                uintx4 hi, lo;
                unsigned h[4], l[4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const float a = (e ^ swapped) ? f.raw[2 * k].y : f.raw[2 * k].x, b = (e ^ swapped) ? f.raw[2 * k + 1].y : f.raw[2 * k + 1].x;
                    split_pair(a, b, h[k], l[k]);
                }
                hi.x = h[0]; hi.y = h[1]; hi.z = h[2]; hi.w = h[3];
                lo.x = l[0]; lo.y = l[1]; lo.z = l[2]; lo.w = l[3];
                unsigned short* at = lds + (1 + 2 * (tid & 127) + (e ^ swapped)) * HSTRIDE + 8 * (tid >> 7);
                *(uintx4*)at = hi;
                *(uintx4*)(at + 16) = lo;
            }
            if (halo_lane) {
                unsigned h, l;
                split_pair(f.hr, 0.0f, h, l);
                unsigned short* at = lds + ((lane / CH) ? W3_ROWS - 1 : 0) * HSTRIDE + (lane % CH);
                at[0] = (unsigned short)h; at[16] = (unsigned short)l;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int e = 0; e < 2; e++)
                    *(uintx4*)(lds + (1 + 2 * (tid & 127) + (e ^ swapped)) * HSTRIDE + 8 * ((tid >> 7) + 2 * i)) = f.wr[i][e];
            if (wave == 0) lds[((lane >> 5) ? W3_ROWS - 1 : 0) * HSTRIDE + (lane & 31)] = (unsigned short)f.hr;
        }
    };

    floatx16 acc[NJ / 2][2][2]; // [64-column half][row block][column block]
#pragma unroll
    for (int q = 0; q < NJ / 2; q++)
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int v = 0; v < 16; v++) acc[q][i][j][v] = 0.0f;

    // Pipeline. Step g = (row step, tap s) multiplies from As[g % 2] and the window buffer row_step % 2, as two halves
    // of the slice's 32 reduction values (h = 0, 1), with one barrier between them:
    //   first half:   read the fragments of (g, h = 1), multiply (g, h = 0) (fragments already in registers), write the
    //                 registers holding the filter tile of step g + 1 to the other As buffer and, at s = 2, the window
    //                 of the next row step to the other window buffer;
    //   barrier;
    //   second half:  issue the filter fetch of step g + 3 into the registers just written out (at s = 2 also the
    //                 window fetch of the row step three ahead), read the
    //                 fragments of (g + 1, h = 0) from the buffers just completed, multiply (g, h = 1).
    // Every fragment is thus read while the half before it is multiplied; all reads of a buffer precede the barrier
    // after which it is overwritten. Fetches past the end of the range are never used.
    auto read_a = [&](const unsigned short* buf, int h, bf16x8 (&a)[2]) {
        const unsigned short* ap = buf + (wm0 + l32) * HSTRIDE + 8 * lk + 16 * h;
#pragma unroll
        for (int i = 0; i < 2; i++) a[i] = *(const bf16x8*)(ap + i * 32 * HSTRIDE);
    };
    // tap s reads the window position column + (s - 1) (forward) or column + (1 - s) (backward data): LDS row + 1;
    // the tap that reads the left neighbour is s = 0 in forward, s = 2 in backward data
    auto read_b = [&](const unsigned short* win, int s, int h, uintx4 (&b)[NJ]) {
        const int shift = MODE == 0 ? s : 2 - s;
#pragma unroll
        for (int jt = 0; jt < NJ; jt++) b[jt] = *(const uintx4*)(win + frag[jt][shift] + 16 * h);
    };
    auto multiply = [&](const bf16x8 (&a)[2], const uintx4 (&b)[NJ]) {
#pragma unroll
        for (int jt = 0; jt < NJ; jt++)
#pragma unroll
            for (int i = 0; i < 2; i++)
                acc[jt / 2][i][jt % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], __builtin_bit_cast(bf16x8, b[jt]), acc[jt / 2][i][jt % 2], 0, 0, 0);
    };

    al.template load<TM>(sa, row_begin * W3_DEPTH, k_end, tid, ra[0]);
    load_window(row_begin, fa);
    LoadPackedH::template store<TM>(As[0], tid, ra[0]);
    store_window(Bw[0], fa);
    al.template load<TM>(sa, row_begin * W3_DEPTH + KH, k_end, tid, ra[1]);
    al.template load<TM>(sa, row_begin * W3_DEPTH + 2 * KH, k_end, tid, ra[0]);
    load_window(row_begin + 1, fb);
    load_window(row_begin + 2, fa);
    __syncthreads();
    // Float layers multiply hi x hi in the first half of a step and hi x lo + lo x hi in the second, while the next step's
    // hi fragments arrive: those take turns in two sets of registers.
    // (Measured within 1 % of this, same box and run: the lo fragments read a step ahead as well, so that the first half
    // only writes to LDS; three windows in flight; three workgroups per compute unit at 18 spilled registers. A barrier
    // per row step instead of per tap - the three filter tiles of a row step in buffers of their own, 72 KB of LDS -
    // gained 3 % on the 28 x 28 layers and nothing elsewhere.)
    bf16x8 a0[SPLIT ? 2 : 1][2], a1[2];
    uintx4 b0[SPLIT ? 2 : 1][NJ], b1[NJ];
    read_a(As[0], 0, a0[0]);
    read_b(Bw[0], 0, 0, b0[0]);
    // one row step; `f` holds the window of the next row step (fetched two row steps ago): it is written to LDS in the
    // first half of the last tap, and the registers then take the fetch of the window three row steps ahead. `odd`: the
    // parity of the row step counted from row_begin, which fixes the parity of g (the filter registers of a step)
    auto row_step_body = [&](int row_step, Fetched& f, auto odd) {
        constexpr int ODD = decltype(odd)::value;
        const int wb = ODD;
#pragma unroll
        for (int s = 0; s < 3; s++) {
            const int g = (row_step - row_begin) * 3 + s;
            const int cur = (3 * ODD + s) & 1, nxt = cur ^ 1; // = g & 1
            const int rc = SPLIT ? cur : 0, rn = SPLIT ? nxt : 0;
            read_a(As[cur], 1, a1);
            read_b(Bw[wb], s, 1, b1);
            multiply(a0[rc], b0[rc]);
            LoadPackedH::template store<TM>(As[nxt], tid, ra[(3 * ODD + s + 1) & 1]);
            if (s == 2) store_window(Bw[wb ^ 1], f);
            // issue order of the first half: an LDS access behind every MFMA
#pragma unroll
            for (int i = 0; i < 2 * NJ; i++) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x300, 2, 0); }
            __syncthreads();
            al.template load<TM>(sa, row_begin * W3_DEPTH + (g + 3) * KH, k_end, tid, ra[(3 * ODD + s + 1) & 1]);
            if (s == 2) load_window(row_step + 3, f);
            read_a(As[nxt], 0, a0[rn]);
            read_b(s == 2 ? Bw[wb ^ 1] : Bw[wb], s == 2 ? 0 : s + 1, 0, b0[rn]);
            if constexpr (SPLIT) { multiply(a0[rc], b1); multiply(a1, b0[rc]); }
            else multiply(a1, b1);
            // second half: a memory instruction and an LDS read behind every MFMA
#pragma unroll
            for (int i = 0; i < (SPLIT ? 4 : 2) * NJ; i++) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
        }
    };
    for (int row_step = row_begin; row_step < row_end; row_step += 2) {
        row_step_body(row_step, fb, std::integral_constant<int, 0>{});
        if (row_step + 1 < row_end) row_step_body(row_step + 1, fa, std::integral_constant<int, 1>{});
    }

    // A whole tile's result leaves through LDS: each wavefront lays its 64 x 64 block out row by row (bias and rectifier
    // applied, rounded to bfloat16) and writes it eight pixels - 16 bytes - per lane, gated by eight elements of the gate
    // tensor fetched the same way; lane by lane the block would leave in two-byte stores of 64-byte runs. Same values.
    // Needs planes of whole groups of eight pixels (a group stays in its sample) and 16-byte aligned tensors.
    if constexpr (!SPLIT) {
        if (whole && ep.opix % 8 == 0 && (((uintptr_t)ep.out | (uintptr_t)ep.gate) & 15) == 0) {
            static_assert(NJ == 2 && WM == 1, "one 64 x 64 block per wavefront");
            constexpr int STG = 72; // row stride of the block in LDS, 16-bit units
            static_assert(4 * 64 * STG <= 2 * W3_ROWS * HSTRIDE, "the four blocks fit the window buffers");
            // the gate's elements first (what the lane will overwrite, if the gradient goes over the layer's own input):
            // fetched one after the other behind each store they would cost a round trip to memory each
            const int grp = lane & 7;
            const int j = j0 + wn0 + 8 * grp;
            const int n = j / ep.opix, pix = j - n * ep.opix;
            const size_t base = (size_t)n * d.M * ep.opix + pix;
            uintx4 gv[8];
            if (ep.gate && j < d.N) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const int m = m0 + (lane >> 3) + 8 * i;
                    gv[i] = m < d.M ? *(const uintx4*)(ep.gate + base + (size_t)m * ep.opix) : uintx4{0, 0, 0, 0};
                }
            }
            __syncthreads(); // every wavefront has read its last fragments
            unsigned short* stg = &Bw[0][0] + wave * (64 * STG);
#pragma unroll
            for (int it = 0; it < 2; it++)
#pragma unroll
                for (int v = 0; v < 16; v++) {
                    const int row = it * 32 + 8 * (v / 4) + 4 * lk + (v % 4);
                    const int m = m0 + row;
                    const float b = (ep.bias && m < d.M) ? ep.bias[m] : 0.0f;
#pragma unroll
                    for (int jt = 0; jt < 2; jt++) {
                        float r = acc[0][it][jt][v];
                        if (ep.bias) r += b;
                        if (ep.relu) r = relu_value(r);
                        stg[row * STG + jt * 32 + l32] = float_to_bf16_bits(r);
                    }
                }
            __builtin_amdgcn_wave_barrier(); // the block is read by other lanes of the same wavefront: LDS keeps a wavefront's order
            if (j < d.N) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const int row = (lane >> 3) + 8 * i;
                    const int m = m0 + row;
                    if (m >= d.M) continue;
                    uintx4 val = *(const uintx4*)(stg + row * STG + 8 * grp);
                    const size_t idx = base + (size_t)m * ep.opix;
                    if (ep.gate) {
                        // kept where gate > 0: a positive bfloat16 that is not a NaN has bits 0x0001 .. 0x7F80
                        auto keep = [](unsigned w) {
                            return ((((w & 0xFFFFu) - 1u) < 0x7F80u) ? 0x0000FFFFu : 0u) | ((((w >> 16) - 1u) < 0x7F80u) ? 0xFFFF0000u : 0u);
                        };
                        val.x &= keep(gv[i].x); val.y &= keep(gv[i].y); val.z &= keep(gv[i].z); val.w &= keep(gv[i].w);
                    }
                    *(uintx4*)(ep.out + idx) = val;
                }
            }
            return;
        }
    }
#pragma unroll
    for (int q = 0; q < NJ / 2; q++) {
        if (StoreNCHW<E>::TAIL && d.full_tiles > 0 && !whole)
            ep.store_tail(acc[q], wm0, wn0 + 64 * q, lane, (long)(tile - d.full_tiles) * d.splits + ks, TM, W3_TN);
        else
            ep.store(acc[q], m0 + wm0, j0 + wn0 + 64 * q, lane, ks, d, !whole);
    }
}

} // namespace vdnn
