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

// x and y below 2 GiB each (offsets are 32-bit), N*H*W below 2^31.
template <int CC, int RBLK, class E>
__global__ void __launch_bounds__(256) conv_fwd_smallc3x3_kernel(const E* __restrict__ x, const float* __restrict__ w, const float* __restrict__ bias,
                                                                  E* __restrict__ y, int N, int K, int H, int W, int relu) {
    constexpr int KRED = 9 * CC, ES = ElemBytes<E>::V;
    // with an odd reduction length the bias rides in the unused last index (input value 1); otherwise it is added afterwards
    constexpr bool BIAS_SLOT = KRED % 2 == 1;
    constexpr int KS = (KRED + 1) / 2;
    const int lane = threadIdx.x & 63, l32 = lane & 31, lk = lane >> 5;
    const int PQ = H * W;
    const int total = N * PQ;
    const int nunits = (total + 31) / 32;
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
    // (sample, row, column) is carried from unit to unit
    const int per = (nunits + nwaves - 1) / nwaves;
    const int first = wave0 * per, last = first + per < nunits ? first + per : nunits;
    int px = first * 32 + l32;
    int n, p, q;
    {
        const int pc = px < total ? px : 0;
        n = pc / PQ;
        const int pq = pc - n * PQ;
        p = pq / W; q = pq - p * W;
    }
    float b[KS];
    int obase = OOB; // byte offset of (n, output channel 4*lk, p, q) in y, or out of range
    auto fetch = [&](bool in_run, float (&dst)[KS], int& out_base) {
        const bool inside = in_run && px < total;
        const int pq = p * W + q;
        const int base = (n * CC * PQ + pq) * ES;
        // the nine places of the window that lie inside the image, as bits r*3 + s
        const unsigned colok = (q > 0 ? 1u : 0u) | 2u | (q < W - 1 ? 4u : 0u);
        const unsigned win = inside ? ((p > 0 ? colok : 0u) | (colok << 3) | (p < H - 1 ? colok << 6 : 0u)) : 0u;
#pragma unroll
        for (int t = 0; t < KS; t++) {
            const unsigned tap = (unsigned)(ktap[t / 16] >> (4 * (t % 16))) & 15u;
            float v = buf_load_e<E>(rs, ((win >> tap) & 1u) ? base + koff[t] : OOB, 0);
            if (BIAS_SLOT && t == KS - 1) v = lk ? 1.0f : v; // reduction index KRED: the bias' factor
            dst[t] = v;
        }
        out_base = inside ? ((n * K + 4 * lk) * PQ + pq) * ES : OOB;
        // one unit further: 32 pixels
        px += 32; q += 32;
        while (q >= W) { q -= W; p += 1; }
        while (p >= H) { p -= H; n += 1; }
    };

    fetch(first < last, b, obase);
    for (int unit = first; unit < last; unit++) {
        float bn[KS];
        int obase_next;
        fetch(unit + 1 < last, bn, obase_next);
        floatx16 acc[RBLK];
#pragma unroll
        for (int i = 0; i < RBLK; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][v] = 0.0f;
#pragma unroll
        for (int t = 0; t < KS; t++)
#pragma unroll
            for (int i = 0; i < RBLK; i++) acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][t], b[t], acc[i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < RBLK; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) {
                const int mrow = 32 * i + 8 * (v / 4) + (v % 4); // + 4*lk, which the lane's offset carries
                float r = acc[i][v];
                if (!BIAS_SLOT && bias) r += bv[i][v];
                if (relu) r = relu_value(r);
                // rows past K (the last block of a layer with fewer channels) are sent out of range
                const int soff = __builtin_amdgcn_readfirstlane(mrow * PQ * ES);
                buf_store_e<E>(ro, r, (mrow + 4 * lk < K) ? obase : OOB, soff);
            }
#pragma unroll
        for (int t = 0; t < KS; t++) b[t] = bn[t];
        obase = obase_next;
    }
}

} // namespace vdnn
