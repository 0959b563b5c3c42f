// Operands of the fully connected layers for the tile engine on the bfloat16 matrix cores (igemm_bf16_kernel).
// With bfloat16 activations the layers' products have two bfloat16 factors - the activation as stored, the
// filter's float master copy rounded to nearest even on its way into LDS - so the bfloat16 instruction forms
// them exactly and only the order of the float summation differs from the float engine. At the batch sizes
// of training (a hundred-odd rows) the float matrix cores bound these layers; on the bfloat16 cores what is
// left is streaming the filter once (forward, backward data) or reading and writing it once (the update).
//
// All loaders put a tile into LDS reduction-major (row stride HSTRIDE), eight consecutive reduction values per
// 128-bit store. The reduction range may end anywhere at a multiple of eight: groups past the end read as zero
// on both sides.
#pragma once
#include "mfma_bf16.h"

namespace vdnn {

__device__ __forceinline__ uintx4 pack8_bf16(const float (&f)[8]) {
    uintx4 q;
    q.x = pack2_bf16(f[0], f[1]);
    q.y = pack2_bf16(f[2], f[3]);
    q.z = pack2_bf16(f[4], f[5]);
    q.w = pack2_bf16(f[6], f[7]);
    return q;
}

// ---- reduction-major operand: element (row, kk) at base[row*ld + kk] -----------------------------------
// thread t: values 8*(t%4) .. +7 of rows t/4 + 64*i. SRC = bf16_t: one 128-bit load per row, stored as it is;
// SRC = float: two 128-bit loads per row, rounded and packed when stored.
template <class SRC>
struct LoadRedAsH {
    static constexpr int ES = ElemBytes<SRC>::V;
    static constexpr int Q = ES / 2;   // 128-bit loads per group of eight values
    const SRC* base;
    long ld;        // elements between rows (rows start at multiples of 16 bytes)
    int rows;
    unsigned bytes; // below 2 GiB
    template <int T> struct Regs { uintx4 v[T / 64][Q]; };
    template <int T> struct State { int vrow[T / 64]; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(base, bytes);
#pragma unroll
        for (int i = 0; i < T / 64; i++) {
            const int row = row0 + (tid >> 2) + 64 * i;
            st.vrow[i] = row < rows ? (int)(((long)row * ld + 8 * (tid & 3)) * ES) : OOB;
        }
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int kend, int tid, Regs<T>& r) const {
        const bool dead = kk0 + 8 * (tid & 3) >= kend;
        const int soff = kk0 * ES;
#pragma unroll
        for (int i = 0; i < T / 64; i++)
#pragma unroll
            for (int q = 0; q < Q; q++)
                r.v[i][q] = __builtin_bit_cast(uintx4, __builtin_amdgcn_raw_buffer_load_b128(st.rsrc, dead ? OOB : st.vrow[i], soff + 16 * q, 0));
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
#pragma unroll
        for (int i = 0; i < T / 64; i++) {
            uintx4 q;
            if constexpr (Q == 1) q = r.v[i][0];
            else {
                const floatx4 lo = __builtin_bit_cast(floatx4, r.v[i][0]), hi = __builtin_bit_cast(floatx4, r.v[i][Q - 1]);
                const float f[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                q = pack8_bf16(f);
            }
            *(uintx4*)(lds + ((tid >> 2) + 64 * i) * HSTRIDE + 8 * (tid & 3)) = q;
        }
    }
};

// ---- row-major operand: element (row, kk) at base[kk*ld_k + row] ---------------------------------------
// Lanes run along the rows (every load of a wavefront is one run of memory), the reduction index is
// wave-uniform and lives in the scalar offset. thread t: row t % T, groups t / T + (256 / T) g of eight
// reduction values: eight loads, one 128-bit LDS store per group.
template <class SRC>
struct LoadRowAsH {
    static constexpr int ES = ElemBytes<SRC>::V;
    const SRC* base;
    long ld_k;      // elements between consecutive kk
    int rows;
    unsigned bytes; // below 2 GiB
    template <int T> struct Regs { float s[T * 4 / NT][8]; };
    template <int T> struct State { int vrow; __amdgpu_buffer_rsrc_t rsrc; };
    template <int T>
    __device__ __forceinline__ void init(State<T>& st, int row0, int tid, int, int) const {
        st.rsrc = make_rsrc(base, bytes);
        const int row = row0 + tid % T;
        st.vrow = row < rows ? row * ES : OOB;
    }
    template <int T>
    __device__ __forceinline__ void load(State<T>& st, int kk0, int kend, int tid, Regs<T>& r) const {
        const int g0 = __builtin_amdgcn_readfirstlane(tid / T);
#pragma unroll
        for (int g = 0; g < T * 4 / NT; g++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const int kk = kk0 + 8 * (g0 + (NT / T) * g) + e;
                const int soff = kk < kend ? (int)((long)kk * ld_k * ES) : 0x7FFFFFF0;
                r.s[g][e] = buf_load_e<SRC>(st.rsrc, st.vrow, soff);
            }
    }
    template <int T>
    __device__ static __forceinline__ void store(unsigned short* lds, int tid, const Regs<T>& r) {
        const int g0 = tid / T;
#pragma unroll
        for (int g = 0; g < T * 4 / NT; g++)
            *(uintx4*)(lds + (tid % T) * HSTRIDE + 8 * (g0 + (NT / T) * g)) = pack8_bf16(r.s[g]);
    }
};

// the transposing loader holds sixteen loads' worth of registers per operand: two workgroups per compute unit
template <class A, class SRC> struct MinResident<A, LoadRowAsH<SRC>> { static constexpr int V = 2; };

} // namespace vdnn
