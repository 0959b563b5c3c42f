// Zero-value compression of offloaded tensors. The reference moves every offloaded tensor whole
// (cudaMemcpyAsync in offloadSrcData / prefetchPreviousSrcData, layer.cu:969-987). A rectified tensor is
// about half zeros, and the link to host memory is sixty times slower than HBM, so here a kernel on the
// copy stream compacts the tensor while it writes it into the pinned host buffer, and a second kernel
// expands it while it reads it back. Both reach the host buffer through the device's mapping of pinned
// memory; no staging copy exists on either side. The code is lossless: every element comes back with
// the bits it had (an element is dropped only when all its bits are zero).
//
// Host format. The tensor is cut into chunks of kZvcChunk elements; chunk i owns the slot that starts at
// byte i * (kZvcMapBytes + kZvcChunk * elem_bytes). A slot holds 64 little-endian 64-bit words, bit l of
// word g set when element 64 g + l of the chunk is kept, followed by the kept elements in order. Only
// the map and the kept elements (rounded up to 16 bytes, zero filled) cross the link; the rest of the
// slot is never touched.
#include "backend_internal.h"

namespace vdnn {

static constexpr int kZvcChunk = 4096;      // elements per slot
static constexpr int kZvcMapBytes = kZvcChunk / 8;
static constexpr int kZvcGroups = kZvcChunk / 64;          // 64-bit words of the map
static constexpr int kZvcGroupsPerWave = kZvcGroups / 4;   // 256 threads = 4 waves
static constexpr int kZvcPad = 8;           // elements of zero fill behind the last kept element

__host__ __device__ inline size_t zvc_slot_bytes(int elem_bytes) { return size_t(kZvcMapBytes) + size_t(kZvcChunk) * elem_bytes; }

// A workgroup is kZvcTeams teams of 256 threads, each team on a slot of its own: the kernels spend their life
// waiting for the link, so what matters is bytes in flight per resident workgroup. A resident workgroup costs
// the convolutions of the other streams a place on its compute unit; few large workgroups cost few places.
static constexpr int kZvcTeams = 4;
static constexpr int kZvcThreads = 256 * kZvcTeams;

// E is the element as raw bits (uint32_t for float, uint16_t for bfloat16).
template <class E>
__global__ __launch_bounds__(kZvcThreads) void zvc_pack_kernel(const E* __restrict__ src, unsigned char* __restrict__ host,
                                                               size_t count, size_t chunks, unsigned long long* __restrict__ wire_bytes) {
    __shared__ unsigned long long words[kZvcTeams][kZvcGroups];
    __shared__ unsigned wave_total[kZvcTeams][4];
    __shared__ __attribute__((aligned(16))) E stage[kZvcTeams][kZvcChunk + kZvcPad];
    const int team = threadIdx.x >> 8, tid = threadIdx.x & 255;
    const int lane = tid & 63, wave = tid >> 6;
    const unsigned long long below = (1ull << lane) - 1ull;
    const size_t stride = size_t(gridDim.x) * kZvcTeams;
    // every team makes the same number of trips, so that the barriers meet; a team past the end idles through them
    for (size_t first_chunk = size_t(blockIdx.x) * kZvcTeams; first_chunk < chunks; first_chunk += stride) {
        const size_t chunk = first_chunk + team;
        const bool live = chunk < chunks;
        const size_t base = chunk * kZvcChunk + size_t(wave) * kZvcGroupsPerWave * 64 + lane;
        E v[kZvcGroupsPerWave];
        unsigned long long m[kZvcGroupsPerWave];
        unsigned kept = 0;
#pragma unroll
        for (int i = 0; i < kZvcGroupsPerWave; ++i) {
            const size_t idx = base + size_t(i) * 64;
            v[i] = live && idx < count ? src[idx] : E(0);
        }
#pragma unroll
        for (int i = 0; i < kZvcGroupsPerWave; ++i) {
            m[i] = __ballot(v[i] != 0);
            kept += __popcll(m[i]);
            if (lane == i) words[team][wave * kZvcGroupsPerWave + i] = m[i];
        }
        if (lane == 0) wave_total[team][wave] = kept;
        __syncthreads();
        unsigned pos = 0, total = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) { const unsigned t = wave_total[team][w]; pos += w < wave ? t : 0u; total += t; }
#pragma unroll
        for (int i = 0; i < kZvcGroupsPerWave; ++i) {
            if (v[i] != 0) stage[team][pos + __popcll(m[i] & below)] = v[i];
            pos += __popcll(m[i]);
        }
        if (tid < kZvcPad) stage[team][total + tid] = E(0);
        __syncthreads();
        if (live) {
            unsigned char* slot = host + chunk * zvc_slot_bytes(sizeof(E));
            typedef unsigned v4u __attribute__((ext_vector_type(4)));
            if (tid < kZvcGroups) __builtin_nontemporal_store(words[team][tid], reinterpret_cast<unsigned long long*>(slot) + tid);
            const unsigned n16 = (total * unsigned(sizeof(E)) + 15u) / 16u;
            v4u* out = reinterpret_cast<v4u*>(slot + kZvcMapBytes);
            const v4u* in = reinterpret_cast<const v4u*>(stage[team]);
            for (unsigned u = tid; u < n16; u += 256) __builtin_nontemporal_store(in[u], out + u);
            if (tid == 0 && wire_bytes) atomicAdd(wire_bytes, (unsigned long long)(kZvcMapBytes + n16 * 16u));
            // a team has one slot on its way at a time: stores that pile up ahead of the link hold up the
            // stores of the kernels on the other streams behind them
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();
    }
}

template <class E>
__global__ __launch_bounds__(kZvcThreads) void zvc_unpack_kernel(const unsigned char* __restrict__ host, E* __restrict__ dst,
                                                                 size_t count, size_t chunks) {
    __shared__ unsigned long long words[kZvcTeams][kZvcGroups];
    __shared__ unsigned first[kZvcTeams][kZvcGroups + 1];   // kept elements ahead of each group, and their number overall
    __shared__ __attribute__((aligned(16))) E stage[kZvcTeams][kZvcChunk + kZvcPad];
    const int team = threadIdx.x >> 8, tid = threadIdx.x & 255;
    const int lane = tid & 63, wave = tid >> 6;
    const unsigned long long below = (1ull << lane) - 1ull;
    const size_t stride = size_t(gridDim.x) * kZvcTeams;
    for (size_t first_chunk = size_t(blockIdx.x) * kZvcTeams; first_chunk < chunks; first_chunk += stride) {
        const size_t chunk = first_chunk + team;
        const bool live = chunk < chunks;
        const unsigned char* slot = host + chunk * zvc_slot_bytes(sizeof(E));
        if (wave == 0) {
            const unsigned long long w = live ? reinterpret_cast<const unsigned long long*>(slot)[lane] : 0ull;
            words[team][lane] = w;
            unsigned sum = __popcll(w);
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const unsigned up = __shfl_up(sum, d, 64);
                sum += lane >= d ? up : 0u;
            }
            first[team][lane + 1] = sum;
            if (lane == 0) first[team][0] = 0;
        }
        __syncthreads();
        const unsigned total = first[team][kZvcGroups];
        const unsigned n16 = (total * unsigned(sizeof(E)) + 15u) / 16u;
        const uint4* in = reinterpret_cast<const uint4*>(slot + kZvcMapBytes);
        uint4* st = reinterpret_cast<uint4*>(stage[team]);
        for (unsigned u = tid; u < n16; u += 256) st[u] = in[u];
        __syncthreads();
        const size_t base = chunk * kZvcChunk + size_t(wave) * kZvcGroupsPerWave * 64 + lane;
#pragma unroll
        for (int i = 0; i < kZvcGroupsPerWave; ++i) {
            const int g = wave * kZvcGroupsPerWave + i;
            const unsigned long long w = words[team][g];
            const E value = (w >> lane) & 1ull ? stage[team][first[team][g] + __popcll(w & below)] : E(0);
            const size_t idx = base + size_t(i) * 64;
            if (live && idx < count) dst[idx] = value;
        }
        __syncthreads();
    }
}

static int zvc_grid(vdnn_ctx* ctx, size_t chunks, bool pack) {
    // enough slots in flight to keep the link busy across their round trips, on an eighth of the compute units
    (void)pack;
    const size_t cap = size_t(ctx->num_cu) / 8;
    const size_t need = (chunks + kZvcTeams - 1) / kZvcTeams;
    return int(need < cap ? need : cap);
}

} // namespace vdnn

using namespace vdnn;

size_t vdnn_zvc_buffer_bytes(size_t count, int elem_bytes) {
    if (elem_bytes != 2 && elem_bytes != 4) return 0;
    const size_t chunks = (count + kZvcChunk - 1) / kZvcChunk;
    return chunks * zvc_slot_bytes(elem_bytes);
}

int vdnn_zvc_offload_async(vdnn_ctx* ctx, void* dst_host, const void* src_dev, size_t count, int elem_bytes, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    VDNN_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "elements are two or four bytes");
    if (ctx->plan_only || count == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_host && src_dev, "null pointer");
    VDNN_REQUIRE(((uintptr_t)dst_host & 15) == 0 && ((uintptr_t)src_dev & (elem_bytes - 1)) == 0, "misaligned buffer");
    if (!ctx->zvc_wire_bytes) {
        VDNN_HIP(hipMalloc((void**)&ctx->zvc_wire_bytes, sizeof(unsigned long long)));
        VDNN_HIP(hipMemset(ctx->zvc_wire_bytes, 0, sizeof(unsigned long long)));
    }
    hipStream_t s = stream ? (hipStream_t)stream : ctx->d2h;
    const size_t chunks = (count + kZvcChunk - 1) / kZvcChunk;
    ProfScope prof(ctx, s, "offload_zvc", 0.0, (double)(count * elem_bytes));
    if (elem_bytes == 4)
        zvc_pack_kernel<uint32_t><<<zvc_grid(ctx, chunks, true), kZvcThreads, 0, s>>>((const uint32_t*)src_dev, (unsigned char*)dst_host, count, chunks, ctx->zvc_wire_bytes);
    else
        zvc_pack_kernel<uint16_t><<<zvc_grid(ctx, chunks, true), kZvcThreads, 0, s>>>((const uint16_t*)src_dev, (unsigned char*)dst_host, count, chunks, ctx->zvc_wire_bytes);
    VDNN_HIP(hipGetLastError());
    ctx->zvc_raw_bytes += (unsigned long long)count * elem_bytes;
    return VDNN_OK;
}

int vdnn_zvc_prefetch_async(vdnn_ctx* ctx, void* dst_dev, const void* src_host, size_t count, int elem_bytes, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    VDNN_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "elements are two or four bytes");
    if (ctx->plan_only || count == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_dev && src_host, "null pointer");
    VDNN_REQUIRE(((uintptr_t)src_host & 15) == 0 && ((uintptr_t)dst_dev & (elem_bytes - 1)) == 0, "misaligned buffer");
    hipStream_t s = stream ? (hipStream_t)stream : ctx->h2d;
    const size_t chunks = (count + kZvcChunk - 1) / kZvcChunk;
    ProfScope prof(ctx, s, "prefetch_zvc", 0.0, (double)(count * elem_bytes));
    if (elem_bytes == 4)
        zvc_unpack_kernel<uint32_t><<<zvc_grid(ctx, chunks, false), kZvcThreads, 0, s>>>((const unsigned char*)src_host, (uint32_t*)dst_dev, count, chunks);
    else
        zvc_unpack_kernel<uint16_t><<<zvc_grid(ctx, chunks, false), kZvcThreads, 0, s>>>((const unsigned char*)src_host, (uint16_t*)dst_dev, count, chunks);
    VDNN_HIP(hipGetLastError());
    return VDNN_OK;
}

int vdnn_zvc_traffic(vdnn_ctx* ctx, unsigned long long* tensor_bytes, unsigned long long* link_bytes) {
    VDNN_REQUIRE(ctx && tensor_bytes && link_bytes, "null argument");
    *tensor_bytes = ctx->zvc_raw_bytes;
    *link_bytes = 0;
    if (ctx->plan_only || !ctx->zvc_wire_bytes) return VDNN_OK;
    VDNN_HIP(hipDeviceSynchronize());
    VDNN_HIP(hipMemcpy(link_bytes, ctx->zvc_wire_bytes, sizeof(unsigned long long), hipMemcpyDeviceToHost));
    return VDNN_OK;
}
