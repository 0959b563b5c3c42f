// Zero-value compression of offloaded tensors. The reference moves every offloaded tensor whole
// (cudaMemcpyAsync in offloadSrcData / prefetchPreviousSrcData, layer.cu:969-987). A rectified tensor is
// about half zeros, and the link to host memory is more than a hundred times slower than HBM, so here the
// tensor crosses the link without its zero elements. The code is lossless: every element comes back with
// the bits it had (an element is dropped only when all its bits are zero).
//
// Packed stream. The tensor is cut into chunks of kZvcChunk elements. The stream starts with a table of one
// 32-bit word per chunk (padded to 16 bytes): the offset of the chunk's record in units of 16 bytes. A record
// is a map of 64 little-endian 64-bit words followed by the kept elements in the order of the map's bits, zero
// filled to a multiple of 16 bytes. The map follows the way a wave reads memory: a lane holds V = 16 / (bytes per
// element) consecutive elements, one 128-bit load, so 64 lanes cover a block of 64 V elements and the block's map
// is V words - bit l of word j of block b (word b V + j of the chunk) is set when element 64 V b + V l + j of the
// chunk is kept. Records follow the table
// without gaps, in the order in which the packing teams claimed their place (an atomic cursor), so the
// stream is as long as its content and its length is known on the device only.
//
// Offload. The packing kernel reads the tensor at HBM speed. Bytes of the stream below `staging_bytes` go to
// a staging buffer in device memory, which the copy engine then moves to the pinned host buffer like any
// other offload; bytes beyond it are stored by the kernel straight into the host buffer through the device's
// mapping of pinned memory. The caller sizes the staging buffer from the length the same tensor had the step
// before (the kernel reports it in a host word); any size is correct. Stores from a kernel to host memory
// hold up the stores of the kernels on the other streams (a convolution forward ran at 0.6 of its rate
// beside a kernel that wrote the whole stream that way), loads from host memory do not: so the way out
// goes through the copy engine, and the way back is a kernel that reads the host buffer and expands as it goes.
#include "backend_internal.h"

namespace vdnn {

static constexpr int kZvcChunk = 4096;      // elements per record
static constexpr int kZvcMapBytes = kZvcChunk / 8;
static constexpr int kZvcGroups = kZvcChunk / 64;          // 64-bit words of the map
static constexpr int kZvcGroupsPerWave = kZvcGroups / 4;   // a team is 256 threads = 4 waves
static constexpr int kZvcPad = 8;           // elements of zero fill behind the last kept element
// A workgroup is kZvcTeams teams of 256 threads, each team on a chunk of its own. The expanding kernel spends
// its life waiting for the link, so what matters there is bytes in flight per resident workgroup; a resident
// workgroup costs the convolutions of the other streams a place on its compute unit, and few large
// workgroups cost few places.
static constexpr int kZvcTeams = 4;
static constexpr int kZvcThreads = 256 * kZvcTeams;
static constexpr int kZvcCursors = 64;      // offloads that may be in flight at once

__host__ __device__ inline size_t zvc_table_bytes(size_t chunks) { return (chunks * 4 + 15) / 16 * 16; }
__host__ __device__ inline size_t zvc_record_bytes_max(int elem_bytes) { return size_t(kZvcMapBytes) + size_t(kZvcChunk) * elem_bytes; }

typedef unsigned v4u __attribute__((ext_vector_type(4)));

// One record as it lies in the stream: the map, then the kept elements.
template <class E>
struct alignas(16) ZvcRecord {
    unsigned long long words[kZvcGroups];
    E kept[kZvcChunk + kZvcPad];
};

__global__ void zvc_begin_kernel(unsigned long long* cursor, unsigned long long table_bytes) { *cursor = table_bytes; }

// total: length of the stream. link: bytes that cross the link for it (the copy engine moves `staging_bytes`
// whatever the stream's length; with staging_bytes = ~0 the block stays on the device and only what did not fit
// crossed the link - the caller passes the block's size in `kept_bytes` then).
__global__ void zvc_end_kernel(const unsigned long long* cursor, unsigned long long staging_bytes, unsigned long long kept_bytes,
                               unsigned long long* total_host, unsigned long long* link_bytes) {
    const unsigned long long total = *cursor;
    if (total_host) *total_host = total;
    if (staging_bytes == ~0ull) atomicAdd(link_bytes, total > kept_bytes ? total - kept_bytes : 0ull);
    else atomicAdd(link_bytes, total > staging_bytes ? total : staging_bytes);
}

// E is the element as raw bits (uint32_t for float, uint16_t for bfloat16).
template <class E>
__global__ __launch_bounds__(kZvcThreads) void zvc_pack_kernel(const E* __restrict__ src, size_t count, size_t chunks,
                                                               unsigned char* __restrict__ staging, size_t staging_bytes,
                                                               unsigned char* __restrict__ host, unsigned long long* __restrict__ cursor) {
    __shared__ ZvcRecord<E> rec[kZvcTeams];
    __shared__ unsigned wave_total[kZvcTeams][4];
    __shared__ unsigned long long place[kZvcTeams];
    const int team = threadIdx.x >> 8, tid = threadIdx.x & 255;
    const int lane = tid & 63, wave = tid >> 6;
    const unsigned long long below = (1ull << lane) - 1ull;
    const size_t stride = size_t(gridDim.x) * kZvcTeams;
    const bool aligned = (reinterpret_cast<uintptr_t>(src) & 15) == 0;   // (chunks start at multiples of 16 bytes)
    // every team makes the same number of trips, so that the barriers meet; a team past the end idles through them
    for (size_t first_chunk = size_t(blockIdx.x) * kZvcTeams; first_chunk < chunks; first_chunk += stride) {
        const size_t chunk = first_chunk + team;
        const bool live = chunk < chunks;
        // this wave's 16 words are kZvcGroupsPerWave / V blocks; v[b V + j] is this lane's element j of block b
        constexpr int V = 16 / int(sizeof(E));
        const size_t base = chunk * kZvcChunk + size_t(wave) * kZvcGroupsPerWave * 64 + size_t(lane) * V;
        E v[kZvcGroupsPerWave];
        unsigned long long m[kZvcGroupsPerWave];
        unsigned kept = 0;
#pragma unroll
        for (int b = 0; b < kZvcGroupsPerWave / V; ++b) {
            const size_t idx = base + size_t(b) * 64 * V;
            if (live && aligned && idx + V <= count) {
                const v4u q = *reinterpret_cast<const v4u*>(src + idx);
                const E* e = reinterpret_cast<const E*>(&q);
#pragma unroll
                for (int j = 0; j < V; ++j) v[b * V + j] = e[j];
            } else {
#pragma unroll
                for (int j = 0; j < V; ++j) v[b * V + j] = live && idx + j < count ? src[idx + j] : E(0);
            }
        }
#pragma unroll
        for (int i = 0; i < kZvcGroupsPerWave; ++i) {
            m[i] = __ballot(v[i] != 0);
            kept += __popcll(m[i]);
            if (lane == i) rec[team].words[wave * kZvcGroupsPerWave + i] = m[i];
        }
        if (lane == 0) wave_total[team][wave] = kept;
        __syncthreads();
        unsigned pos = 0, total = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) { const unsigned t = wave_total[team][w]; pos += w < wave ? t : 0u; total += t; }
        const unsigned units = kZvcMapBytes / 16 + (total * unsigned(sizeof(E)) + 15u) / 16u;   // 16-byte units of the record
        if (threadIdx.x == 0) {
            // one claim for the workgroup's records: every claim is an atomic on the same word, and the device does
            // about one of those in 3.5 ns (a quarter of this kernel's time on a float tensor, half on a bfloat16 one)
            unsigned bytes[kZvcTeams], all = 0;
#pragma unroll
            for (int t = 0; t < kZvcTeams; ++t) {
                unsigned n = 0;
#pragma unroll
                for (int w = 0; w < 4; ++w) n += wave_total[t][w];
                bytes[t] = first_chunk + t < chunks ? kZvcMapBytes + (n * unsigned(sizeof(E)) + 15u) / 16u * 16u : 0u;
                all += bytes[t];
            }
            unsigned long long at = atomicAdd(cursor, (unsigned long long)all);
#pragma unroll
            for (int t = 0; t < kZvcTeams; ++t) { place[t] = at; at += bytes[t]; }
        }
#pragma unroll
        for (int i = 0; i < kZvcGroupsPerWave; ++i) {
            if (v[i] != 0) rec[team].kept[pos + __popcll(m[i] & below)] = v[i];
            pos += __popcll(m[i]);
        }
        if (tid < kZvcPad) rec[team].kept[total + tid] = E(0);
        __syncthreads();
        if (live) {
            const size_t at = place[team];
            if (tid == 0) {
                const size_t entry = chunk * 4;
                *reinterpret_cast<unsigned*>((entry < staging_bytes ? staging : host) + entry) = unsigned(at / 16);
            }
            const v4u* in = reinterpret_cast<const v4u*>(&rec[team]);
            for (unsigned u = tid; u < units; u += 256) {
                const size_t o = at + size_t(u) * 16;
                *reinterpret_cast<v4u*>((o < staging_bytes ? staging : host) + o) = in[u];
            }
            // a team has one record on its way to host memory at a time: stores that pile up ahead of the link
            // hold up the stores of the kernels on the other streams behind them
            if (at + size_t(units) * 16 > staging_bytes) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();
    }
}

// The stream's bytes below `device_bytes` are read from `device` (a staging block that was kept), the rest from `host`.
template <class E>
__global__ __launch_bounds__(kZvcThreads) void zvc_unpack_kernel(const unsigned char* __restrict__ device, size_t device_bytes,
                                                                 const unsigned char* __restrict__ host, E* __restrict__ dst,
                                                                 size_t count, size_t chunks) {
    __shared__ unsigned long long words[kZvcTeams][kZvcGroups];
    __shared__ unsigned first[kZvcTeams][kZvcGroups + 1];   // kept elements ahead of each group, and their number overall
    __shared__ unsigned long long place[kZvcTeams];
    __shared__ __attribute__((aligned(16))) E kept[kZvcTeams][kZvcChunk + kZvcPad];
    const int team = threadIdx.x >> 8, tid = threadIdx.x & 255;
    const int lane = tid & 63, wave = tid >> 6;
    const unsigned long long below = (1ull << lane) - 1ull;
    const size_t stride = size_t(gridDim.x) * kZvcTeams;
    const bool aligned = (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
    for (size_t first_chunk = size_t(blockIdx.x) * kZvcTeams; first_chunk < chunks; first_chunk += stride) {
        const size_t chunk = first_chunk + team;
        const bool live = chunk < chunks;
        if (wave == 0) {
            const size_t entry = chunk * 4;
            const size_t at = live ? size_t(*reinterpret_cast<const unsigned*>((entry < device_bytes ? device : host) + entry)) * 16 : 0;
            const size_t mine = at + size_t(lane) * 8;
            const unsigned long long w = live ? *reinterpret_cast<const unsigned long long*>((mine < device_bytes ? device : host) + mine) : 0ull;
            words[team][lane] = w;
            unsigned sum = __popcll(w);
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const unsigned up = __shfl_up(sum, d, 64);
                sum += lane >= d ? up : 0u;
            }
            first[team][lane + 1] = sum;
            if (lane == 0) { first[team][0] = 0; place[team] = at; }
        }
        __syncthreads();
        const unsigned total = first[team][kZvcGroups];
        const unsigned n16 = (total * unsigned(sizeof(E)) + 15u) / 16u;
        const size_t values = place[team] + kZvcMapBytes;
        v4u* st = reinterpret_cast<v4u*>(kept[team]);
        for (unsigned u = tid; u < n16; u += 256) {
            const size_t o = values + size_t(u) * 16;
            st[u] = *reinterpret_cast<const v4u*>((o < device_bytes ? device : host) + o);
        }
        __syncthreads();
        constexpr int V = 16 / int(sizeof(E));
        const size_t base = chunk * kZvcChunk + size_t(wave) * kZvcGroupsPerWave * 64 + size_t(lane) * V;
#pragma unroll
        for (int b = 0; b < kZvcGroupsPerWave / V; ++b) {
            v4u q;
            E* e = reinterpret_cast<E*>(&q);
#pragma unroll
            for (int j = 0; j < V; ++j) {
                const int g = wave * kZvcGroupsPerWave + b * V + j;
                const unsigned long long w = words[team][g];
                e[j] = (w >> lane) & 1ull ? kept[team][first[team][g] + __popcll(w & below)] : E(0);
            }
            const size_t idx = base + size_t(b) * 64 * V;
            if (live && aligned && idx + V <= count) {
                *reinterpret_cast<v4u*>(dst + idx) = q;
            } else {
#pragma unroll
                for (int j = 0; j < V; ++j) if (live && idx + j < count) dst[idx + j] = e[j];
            }
        }
        __syncthreads();
    }
}

static int zvc_ensure_counters(vdnn_ctx* ctx) {
    if (ctx->zvc_counters) return VDNN_OK;
    // [0]: bytes over the link; [1 .. kZvcCursors]: stream cursors, one per offload in flight
    VDNN_HIP(hipMalloc((void**)&ctx->zvc_counters, sizeof(unsigned long long) * (1 + kZvcCursors)));
    VDNN_HIP(hipMemset(ctx->zvc_counters, 0, sizeof(unsigned long long) * (1 + kZvcCursors)));
    return VDNN_OK;
}

static int zvc_offload(vdnn_ctx* ctx, void* dst_host, void* staging_dev, size_t staging_bytes, const void* src_dev, size_t count,
                       int elem_bytes, unsigned long long* total_host, vdnn_stream_t pack_stream, vdnn_stream_t copy_stream, vdnn_event_t packed,
                       bool keep_on_device) {
    VDNN_REQUIRE(ctx, "null context");
    VDNN_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "elements are two or four bytes");
    if (ctx->plan_only) return VDNN_OK;
    hipStream_t cs = copy_stream ? (hipStream_t)copy_stream : ctx->d2h;
    // without an event to order the two streams the kernels run on the copy stream
    hipStream_t ps = !packed ? cs : pack_stream ? (hipStream_t)pack_stream : ctx->pack;
    if (count == 0) {
        if (packed) { VDNN_HIP(hipEventRecord((hipEvent_t)packed, ps)); VDNN_HIP(hipStreamWaitEvent(cs, (hipEvent_t)packed, 0)); }
        return VDNN_OK;
    }
    VDNN_REQUIRE(dst_host && src_dev, "null pointer");
    VDNN_REQUIRE(((uintptr_t)dst_host & 15) == 0 && ((uintptr_t)src_dev & (elem_bytes - 1)) == 0, "misaligned buffer");
    VDNN_REQUIRE(staging_bytes == 0 || (staging_dev && ((uintptr_t)staging_dev & 15) == 0 && staging_bytes % 16 == 0),
                 "staging buffer: 16-byte aligned, a multiple of 16 bytes");
    VDNN_REQUIRE(staging_bytes <= vdnn_zvc_buffer_bytes(count, elem_bytes), "staging buffer longer than the longest stream");
    if (int rc = zvc_ensure_counters(ctx)) return rc;
    const size_t chunks = (count + kZvcChunk - 1) / kZvcChunk;
    unsigned long long* cursor = ctx->zvc_counters + 1 + (ctx->zvc_next_cursor++ % kZvcCursors);
    // with a staging buffer the kernel works at HBM speed and should be gone soon; without one it is bound by
    // the link and by how many stores it may have in flight
    const size_t need = (chunks + kZvcTeams - 1) / kZvcTeams;
    const size_t cap = staging_bytes ? size_t(ctx->num_cu) * 2 : size_t(ctx->num_cu) / 8;
    const int grid = int(need < cap ? need : cap);
    {
        ProfScope prof(ctx, ps, staging_bytes ? "offload_zvc_pack" : "offload_zvc", 0.0, (double)(count * elem_bytes));
        zvc_begin_kernel<<<1, 1, 0, ps>>>(cursor, zvc_table_bytes(chunks));
        if (elem_bytes == 4)
            zvc_pack_kernel<uint32_t><<<grid, kZvcThreads, 0, ps>>>((const uint32_t*)src_dev, count, chunks, (unsigned char*)staging_dev, staging_bytes,
                                                                     (unsigned char*)dst_host, cursor);
        else
            zvc_pack_kernel<uint16_t><<<grid, kZvcThreads, 0, ps>>>((const uint16_t*)src_dev, count, chunks, (unsigned char*)staging_dev, staging_bytes,
                                                                     (unsigned char*)dst_host, cursor);
        VDNN_HIP(hipGetLastError());
        zvc_end_kernel<<<1, 1, 0, ps>>>(cursor, keep_on_device ? ~0ull : (unsigned long long)staging_bytes, (unsigned long long)staging_bytes, total_host,
                                     ctx->zvc_counters);
        VDNN_HIP(hipGetLastError());
    }
    if (packed) {
        VDNN_HIP(hipEventRecord((hipEvent_t)packed, ps));
        VDNN_HIP(hipStreamWaitEvent(cs, (hipEvent_t)packed, 0));
    }
    if (staging_bytes && !keep_on_device) {
        ProfScope prof(ctx, cs, "offload_zvc_copy", 0.0, (double)(count * elem_bytes));
        VDNN_HIP(hipMemcpyAsync(dst_host, staging_dev, staging_bytes, hipMemcpyDeviceToHost, cs));
    }
    ctx->zvc_raw_bytes += (unsigned long long)count * elem_bytes;
    return VDNN_OK;
}

} // namespace vdnn

using namespace vdnn;

size_t vdnn_zvc_buffer_bytes(size_t count, int elem_bytes) {
    if (elem_bytes != 2 && elem_bytes != 4) return 0;
    const size_t chunks = (count + kZvcChunk - 1) / kZvcChunk;
    return zvc_table_bytes(chunks) + chunks * zvc_record_bytes_max(elem_bytes);
}

int vdnn_zvc_offload_async(vdnn_ctx* ctx, void* dst_host, const void* src_dev, size_t count, int elem_bytes, vdnn_stream_t stream) {
    return zvc_offload(ctx, dst_host, nullptr, 0, src_dev, count, elem_bytes, nullptr, nullptr, stream, nullptr, false);
}

int vdnn_zvc_offload_staged_async(vdnn_ctx* ctx, void* dst_host, void* staging_dev, size_t staging_bytes, const void* src_dev, size_t count,
                                  int elem_bytes, unsigned long long* total_host, vdnn_stream_t pack_stream, vdnn_stream_t copy_stream,
                                  vdnn_event_t packed, int keep_on_device) {
    return zvc_offload(ctx, dst_host, staging_dev, staging_bytes, src_dev, count, elem_bytes, total_host, pack_stream, copy_stream, packed,
                       keep_on_device != 0);
}

static int zvc_prefetch(vdnn_ctx* ctx, void* dst_dev, const void* staging_dev, size_t staging_bytes, const void* src_host, size_t count,
                        int elem_bytes, vdnn_stream_t stream) {
    VDNN_REQUIRE(ctx, "null context");
    VDNN_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "elements are two or four bytes");
    if (ctx->plan_only || count == 0) return VDNN_OK;
    VDNN_REQUIRE(dst_dev && src_host, "null pointer");
    VDNN_REQUIRE(((uintptr_t)src_host & 15) == 0 && ((uintptr_t)dst_dev & (elem_bytes - 1)) == 0, "misaligned buffer");
    VDNN_REQUIRE(staging_bytes == 0 || (staging_dev && ((uintptr_t)staging_dev & 15) == 0 && staging_bytes % 16 == 0),
                 "staging buffer: 16-byte aligned, a multiple of 16 bytes");
    hipStream_t s = stream ? (hipStream_t)stream : ctx->h2d;
    const size_t chunks = (count + kZvcChunk - 1) / kZvcChunk;
    // from host memory: enough records in flight to keep the link busy across their round trips, on an eighth of
    // the compute units; from a block on the device: the whole device, briefly
    const size_t need = (chunks + kZvcTeams - 1) / kZvcTeams;
    const size_t cap = staging_bytes ? size_t(ctx->num_cu) * 2 : size_t(ctx->num_cu) / 8;
    const int grid = int(need < cap ? need : cap);
    ProfScope prof(ctx, s, staging_bytes ? "prefetch_zvc_device" : "prefetch_zvc", 0.0, (double)(count * elem_bytes));
    if (elem_bytes == 4)
        zvc_unpack_kernel<uint32_t><<<grid, kZvcThreads, 0, s>>>((const unsigned char*)staging_dev, staging_bytes, (const unsigned char*)src_host,
                                                                  (uint32_t*)dst_dev, count, chunks);
    else
        zvc_unpack_kernel<uint16_t><<<grid, kZvcThreads, 0, s>>>((const unsigned char*)staging_dev, staging_bytes, (const unsigned char*)src_host,
                                                                  (uint16_t*)dst_dev, count, chunks);
    VDNN_HIP(hipGetLastError());
    return VDNN_OK;
}

int vdnn_zvc_prefetch_async(vdnn_ctx* ctx, void* dst_dev, const void* src_host, size_t count, int elem_bytes, vdnn_stream_t stream) {
    return zvc_prefetch(ctx, dst_dev, nullptr, 0, src_host, count, elem_bytes, stream);
}

int vdnn_zvc_prefetch_staged_async(vdnn_ctx* ctx, void* dst_dev, const void* staging_dev, size_t staging_bytes, const void* src_host,
                                   size_t count, int elem_bytes, vdnn_stream_t stream) {
    return zvc_prefetch(ctx, dst_dev, staging_dev, staging_bytes, src_host, count, elem_bytes, stream);
}

int vdnn_zvc_traffic(vdnn_ctx* ctx, unsigned long long* tensor_bytes, unsigned long long* link_bytes) {
    VDNN_REQUIRE(ctx && tensor_bytes && link_bytes, "null argument");
    *tensor_bytes = ctx->zvc_raw_bytes;
    *link_bytes = 0;
    if (ctx->plan_only || !ctx->zvc_counters) return VDNN_OK;
    VDNN_HIP(hipDeviceSynchronize());
    VDNN_HIP(hipMemcpy(link_bytes, ctx->zvc_counters, sizeof(unsigned long long), hipMemcpyDeviceToHost));
    return VDNN_OK;
}
