// probe.hip -- measuring kernels for bench.py, built into their own library
// (benchlib/libtccl_probe.so); nothing here is part of the product or its ABI.
//
//  * the read half and the write half of the phased sum, each on its own, with the same launch
//    shape (256 lanes, 128 KiB tiles, two workgroups per compute unit, one launch per resident
//    wave of tiles).  What the memory system gives a pure read pass and a pure write pass
//    bounds what the sum can reach (its launch is a read phase followed by a write burst), so
//    the benchmark can print that bound beside the sum's own time on whatever GPU it runs on;
//  * an empty kernel, for the launch floor of a timed single launch;
//  * a kernel that reports where the hardware put each of its workgroups.
#include "../tccl_amd/csrc/host.h"
#include "../tccl_amd/csrc/vec.h"
#include "probe.h"

namespace tccl {

// compute units of the current device (the product's own helper lives in its library)
static int probe_compute_units()
{
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        prop.multiProcessorCount > 0)
        return prop.multiProcessorCount;
    return 256;
}

template <int NSRC>
struct ProbeSrc {
    const char *p[NSRC];
};

// Loads and reduces a tile exactly as sum_tile_phased does (bf16 arithmetic), but keeps only
// a checksum of the results; the store below depends on it, so nothing can be optimised
// away, and it fires for one checksum value in 2^32.
template <int NSRC>
__global__ void __launch_bounds__(kPhasedBlock) probe_read_kernel(ProbeSrc<NSRC> src, char *sink, size_t bytes)
{
    constexpr int U = PhasedUnroll<NSRC>::value;
    constexpr int KMAX = kPhasedVecs / U;
    constexpr uint32_t tile_bytes = kPhasedBlock * kPhasedVecs * kVecBytes;
    constexpr uint32_t span_bytes = kPhasedBlock * U * kVecBytes;
    const size_t off = static_cast<size_t>(blockIdx.x) * tile_bytes;
    const size_t left = bytes > off ? bytes - off : 0;
    const uint32_t valid = static_cast<uint32_t>(left < tile_bytes ? left : tile_bytes);
    __amdgpu_buffer_rsrc_t rs[NSRC];
#pragma unroll
    for (int s = 0; s < NSRC; ++s) rs[s] = tile_rsrc(src.p[s] + off, valid);
    const uint32_t lane_off = threadIdx.x * kVecBytes;
    uint32_t keep = 0;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        u32x4 v[U][NSRC];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int s = 0; s < NSRC; ++s)
                v[u][s] = __builtin_amdgcn_raw_buffer_load_b128(
                    rs[s], k * span_bytes + u * (kPhasedBlock * kVecBytes) + lane_off, 0, kAuxLoadStream);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            Bf16Sum acc;
            acc.zero();
#pragma unroll
            for (int s = 0; s < NSRC; ++s) acc.add(v[u][s]);
            const u32x4 r = acc.result();
            keep ^= r[0] ^ r[1] ^ r[2] ^ r[3];
        }
    }
    if (keep == 0x9E3779B9u) {
        const __amdgpu_buffer_rsrc_t rd = tile_rsrc(sink, kPhasedBlock * kVecBytes);
        const u32x4 out = {keep, keep, keep, keep};
        __builtin_amdgcn_raw_buffer_store_b128(out, rd, lane_off, 0, 0);
    }
}

// Writes a tile the way sum_tile_phased writes its results: 32 stores per lane back to back.
__global__ void __launch_bounds__(kPhasedBlock) probe_write_kernel(char *dst, size_t bytes, uint32_t value)
{
    constexpr uint32_t tile_bytes = kPhasedBlock * kPhasedVecs * kVecBytes;
    const size_t off = static_cast<size_t>(blockIdx.x) * tile_bytes;
    const size_t left = bytes > off ? bytes - off : 0;
    const uint32_t valid = static_cast<uint32_t>(left < tile_bytes ? left : tile_bytes);
    const __amdgpu_buffer_rsrc_t rd = tile_rsrc(dst + off, valid);
    const uint32_t lane_off = threadIdx.x * kVecBytes;
    const u32x4 v = {value, value + threadIdx.x, value ^ blockIdx.x, value};
#pragma unroll
    for (int k = 0; k < kPhasedVecs; ++k)
        __builtin_amdgcn_raw_buffer_store_b128(v, rd, k * (kPhasedBlock * kVecBytes) + lane_off, 0, kAuxStoreStream);
}

// The same stores in 32 KiB tiles (8 per lane): four times as many workgroups, whose write fronts
// move through memory more closely together; the fastest way found to write HBM in tiles.
__global__ void __launch_bounds__(kPhasedBlock) probe_write_small_kernel(char *dst, size_t bytes, uint32_t value)
{
    constexpr int VECS = 8;
    constexpr uint32_t tile_bytes = kPhasedBlock * VECS * kVecBytes;
    const size_t off = static_cast<size_t>(blockIdx.x) * tile_bytes;
    const size_t left = bytes > off ? bytes - off : 0;
    const uint32_t valid = static_cast<uint32_t>(left < tile_bytes ? left : tile_bytes);
    const __amdgpu_buffer_rsrc_t rd = tile_rsrc(dst + off, valid);
    const uint32_t lane_off = threadIdx.x * kVecBytes;
    const u32x4 v = {value, value + threadIdx.x, value ^ blockIdx.x, value};
#pragma unroll
    for (int k = 0; k < VECS; ++k)
        __builtin_amdgcn_raw_buffer_store_b128(v, rd, k * (kPhasedBlock * kVecBytes) + lane_off, 0, kAuxStoreStream);
}

// One workgroup per compute unit, each writing 4 KiB per step at a stride of the whole grid: the
// GPU writes one dense 1 MiB window at a time with one wave per SIMD.  The fastest way found to
// write HBM (more workgroups, or more bytes per workgroup per step, are slower); no kernel that
// reads what it writes in tiles can write like this.
__global__ void __launch_bounds__(kPhasedBlock) probe_write_dense_kernel(char *dst, size_t bytes, uint32_t value)
{
    constexpr size_t piece = static_cast<size_t>(kPhasedBlock) * kVecBytes;
    const u32x4 v = {value, value + threadIdx.x, value ^ blockIdx.x, value};
    for (size_t off = blockIdx.x * piece; off < bytes; off += gridDim.x * piece) {
        const size_t left = bytes - off;
        const __amdgpu_buffer_rsrc_t rd = tile_rsrc(dst + off, static_cast<uint32_t>(left < piece ? left : piece));
        __builtin_amdgcn_raw_buffer_store_b128(v, rd, threadIdx.x * kVecBytes, 0, kAuxStoreStream);
    }
}

template <int NSRC>
static hipError_t launch_probe_read(const void *const *bufs, char *sink, size_t bytes, hipStream_t stream)
{
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * kPhasedVecs * kVecBytes;
    const size_t slice = static_cast<size_t>(probe_compute_units()) * 2 * tile_bytes; // one resident wave of tiles
    for (size_t off = 0; off < bytes; off += slice) {
        const size_t n = bytes - off < slice ? bytes - off : slice;
        ProbeSrc<NSRC> t;
        for (int i = 0; i < NSRC; ++i) t.p[i] = static_cast<const char *>(bufs[i]) + off;
        const size_t grid = (n + tile_bytes - 1) / tile_bytes;
        hipLaunchKernelGGL(probe_read_kernel<NSRC>, dim3(static_cast<unsigned>(grid)), dim3(kPhasedBlock), 0, stream, t,
                           sink, n);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

} // namespace tccl

using namespace tccl;

extern "C" int tccl_probe_read(const void *const *bufs, int world, size_t bytes_per_buffer, void *sink, void *stream)
{
    if (bufs == nullptr || sink == nullptr || world < 1 || world > TCCL_MAX_WORLD) return TCCL_EINVAL;
    if (bytes_per_buffer % kVecBytes != 0 || !aligned16(sink)) return TCCL_EALIGN;
    for (int i = 0; i < world; ++i) {
        if (bufs[i] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[i])) return TCCL_EALIGN;
    }
    if (bytes_per_buffer == 0) return TCCL_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    char *k = static_cast<char *>(sink);
    hipError_t e;
    switch (world) {
    case 1: e = launch_probe_read<1>(bufs, k, bytes_per_buffer, s); break;
    case 2: e = launch_probe_read<2>(bufs, k, bytes_per_buffer, s); break;
    case 3: e = launch_probe_read<3>(bufs, k, bytes_per_buffer, s); break;
    case 4: e = launch_probe_read<4>(bufs, k, bytes_per_buffer, s); break;
    case 5: e = launch_probe_read<5>(bufs, k, bytes_per_buffer, s); break;
    case 6: e = launch_probe_read<6>(bufs, k, bytes_per_buffer, s); break;
    case 7: e = launch_probe_read<7>(bufs, k, bytes_per_buffer, s); break;
    default: e = launch_probe_read<8>(bufs, k, bytes_per_buffer, s); break;
    }
    return hip_code(e);
}

extern "C" int tccl_probe_write(void *dst, size_t bytes, void *stream)
{
    if (dst == nullptr) return TCCL_EINVAL;
    if (bytes % kVecBytes != 0 || !aligned16(dst)) return TCCL_EALIGN;
    if (bytes == 0) return TCCL_OK;
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * kPhasedVecs * kVecBytes;
    const size_t slice = static_cast<size_t>(probe_compute_units()) * 2 * tile_bytes;
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (size_t off = 0; off < bytes; off += slice) {
        const size_t n = bytes - off < slice ? bytes - off : slice;
        const size_t grid = (n + tile_bytes - 1) / tile_bytes;
        hipLaunchKernelGGL(probe_write_kernel, dim3(static_cast<unsigned>(grid)), dim3(kPhasedBlock), 0, s,
                           static_cast<char *>(dst) + off, n, 0x3F803F80u);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return hip_code(e);
    }
    return TCCL_OK;
}

namespace tccl {

// One contiguous range read by a grid-stride loop, four vectors per lane in flight, streaming
// loads: the most this GPU was found to read from HBM with any access pattern.
__global__ void __launch_bounds__(kPhasedBlock) probe_read_dense_kernel(const char *p, size_t bytes, char *sink)
{
    constexpr int U = 4;
    constexpr size_t step = static_cast<size_t>(U) * kPhasedBlock * kVecBytes;
    uint32_t keep = 0;
    for (size_t off = blockIdx.x * step; off < bytes; off += gridDim.x * step) {
        const size_t left = bytes - off;
        const __amdgpu_buffer_rsrc_t rs = tile_rsrc(p + off, static_cast<uint32_t>(left < step ? left : step));
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, u * (kPhasedBlock * kVecBytes) + threadIdx.x * kVecBytes, 0,
                                                         kAuxLoadStream);
#pragma unroll
        for (int u = 0; u < U; ++u) keep ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
    if (keep == 0x9E3779B9u) {
        const __amdgpu_buffer_rsrc_t rd = tile_rsrc(sink, kPhasedBlock * kVecBytes);
        const u32x4 out = {keep, keep, keep, keep};
        __builtin_amdgcn_raw_buffer_store_b128(out, rd, threadIdx.x * kVecBytes, 0, 0);
    }
}

// A plain copy in the shape that measured fastest on data that is in no cache: one workgroup per
// compute unit, four vectors per lane, streaming loads, write-through stores.
__global__ void __launch_bounds__(kPhasedBlock) probe_copy_kernel(const char *src, char *dst, size_t bytes)
{
    constexpr int U = 4;
    constexpr size_t step = static_cast<size_t>(U) * kPhasedBlock * kVecBytes;
    for (size_t off = blockIdx.x * step; off < bytes; off += gridDim.x * step) {
        const size_t left = bytes - off;
        const uint32_t valid = static_cast<uint32_t>(left < step ? left : step);
        const __amdgpu_buffer_rsrc_t rs = tile_rsrc(src + off, valid), rd = tile_rsrc(dst + off, valid);
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
            v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, u * (kPhasedBlock * kVecBytes) + threadIdx.x * kVecBytes, 0,
                                                         kAuxLoadStream);
#pragma unroll
        for (int u = 0; u < U; ++u)
            __builtin_amdgcn_raw_buffer_store_b128(v[u], rd, u * (kPhasedBlock * kVecBytes) + threadIdx.x * kVecBytes, 0,
                                                   kAuxStoreStream);
    }
}

// The large all-reduce's tile (8 bf16 sources, 128 KiB, 256 lanes x 32 vectors) with three
// readings of the 100 MHz wall clock per workgroup: at its start, when its last load has been
// reduced, and when its last store has been acknowledged.
__global__ void __launch_bounds__(kPhasedBlock) probe_sum_timed_kernel(ProbeSrc<8> src, char *out, size_t bytes, long long *stamps)
{
    const long long t0 = wall_clock64();
    constexpr uint32_t tile_bytes = kPhasedBlock * kPhasedVecs * kVecBytes;
    constexpr uint32_t span_bytes = kPhasedBlock * kVecBytes;
    const size_t off = static_cast<size_t>(blockIdx.x) * tile_bytes;
    const size_t left = bytes > off ? bytes - off : 0;
    const uint32_t valid = static_cast<uint32_t>(left < tile_bytes ? left : tile_bytes);
    __amdgpu_buffer_rsrc_t rs[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) rs[s] = tile_rsrc(src.p[s] + off, valid);
    const uint32_t lane_off = threadIdx.x * kVecBytes;
    u32x4 r[kPhasedVecs];
#pragma unroll
    for (int k = 0; k < kPhasedVecs; ++k) {
        u32x4 v[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) v[s] = __builtin_amdgcn_raw_buffer_load_b128(rs[s], k * span_bytes + lane_off, 0, kAuxLoadStream);
        Bf16Sum acc;
        acc.zero();
#pragma unroll
        for (int s = 0; s < 8; ++s) acc.add(v[s]);
        r[k] = acc.result();
    }
    __builtin_amdgcn_sched_barrier(0);
    const long long t1 = wall_clock64();
    __builtin_amdgcn_sched_barrier(0);
    const __amdgpu_buffer_rsrc_t rd = tile_rsrc(out + off, valid);
#pragma unroll
    for (int k = 0; k < kPhasedVecs; ++k) __builtin_amdgcn_raw_buffer_store_b128(r[k], rd, k * span_bytes + lane_off, 0, kAuxStoreStream);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const long long t2 = wall_clock64();
    if (threadIdx.x == 0) {
        stamps[3 * blockIdx.x] = t0;
        stamps[3 * blockIdx.x + 1] = t1;
        stamps[3 * blockIdx.x + 2] = t2;
    }
}

__global__ void probe_empty_kernel() {}

// One lane writes the 100 MHz wall clock, which every process on the GPU reads the same.
__global__ void probe_stamp_kernel(long long *slot)
{
    if (threadIdx.x == 0) *slot = static_cast<long long>(wall_clock64());
}

// The same grid as a sum launch doing nothing, and doing the least a streaming kernel can do:
// every lane loads one vector and stores it (one round trip to memory each way).  Their
// durations are the part of a short kernel's time that does not depend on its bytes.
__global__ void __launch_bounds__(kPhasedBlock) probe_empty_grid_kernel() {}

__global__ void __launch_bounds__(kPhasedBlock) probe_touch_kernel(const char *src, char *dst)
{
    const uint32_t bytes = kPhasedBlock * kVecBytes;
    const size_t off = static_cast<size_t>(blockIdx.x) * bytes;
    const __amdgpu_buffer_rsrc_t rs = tile_rsrc(src + off, bytes);
    const __amdgpu_buffer_rsrc_t rd = tile_rsrc(dst + off, bytes);
    const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rs, threadIdx.x * kVecBytes, 0, kAuxLoadStream);
    __builtin_amdgcn_raw_buffer_store_b128(v, rd, threadIdx.x * kVecBytes, 0, kAuxStoreStream);
}

// Every workgroup holds its slot for `hold_ticks` of the 100 MHz wall clock (so that the whole
// grid is resident together) and reports the XCD and the hardware id it ran on.
__global__ void __launch_bounds__(kPhasedBlock) probe_placement_kernel(uint32_t *out, long long hold_ticks)
{
    const uint32_t hw = __builtin_amdgcn_s_getreg(4 | (0 << 6) | (31 << 11));   // HW_REG_HW_ID
    const uint32_t xcc = __builtin_amdgcn_s_getreg(20 | (0 << 6) | (31 << 11)); // HW_REG_XCC_ID
    const long long t0 = wall_clock64();
    while (wall_clock64() - t0 < hold_ticks) __builtin_amdgcn_s_sleep(8);
    if (threadIdx.x == 0) {
        out[2 * blockIdx.x] = hw;
        out[2 * blockIdx.x + 1] = xcc;
    }
}

} // namespace tccl

extern "C" int tccl_probe_write_small(void *dst, size_t bytes, void *stream)
{
    if (dst == nullptr) return TCCL_EINVAL;
    if (bytes % kVecBytes != 0 || !aligned16(dst)) return TCCL_EALIGN;
    if (bytes == 0) return TCCL_OK;
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * 8 * kVecBytes;
    const size_t grid = (bytes + tile_bytes - 1) / tile_bytes;
    if (grid > 0x7FFFFFFFu) return TCCL_EINVAL;
    hipLaunchKernelGGL(probe_write_small_kernel, dim3(static_cast<unsigned>(grid)), dim3(kPhasedBlock), 0,
                       static_cast<hipStream_t>(stream), static_cast<char *>(dst), bytes, 0x3F803F80u);
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_write_dense(void *dst, size_t bytes, void *stream)
{
    if (dst == nullptr) return TCCL_EINVAL;
    if (bytes % kVecBytes != 0 || !aligned16(dst)) return TCCL_EALIGN;
    if (bytes == 0) return TCCL_OK;
    hipLaunchKernelGGL(probe_write_dense_kernel, dim3(probe_compute_units()), dim3(kPhasedBlock), 0,
                       static_cast<hipStream_t>(stream), static_cast<char *>(dst), bytes, 0x3F803F80u);
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_read_dense(const void *buf, size_t bytes, void *sink, void *stream)
{
    if (buf == nullptr || sink == nullptr) return TCCL_EINVAL;
    if (bytes % kVecBytes != 0 || !aligned16(buf) || !aligned16(sink)) return TCCL_EALIGN;
    if (bytes == 0) return TCCL_OK;
    hipLaunchKernelGGL(probe_read_dense_kernel, dim3(probe_compute_units() * 2), dim3(kPhasedBlock), 0,
                       static_cast<hipStream_t>(stream), static_cast<const char *>(buf), bytes, static_cast<char *>(sink));
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_copy(const void *src, void *dst, size_t bytes, void *stream)
{
    if (src == nullptr || dst == nullptr) return TCCL_EINVAL;
    if (bytes % kVecBytes != 0 || !aligned16(src) || !aligned16(dst)) return TCCL_EALIGN;
    if (bytes == 0) return TCCL_OK;
    hipLaunchKernelGGL(probe_copy_kernel, dim3(probe_compute_units()), dim3(kPhasedBlock), 0,
                       static_cast<hipStream_t>(stream), static_cast<const char *>(src), static_cast<char *>(dst), bytes);
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_sum_timed(const void *const *bufs, void *out, size_t bytes_per_buffer, long long *stamps, void *stream)
{
    if (bufs == nullptr || out == nullptr || stamps == nullptr) return TCCL_EINVAL;
    if (bytes_per_buffer % kVecBytes != 0 || !aligned16(out)) return TCCL_EALIGN;
    ProbeSrc<8> t;
    for (int i = 0; i < 8; ++i) {
        if (bufs[i] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[i])) return TCCL_EALIGN;
        t.p[i] = static_cast<const char *>(bufs[i]);
    }
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * kPhasedVecs * kVecBytes;
    const size_t grid = (bytes_per_buffer + tile_bytes - 1) / tile_bytes;
    if (grid < 1 || grid > 65536) return TCCL_EINVAL;
    hipLaunchKernelGGL(probe_sum_timed_kernel, dim3(static_cast<unsigned>(grid)), dim3(kPhasedBlock), 0,
                       static_cast<hipStream_t>(stream), t, static_cast<char *>(out), bytes_per_buffer, stamps);
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_empty(void *stream)
{
    hipLaunchKernelGGL(probe_empty_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream));
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_stamp(long long *slot, void *stream)
{
    if (slot == nullptr) return TCCL_EINVAL;
    hipLaunchKernelGGL(probe_stamp_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), slot);
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_empty_grid(int workgroups, void *stream)
{
    if (workgroups < 1 || workgroups > 65536) return TCCL_EINVAL;
    hipLaunchKernelGGL(probe_empty_grid_kernel, dim3(workgroups), dim3(kPhasedBlock), 0, static_cast<hipStream_t>(stream));
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_touch(const void *src, void *dst, int workgroups, void *stream)
{
    if (src == nullptr || dst == nullptr || workgroups < 1 || workgroups > 65536) return TCCL_EINVAL;
    hipLaunchKernelGGL(probe_touch_kernel, dim3(workgroups), dim3(kPhasedBlock), 0, static_cast<hipStream_t>(stream),
                       static_cast<const char *>(src), static_cast<char *>(dst));
    return hip_code(hipGetLastError());
}

extern "C" int tccl_probe_placement(uint32_t *out, int workgroups, int hold_us, void *stream)
{
    if (out == nullptr || workgroups < 1 || workgroups > (1 << 20) || hold_us < 0 || hold_us > 100000) return TCCL_EINVAL;
    hipLaunchKernelGGL(probe_placement_kernel, dim3(workgroups), dim3(kPhasedBlock), 0, static_cast<hipStream_t>(stream),
                       out, static_cast<long long>(hold_us) * 100);
    return hip_code(hipGetLastError());
}
