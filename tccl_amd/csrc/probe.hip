// probe.hip -- two measuring kernels: the read half and the write half of the phased sum,
// each on its own, with the same launch shape (256 lanes, 128 KiB tiles, two workgroups per
// compute unit, one launch per resident wave of tiles).  What the memory system gives a pure
// read pass and a pure write pass bounds what the sum can reach (its launch is a read phase
// followed by a write burst), so a benchmark can print that bound beside the sum's own time
// on whatever GPU it runs on.  No counterpart in the reference.
#include "host.h"
#include "vec.h"

namespace tccl {

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

template <int NSRC>
static hipError_t launch_probe_read(const void *const *bufs, char *sink, size_t bytes, hipStream_t stream)
{
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * kPhasedVecs * kVecBytes;
    const size_t slice = static_cast<size_t>(compute_units()) * 2 * tile_bytes; // one resident wave of tiles
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
    const size_t slice = static_cast<size_t>(compute_units()) * 2 * tile_bytes;
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
