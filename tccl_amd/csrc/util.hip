// util.hip -- launch-shape selection, error strings, HIP-event helpers, device facts.
#include <atomic>

#include "host.h"
#include "vec.h"

namespace tccl {

int compute_units()
{
    static std::atomic<int> cached{0};
    int cu = cached.load(std::memory_order_relaxed);
    if (cu > 0) return cu;
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
        prop.multiProcessorCount > 0)
        cu = prop.multiProcessorCount;
    else
        cu = 256; // MI355X
    cached.store(cu, std::memory_order_relaxed);
    return cu;
}

Shape resolve_shape(const tccl_launch_cfg *cfg, size_t nvec, int nsrc, int rows, bool is_copy)
{
    tccl_launch_cfg c = {};
    if (cfg) c = *cfg;
    Shape sh;
    const int cus = compute_units();
    // Copies of data that is not already in a cache (the case that counts: a collective's input has
    // just been produced elsewhere) run best with four vectors per lane in flight and streaming loads
    // and stores, on two workgroups per compute unit (one from 384 MiB of output): measured on buffers
    // rotated so that nothing is served from the 256 MB memory-side cache, that shape is as fast as or
    // faster than full occupancy with plain loads at every size from 8 MiB to 512 MiB (+7 % at 128 MiB).
    const size_t copy_bytes = is_copy ? nvec * rows * kVecBytes : 0;
    const bool big_copy = copy_bytes >= (static_cast<size_t>(384) << 20);
    const bool mid_copy = !big_copy && copy_bytes >= (static_cast<size_t>(8) << 20);

    sh.block = (c.block == 64 || c.block == 128 || c.block == 256 || c.block == 512) ? c.block : 256;

    // Vectors in flight per lane: aim for about eight 16-byte loads, but never so many that
    // a small input is spread over fewer workgroups than twice the compute units.
    if (c.unroll == 1 || c.unroll == 2 || c.unroll == 4) {
        sh.unroll = c.unroll;
    } else {
        int u = is_copy ? ((big_copy || mid_copy) ? 4 : 2) : 8 / nsrc;
        u = u >= 4 ? 4 : (u >= 2 ? 2 : 1);
        while (u > 1 && nvec * rows / (static_cast<size_t>(sh.block) * u) < static_cast<size_t>(cus) * 2) u /= 2;
        sh.unroll = u;
    }
    if (nsrc > 4 && sh.unroll > 2) sh.unroll = 2;

    sh.tile_iters = c.tile_iters > 0 ? c.tile_iters : 1;

    const size_t tile = static_cast<size_t>(sh.block) * sh.unroll * sh.tile_iters;
    size_t ntiles = (nvec + tile - 1) / tile * rows; // the grid is shared by all rows
    if (ntiles == 0) ntiles = 1;

    const int flags = c.flags;
    sh.xcd_contiguous = (flags & TCCL_CFG_XCD_CONTIGUOUS) != 0;
    if (flags & TCCL_CFG_TEMPORAL) {
        sh.nt_load = false;
        sh.nt_store = false;
    } else {
        sh.nt_load = (flags & TCCL_CFG_NONTEMPORAL_LOAD) != 0;
        sh.nt_store = (flags & TCCL_CFG_NONTEMPORAL_STORE) != 0;
        const bool unspecified = (flags & (TCCL_CFG_NONTEMPORAL_LOAD | TCCL_CFG_NONTEMPORAL_STORE)) == 0;
        if ((big_copy || mid_copy) && unspecified) sh.nt_load = sh.nt_store = true;
    }

    // Workgroups: enough to keep every compute unit at full wave occupancy
    // (2048 lanes per CU).
    size_t grid;
    if (c.grid > 0) {
        grid = static_cast<size_t>(c.grid);
    } else {
        const size_t per_cu = big_copy ? 1 : (mid_copy ? 2 : 2048 / sh.block);
        grid = static_cast<size_t>(cus) * per_cu;
    }
    if (grid > ntiles) grid = ntiles;
    if (sh.xcd_contiguous) grid = (grid + kNumXcd - 1) / kNumXcd * kNumXcd;
    if (grid > 0x7FFFFFFFu) grid = 0x7FFFFFFFu;
    sh.grid = static_cast<int>(grid);
    return sh;
}

} // namespace tccl

using namespace tccl;

extern "C" int tccl_abi_version(void) { return TCCL_ABI_VERSION; }

extern "C" const char *tccl_error_string(int code)
{
    switch (code) {
    case TCCL_OK: return "ok";
    case TCCL_EINVAL: return "invalid argument (NULL pointer, world/rank/dtype out of range)";
    case TCCL_EALIGN: return "pointer or size is not a multiple of 16 bytes";
    case TCCL_EPOW2: return "world size is not a power of two >= 2";
    case TCCL_ESCRATCH: return "the request needs more scratch memory than the library's static buffer holds";
    case TCCL_ETIMEOUT: return "a wait of a signalling kernel expired: that collective's results are incomplete";
    default:
        if (code <= TCCL_EHIP_BASE) return hipGetErrorString(static_cast<hipError_t>(TCCL_EHIP_BASE - code));
        return "unknown error";
    }
}

extern "C" int tccl_event_create(void **event_out)
{
    if (event_out == nullptr) return TCCL_EINVAL;
    hipEvent_t e = nullptr;
    hipError_t rc = hipEventCreate(&e);
    *event_out = e;
    return hip_code(rc);
}

extern "C" int tccl_event_destroy(void *event) { return hip_code(hipEventDestroy(static_cast<hipEvent_t>(event))); }

extern "C" int tccl_event_record(void *event, void *stream)
{
    return hip_code(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
}

extern "C" int tccl_event_synchronize(void *event)
{
    return hip_code(hipEventSynchronize(static_cast<hipEvent_t>(event)));
}

extern "C" int tccl_event_elapsed_ms(void *start, void *stop, float *ms_out)
{
    if (ms_out == nullptr) return TCCL_EINVAL;
    return hip_code(hipEventElapsedTime(ms_out, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
}

extern "C" int tccl_stream_synchronize(void *stream)
{
    return hip_code(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
}

extern "C" int tccl_device_info(int *compute_units_out, int *mem_clock_khz, int *mem_bus_bits, size_t *l2_bytes)
{
    int dev = 0;
    hipError_t rc = hipGetDevice(&dev);
    if (rc != hipSuccess) return hip_code(rc);
    hipDeviceProp_t prop;
    rc = hipGetDeviceProperties(&prop, dev);
    if (rc != hipSuccess) return hip_code(rc);
    if (compute_units_out) *compute_units_out = prop.multiProcessorCount;
    if (mem_clock_khz) *mem_clock_khz = prop.memoryClockRate;
    if (mem_bus_bits) *mem_bus_bits = prop.memoryBusWidth;
    if (l2_bytes) *l2_bytes = static_cast<size_t>(prop.l2CacheSize);
    return TCCL_OK;
}
