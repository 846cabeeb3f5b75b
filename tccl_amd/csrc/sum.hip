// sum.hip -- one-shot all-reduce, reduce-scatter share and the single tree reduce step:
// all three are "sum NSRC source streams into one destination stream", launched over
// pointers that the host passes by value in the kernel arguments (they live in SGPRs;
// the reference re-reads a device pointer table for every rank in every iteration,
// triton_one_shot_all_reduce_no_128.py:59).
#include "host.h"
#include "vec.h"

namespace tccl {

template <int NSRC>
struct SrcTable {
    const char *p[NSRC];
};

template <class Sum, int NSRC, int UNROLL, bool NTL, bool NTS>
__global__ void __launch_bounds__(kMaxBlock)
sum_kernel(SrcTable<NSRC> src, char *out, size_t numel, int tile_iters, int xcd_contiguous)
{
    TCCL_STAMP(0, false);
    char *const dst[1] = {out};
    sum_range<Sum, NSRC, 1, UNROLL, NTL, NTS>(src.p, dst, numel, tile_iters, xcd_contiguous != 0);
    TCCL_STAMP(3, true);
}

template <class Sum, int NSRC, int UNROLL, bool NTL, bool NTS>
static hipError_t launch_sum(const char *const *srcs, char *out, size_t numel, const Shape &sh, hipStream_t stream)
{
    SrcTable<NSRC> t;
    for (int i = 0; i < NSRC; ++i) t.p[i] = srcs[i];
    hipLaunchKernelGGL((sum_kernel<Sum, NSRC, UNROLL, NTL, NTS>), dim3(sh.grid), dim3(sh.block), 0, stream, t, out,
                       numel, sh.tile_iters, sh.xcd_contiguous ? 1 : 0);
    return hipGetLastError();
}

template <class Sum, int NSRC, int UNROLL>
static hipError_t launch_sum_nt(const char *const *srcs, char *out, size_t numel, const Shape &sh, hipStream_t stream)
{
    if (sh.nt_load) {
        if (sh.nt_store) return launch_sum<Sum, NSRC, UNROLL, true, true>(srcs, out, numel, sh, stream);
        return launch_sum<Sum, NSRC, UNROLL, true, false>(srcs, out, numel, sh, stream);
    }
    if (sh.nt_store) return launch_sum<Sum, NSRC, UNROLL, false, true>(srcs, out, numel, sh, stream);
    return launch_sum<Sum, NSRC, UNROLL, false, false>(srcs, out, numel, sh, stream);
}

template <class Sum, int NSRC>
static hipError_t launch_sum_unroll(const char *const *srcs, char *out, size_t numel, const Shape &sh,
                                    hipStream_t stream)
{
    switch (sh.unroll) {
    case 1: return launch_sum_nt<Sum, NSRC, 1>(srcs, out, numel, sh, stream);
    case 2: return launch_sum_nt<Sum, NSRC, 2>(srcs, out, numel, sh, stream);
    default:
        // 4 vectors x 8 sources would hold 128 data registers per lane; cap it at 2 there.
        if constexpr (NSRC <= 4)
            return launch_sum_nt<Sum, NSRC, 4>(srcs, out, numel, sh, stream);
        else
            return launch_sum_nt<Sum, NSRC, 2>(srcs, out, numel, sh, stream);
    }
}

template <class Sum>
static hipError_t launch_sum_nsrc(const char *const *srcs, int nsrc, char *out, size_t numel, const Shape &sh,
                                  hipStream_t stream)
{
    switch (nsrc) {
    case 1: return launch_sum_unroll<Sum, 1>(srcs, out, numel, sh, stream);
    case 2: return launch_sum_unroll<Sum, 2>(srcs, out, numel, sh, stream);
    case 3: return launch_sum_unroll<Sum, 3>(srcs, out, numel, sh, stream);
    case 4: return launch_sum_unroll<Sum, 4>(srcs, out, numel, sh, stream);
    case 5: return launch_sum_unroll<Sum, 5>(srcs, out, numel, sh, stream);
    case 6: return launch_sum_unroll<Sum, 6>(srcs, out, numel, sh, stream);
    case 7: return launch_sum_unroll<Sum, 7>(srcs, out, numel, sh, stream);
    case 8: return launch_sum_unroll<Sum, 8>(srcs, out, numel, sh, stream);
    default: return hipErrorInvalidValue;
    }
}

// ---------------------------------------------------------------------------------
// Phased variant: one tile per workgroup, all of a launch's workgroups resident at once.

template <class Sum, int NSRC, int U, bool FULL>
__global__ void __launch_bounds__(kPhasedBlock)
sum_phased_kernel(SrcTable<NSRC> src, char *out, size_t bytes, int kcount, size_t tile_bytes, size_t tail_first,
                  size_t numel)
{
    // tile_bytes <= what kcount iterations cover; where it is less, the lanes beyond it load
    // nothing and store nothing (the tile's buffer descriptor ends there)
    TCCL_STAMP(0, false);
    constexpr int KMAX = kPhasedVecs / U;
    const size_t off = blockIdx.x * tile_bytes;
    const size_t left = bytes > off ? bytes - off : 0;
    const uint32_t valid = static_cast<uint32_t>(left < tile_bytes ? left : tile_bytes);
    char *const dst[1] = {out};
    sum_tile_phased<Sum, NSRC, 1, U, KMAX, FULL, Sum::kPaceLoads>(src.p, dst, off, valid, kcount);
    if (blockIdx.x == 0 && tail_first < numel) sum_tail<Sum, NSRC, 1>(src.p, dst, tail_first, numel);
}

// The same launch with unequal, interleaved tiles (three sources or more): workgroups 2p and 2p+1 share a region of
// 2 * KMAX pieces (a piece = what one iteration covers, 4 KiB), the even one taking KMAX + 1 and
// the odd one KMAX - 1 of them.  Workgroup b runs on XCD b mod 8, and on MI355X the odd XCDs read
// more slowly than the even ones when the whole GPU streams from memory (their L2s wait three
// times as long for DRAM credits; their workgroups finish a 128 KiB tile 6 us later), so the
// launch ends when the odd XCDs do.  One iteration in 32 moved from the odd to the even XCDs
// measured 0.7-1 % faster on one buffer set and on rotated ones; two or more lose again.  The two
// take alternate pieces of their region (the even one also the last two), so that the pair works
// on the same 8 KiB at a time: another 0.6 % on one buffer set and 1 % on rotated ones; wider
// groups (4, 8 or 16 workgroups interleaved, of one XCD or of neighbouring ones) lose 2-4 %.
template <int KMAX>
struct PieceOfEvenWorkgroup { // pieces 0, 2, ..., 2 KMAX - 4, then 2 KMAX - 2 and 2 KMAX - 1
    static constexpr uint32_t at(int k) { return static_cast<uint32_t>(k < KMAX - 1 ? 2 * k : KMAX - 1 + k); }
};
struct PieceOfOddWorkgroup { // pieces 1, 3, ..., 2 KMAX - 3
    static constexpr uint32_t at(int k) { return static_cast<uint32_t>(2 * k + 1); }
};
template <class Sum, int NSRC>
__global__ void __launch_bounds__(kPhasedBlock)
sum_phased_skewed_kernel(SrcTable<NSRC> src, char *out, size_t bytes, size_t tail_first, size_t numel)
{
    TCCL_STAMP(0, false);
    constexpr int KMAX = kPhasedVecs;                                   // one vector per lane per iteration
    constexpr size_t span = static_cast<size_t>(kPhasedBlock) * kVecBytes;
    constexpr size_t region = 2 * KMAX * span;
    const size_t pair_off = static_cast<size_t>(blockIdx.x >> 1) * region;
    const size_t left = bytes > pair_off ? bytes - pair_off : 0;
    const uint32_t valid = static_cast<uint32_t>(left < region ? left : region);
    char *const dst[1] = {out};
    if (blockIdx.x & 1)
        sum_tile_phased<Sum, NSRC, 1, 1, KMAX - 1, true, Sum::kPaceLoads, kAuxLoadStream, PieceOfOddWorkgroup>(
            src.p, dst, pair_off, valid, KMAX - 1);
    else
        sum_tile_phased<Sum, NSRC, 1, 1, KMAX + 1, true, Sum::kPaceLoads, kAuxLoadStream, PieceOfEvenWorkgroup<KMAX>>(
            src.p, dst, pair_off, valid, KMAX + 1);
    if (blockIdx.x == 0 && tail_first < numel) sum_tail<Sum, NSRC, 1>(src.p, dst, tail_first, numel);
}

// Would the plan for one vector per lane per iteration cut `nvec` vectors into full 128 KiB
// tiles (launch_phased_u's default rule: one or two workgroups per compute unit, fewest
// launches, smallest tile that covers a launch's share)?
static bool plans_full_tiles(size_t nvec)
{
    constexpr size_t tile = static_cast<size_t>(kPhasedBlock) * kPhasedVecs;
    size_t wgs = static_cast<size_t>(compute_units()) * 2;
    if (nvec <= (wgs / 2) * tile) wgs /= 2;
    size_t launches = (nvec + wgs * tile - 1) / (wgs * tile);
    if (launches == 0) launches = 1;
    const size_t per_launch = (nvec + launches - 1) / launches;
    return (per_launch + wgs * kPhasedBlock - 1) / (wgs * kPhasedBlock) >= kPhasedVecs;
}

// Outputs up to this size take the plan for small inputs (see launch_phased).
constexpr size_t kSmallInputBytes = static_cast<size_t>(8) << 20;

template <class Sum, int NSRC, int U>
static hipError_t launch_phased_u(const char *const *srcs, char *out, size_t numel, const tccl_launch_cfg *cfg,
                                  hipStream_t stream, bool small_input = false)
{
    constexpr size_t kmax = kPhasedVecs / U;
    constexpr size_t per_vec = kVecBytes / Sum::kElemBytes;
    constexpr size_t span = static_cast<size_t>(kPhasedBlock) * U; // vectors per iteration
    const size_t nvec = numel / per_vec;
    size_t wgs = (cfg && cfg->grid > 0) ? static_cast<size_t>(cfg->grid) : static_cast<size_t>(compute_units()) * 2;
    size_t kcount, small_tile_vec = 0;
    if (cfg && cfg->tile_iters > 0) {
        kcount = static_cast<size_t>(cfg->tile_iters) > kmax ? kmax : cfg->tile_iters;
    } else if (small_input) {
        // one launch of one or two workgroups per compute unit (two where that leaves every
        // workgroup at least a full iteration), the input cut into that many equal tiles whatever
        // its size -- every compute unit carries the same load -- and the fewest iterations
        // that cover a tile (see launch_phased)
        if (nvec < wgs * span) wgs /= 2;
        small_tile_vec = (nvec + wgs - 1) / wgs;
        kcount = (small_tile_vec + span - 1) / span;
        if (kcount < 1) kcount = 1;
        if (kcount > kmax) { // cannot happen below kSmallInputBytes; keeps the plan valid if that grows
            kcount = kmax;
            small_tile_vec = kcount * span;
        }
    } else if (NSRC <= 3 && !(cfg && cfg->grid > 0) &&
               nvec * kVecBytes >= (static_cast<size_t>(NSRC <= 2 ? 48 : 96) << 20)) {
        // With three sources or fewer a quarter or more of the traffic is writes and there
        // is little left to separate: on large inputs one launch over 16 KiB tiles beats a
        // launch per resident wave of big tiles (measured on buffers rotated so that
        // nothing is cached: +3 % with three sources, +6-8 % with one or two).
        kcount = kmax / 8 > 0 ? kmax / 8 : 1;
        wgs = (nvec + kcount * span - 1) / (kcount * span);
    } else {
        // An input that one workgroup per compute unit can cover with full-size tiles is
        // given exactly that (measured 2-9 % better than two smaller tiles per unit at
        // 16-32 MiB of output); anything larger runs two workgroups per unit.
        if (!(cfg && cfg->grid > 0) && nvec <= (wgs / 2) * span * kmax) wgs /= 2;
        // Fewest launches that fit, then the smallest tile that covers a launch's share
        // with `wgs` workgroups, so that every launch is one full, even wave of workgroups.
        size_t launches = (nvec + wgs * span * kmax - 1) / (wgs * span * kmax);
        if (launches == 0) launches = 1;
        const size_t per_launch = (nvec + launches - 1) / launches;
        kcount = (per_launch + wgs * span - 1) / (wgs * span);
        if (kcount < 1) kcount = 1;
        if (kcount > kmax) kcount = kmax;
    }
    if (wgs > (static_cast<size_t>(1) << 30)) wgs = static_cast<size_t>(1) << 30; // grid dimension limit
    const size_t tile_vec = small_tile_vec > 0 ? small_tile_vec : kcount * span;
    const size_t slice_vec = wgs * tile_vec;
    // full-size tiles of many sources, launch shape left to the library: unequal tiles for even and
    // odd XCDs (see sum_phased_skewed_kernel)
    const bool skewed = U == 1 && NSRC >= 3 && kcount == kmax && cfg == nullptr && wgs % 2 == 0;
    const size_t tail_first = nvec * per_vec;

    size_t off = 0;
    do {
        const size_t n = nvec - off < slice_vec ? nvec - off : slice_vec;
        const bool last = off + n >= nvec;
        SrcTable<NSRC> t;
        for (int i = 0; i < NSRC; ++i) t.p[i] = srcs[i] + off * kVecBytes;
        size_t grid = (n + tile_vec - 1) / tile_vec;
        if (grid == 0) grid = 1; // nothing but a ragged tail
        // the tail's element indices are relative to this launch's base pointers
        const size_t rel_first = last ? tail_first - off * per_vec : 0;
        const size_t rel_numel = last ? numel - off * per_vec : 0;
        if (skewed) {
            if constexpr (U == 1 && NSRC >= 3)
                hipLaunchKernelGGL((sum_phased_skewed_kernel<Sum, NSRC>), dim3(static_cast<unsigned>((grid + 1) / 2 * 2)),
                                   dim3(kPhasedBlock), 0, stream, t, out + off * kVecBytes, n * kVecBytes, rel_first,
                                   rel_numel);
        } else if (kcount == kmax)
            hipLaunchKernelGGL((sum_phased_kernel<Sum, NSRC, U, true>), dim3(static_cast<unsigned>(grid)),
                               dim3(kPhasedBlock), 0, stream, t, out + off * kVecBytes, n * kVecBytes,
                               static_cast<int>(kcount), tile_vec * kVecBytes, rel_first, rel_numel);
        else
            hipLaunchKernelGGL((sum_phased_kernel<Sum, NSRC, U, false>), dim3(static_cast<unsigned>(grid)),
                               dim3(kPhasedBlock), 0, stream, t, out + off * kVecBytes, n * kVecBytes,
                               static_cast<int>(kcount), tile_vec * kVecBytes, rel_first, rel_numel);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        off += n;
    } while (off < nvec);
    return hipSuccess;
}

template <class Sum, int NSRC>
static hipError_t launch_phased(const char *const *srcs, char *out, size_t numel, const tccl_launch_cfg *cfg,
                                hipStream_t stream)
{
    if (cfg && cfg->unroll == PhasedUnroll<NSRC>::alt)
        return launch_phased_u<Sum, NSRC, PhasedUnroll<NSRC>::alt>(srcs, out, numel, cfg, stream);
    if (cfg == nullptr) {
        // Up to 8 MiB of output the launch is over before the memory system has reached its steady
        // state, and what counts is how soon every byte has been asked for: one or two iterations
        // per workgroup with 16 loads of 16 bytes per lane in flight (twice the usual vectors per
        // iteration), as long as that still gives every compute unit a workgroup.  Measured on
        // buffers rotated so that nothing is cached, against the plans for larger inputs: 8 sources
        // 2 MiB -18 %, 4 MiB -12 %, 8 MiB -5 %; 4 sources -16 %, -8 %, -6 %; 2 sources 8 MiB -6 %;
        // at 16 MiB the difference is gone.  The input is cut into exactly as many equal tiles as
        // there are workgroups (a tile need not be a whole number of iterations), so sizes between the
        // powers of two do not leave half of the compute units with twice the work: 4.5 MiB 11.1 ->
        // 9.4 us, 5 MiB 11.8 -> 10.1 us.
        constexpr size_t per_vec = kVecBytes / Sum::kElemBytes;
        const size_t nvec = numel / per_vec;
        const size_t one_per_cu = static_cast<size_t>(compute_units()) * kPhasedBlock;
        if (nvec * kVecBytes <= kSmallInputBytes) {
            if (nvec >= one_per_cu * PhasedUnroll<NSRC>::alt)
                return launch_phased_u<Sum, NSRC, PhasedUnroll<NSRC>::alt>(srcs, out, numel, cfg, stream, true);
            return launch_phased_u<Sum, NSRC, PhasedUnroll<NSRC>::value>(srcs, out, numel, cfg, stream, true);
        }
    }
    if constexpr (NSRC == 3 || NSRC == 4) {
        // Three and four sources run two vectors per iteration, except where the input is cut
        // into full tiles: there the unequal, interleaved tiles of sum_phased_skewed_kernel (one
        // vector per iteration) measured 2-4 % faster on rotated buffers.
        constexpr size_t per_vec = kVecBytes / Sum::kElemBytes;
        const size_t nvec = numel / per_vec;
        const bool many_small_tiles = NSRC <= 3 && nvec * kVecBytes >= (static_cast<size_t>(96) << 20);
        if (cfg == nullptr && !many_small_tiles && plans_full_tiles(nvec))
            return launch_phased_u<Sum, NSRC, 1>(srcs, out, numel, cfg, stream);
    }
    return launch_phased_u<Sum, NSRC, PhasedUnroll<NSRC>::value>(srcs, out, numel, cfg, stream);
}

template <class Sum>
static hipError_t launch_phased_nsrc(const char *const *srcs, int nsrc, char *out, size_t numel,
                                     const tccl_launch_cfg *cfg, hipStream_t stream)
{
    switch (nsrc) {
    case 1: return launch_phased<Sum, 1>(srcs, out, numel, cfg, stream);
    case 2: return launch_phased<Sum, 2>(srcs, out, numel, cfg, stream);
    case 3: return launch_phased<Sum, 3>(srcs, out, numel, cfg, stream);
    case 4: return launch_phased<Sum, 4>(srcs, out, numel, cfg, stream);
    case 5: return launch_phased<Sum, 5>(srcs, out, numel, cfg, stream);
    case 6: return launch_phased<Sum, 6>(srcs, out, numel, cfg, stream);
    case 7: return launch_phased<Sum, 7>(srcs, out, numel, cfg, stream);
    case 8: return launch_phased<Sum, 8>(srcs, out, numel, cfg, stream);
    default: return hipErrorInvalidValue;
    }
}

// Inputs with at least this many output bytes take the phased kernel; smaller ones finish
// in a few microseconds either way (the time of a launch) and take the grid-stride kernel,
// whose launch shape adapts to tiny inputs.
static size_t phased_min_bytes(int nsrc) { return static_cast<size_t>(nsrc <= 2 ? 4 : 2) << 20; }

// Sum `nsrc` already-offset source pointers into `out`.  Shared by the three entry points.
int sum_streams(const void *const *srcs, int nsrc, void *out, size_t numel, int dtype, hipStream_t stream,
                const tccl_launch_cfg *cfg)
{
    const int esize = dtype_size(dtype);
    if (esize == 0 || nsrc < 1 || nsrc > TCCL_MAX_WORLD || srcs == nullptr || out == nullptr) return TCCL_EINVAL;
    for (int i = 0; i < nsrc; ++i) {
        if (srcs[i] == nullptr) return TCCL_EINVAL;
        if (!aligned16(srcs[i])) return TCCL_EALIGN;
    }
    if (!aligned16(out)) return TCCL_EALIGN;
    if (numel == 0) return TCCL_OK;
    // a configuration that overrides nothing is no configuration: the library's own plans apply
    if (cfg && cfg->block == 0 && cfg->unroll == 0 && cfg->grid == 0 && cfg->tile_iters == 0 && cfg->flags == 0)
        cfg = nullptr;

    const size_t nvec = numel * static_cast<size_t>(esize) / kVecBytes;
    const char *const *s = reinterpret_cast<const char *const *>(srcs);
    const int flags = cfg ? cfg->flags : 0;
    const bool phased = (flags & TCCL_CFG_PHASED) ||
                        (!(flags & TCCL_CFG_STREAMING) && nvec * kVecBytes >= phased_min_bytes(nsrc));
    if (phased) {
        hipError_t pe = (dtype == TCCL_BF16)
                            ? launch_phased_nsrc<Bf16Sum>(s, nsrc, static_cast<char *>(out), numel, cfg, stream)
                            : launch_phased_nsrc<F32Sum>(s, nsrc, static_cast<char *>(out), numel, cfg, stream);
        return hip_code(pe);
    }
    const Shape sh = resolve_shape(cfg, nvec, nsrc, 1);
    hipError_t e = (dtype == TCCL_BF16) ? launch_sum_nsrc<Bf16Sum>(s, nsrc, static_cast<char *>(out), numel, sh, stream)
                                        : launch_sum_nsrc<F32Sum>(s, nsrc, static_cast<char *>(out), numel, sh, stream);
    return hip_code(e);
}

} // namespace tccl

using namespace tccl;

extern "C" int tccl_all_reduce_sum_ex(const void *const *bufs, int world, void *out, size_t numel, int dtype,
                                      void *stream, const tccl_launch_cfg *cfg)
{
    return sum_streams(bufs, world, out, numel, dtype, static_cast<hipStream_t>(stream), cfg);
}

extern "C" int tccl_all_reduce_sum(const void *const *bufs, int world, void *out, size_t numel, int dtype,
                                   void *stream)
{
    return tccl_all_reduce_sum_ex(bufs, world, out, numel, dtype, stream, nullptr);
}

extern "C" int tccl_reduce_scatter_sum_ex(const void *const *bufs, int world, int rank, void *out,
                                          size_t numel_total, int dtype, void *stream, const tccl_launch_cfg *cfg)
{
    const int esize = dtype_size(dtype);
    if (esize == 0 || bufs == nullptr || world < 1 || world > TCCL_MAX_WORLD || rank < 0 || rank >= world)
        return TCCL_EINVAL;
    // Every rank's share must be the same whole number of 16-byte vectors (the reference asserts
    // numel % (8 * world) == 0, triton_reduce_scatter.py:101-104): the answer is the same for
    // every rank, and no element is left out.
    if (numel_total % static_cast<size_t>(world) != 0) return TCCL_EALIGN;
    const size_t per_rank = numel_total / static_cast<size_t>(world);
    if ((per_rank * static_cast<size_t>(esize)) % kVecBytes != 0) return TCCL_EALIGN;
    const size_t byte_off = static_cast<size_t>(rank) * per_rank * static_cast<size_t>(esize);
    const void *shifted[TCCL_MAX_WORLD];
    for (int i = 0; i < world; ++i) {
        if (bufs[i] == nullptr) return TCCL_EINVAL;
        shifted[i] = static_cast<const char *>(bufs[i]) + byte_off;
    }
    return sum_streams(shifted, world, out, per_rank, dtype, static_cast<hipStream_t>(stream), cfg);
}

extern "C" int tccl_reduce_scatter_sum(const void *const *bufs, int world, int rank, void *out, size_t numel_total,
                                       int dtype, void *stream)
{
    return tccl_reduce_scatter_sum_ex(bufs, world, rank, out, numel_total, dtype, stream, nullptr);
}

extern "C" int tccl_tree_reduce_step(const void *own, const void *child0, const void *child1, void *dst,
                                     size_t numel, int dtype, void *stream)
{
    if (own == nullptr || dst == nullptr) return TCCL_EINVAL;
    const void *srcs[3];
    int n = 0;
    if (child0) srcs[n++] = child0;
    if (child1) srcs[n++] = child1;
    srcs[n++] = own;
    return sum_streams(srcs, n, dst, numel, dtype, static_cast<hipStream_t>(stream), nullptr);
}
