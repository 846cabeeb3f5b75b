// gather.hip -- all-gather pack copy and the single tree copy step.  Typeless 16-byte
// vector copies, bit-exact for every dtype.
#include "host.h"
#include "vec.h"

namespace tccl {

struct RowTable {
    const char *p[TCCL_MAX_WORLD];
};

// Row i is written at out + i * row_bytes (the [world, numel] layout of
// triton_all_gather.py:82).  The reference runs the rank loop innermost
// (triton_all_gather.py:54-62), so one workgroup feeds `world` far-apart store streams at
// once; here the grid walks the rows one after the other.
template <int UNROLL, bool NTL, bool NTS>
__global__ void __launch_bounds__(kMaxBlock)
pack_kernel(RowTable rows, int world, char *out, size_t row_vecs, int tile_iters, int xcd_contiguous)
{
    TCCL_STAMP(0, false);
    pack_rows<UNROLL, NTL, NTS>(rows.p, world, out, row_vecs, tile_iters, xcd_contiguous != 0);
    TCCL_STAMP(3, true);
}

template <int NDST, int UNROLL, bool NTL, bool NTS>
__global__ void __launch_bounds__(kMaxBlock)
copy_kernel(const char *src, char *dst0, char *dst1, size_t nvec, int tile_iters, int xcd_contiguous)
{
    TCCL_STAMP(0, false);
    if constexpr (NDST == 2) {
        char *const dst[2] = {dst0, dst1};
        copy_range<2, UNROLL, NTL, NTS>(src, dst, nvec, tile_iters, xcd_contiguous != 0);
    } else {
        char *const dst[1] = {dst0};
        copy_range<1, UNROLL, NTL, NTS>(src, dst, nvec, tile_iters, xcd_contiguous != 0);
    }
    TCCL_STAMP(3, true);
}

template <int UNROLL, bool NTL, bool NTS>
static hipError_t launch_pack(const RowTable &rows, int world, char *out, size_t row_vecs, const Shape &sh,
                              hipStream_t stream)
{
    hipLaunchKernelGGL((pack_kernel<UNROLL, NTL, NTS>), dim3(sh.grid), dim3(sh.block), 0, stream, rows, world, out,
                       row_vecs, sh.tile_iters, sh.xcd_contiguous ? 1 : 0);
    return hipGetLastError();
}

template <int UNROLL>
static hipError_t launch_pack_nt(const RowTable &rows, int world, char *out, size_t row_vecs, const Shape &sh,
                                 hipStream_t stream)
{
    if (sh.nt_load) {
        if (sh.nt_store) return launch_pack<UNROLL, true, true>(rows, world, out, row_vecs, sh, stream);
        return launch_pack<UNROLL, true, false>(rows, world, out, row_vecs, sh, stream);
    }
    if (sh.nt_store) return launch_pack<UNROLL, false, true>(rows, world, out, row_vecs, sh, stream);
    return launch_pack<UNROLL, false, false>(rows, world, out, row_vecs, sh, stream);
}

template <int NDST, int UNROLL>
static hipError_t launch_copy_nt(const char *src, char *d0, char *d1, size_t nvec, const Shape &sh,
                                 hipStream_t stream)
{
    const int xc = sh.xcd_contiguous ? 1 : 0;
    if (sh.nt_load && sh.nt_store)
        hipLaunchKernelGGL((copy_kernel<NDST, UNROLL, true, true>), dim3(sh.grid), dim3(sh.block), 0, stream, src, d0,
                           d1, nvec, sh.tile_iters, xc);
    else if (sh.nt_load)
        hipLaunchKernelGGL((copy_kernel<NDST, UNROLL, true, false>), dim3(sh.grid), dim3(sh.block), 0, stream, src, d0,
                           d1, nvec, sh.tile_iters, xc);
    else if (sh.nt_store)
        hipLaunchKernelGGL((copy_kernel<NDST, UNROLL, false, true>), dim3(sh.grid), dim3(sh.block), 0, stream, src, d0,
                           d1, nvec, sh.tile_iters, xc);
    else
        hipLaunchKernelGGL((copy_kernel<NDST, UNROLL, false, false>), dim3(sh.grid), dim3(sh.block), 0, stream, src,
                           d0, d1, nvec, sh.tile_iters, xc);
    return hipGetLastError();
}

template <int NDST>
static hipError_t launch_copy_unroll(const char *src, char *d0, char *d1, size_t nvec, const Shape &sh,
                                     hipStream_t stream)
{
    switch (sh.unroll) {
    case 1: return launch_copy_nt<NDST, 1>(src, d0, d1, nvec, sh, stream);
    case 2: return launch_copy_nt<NDST, 2>(src, d0, d1, nvec, sh, stream);
    default: return launch_copy_nt<NDST, 4>(src, d0, d1, nvec, sh, stream);
    }
}

} // namespace tccl

using namespace tccl;

extern "C" int tccl_all_gather_ex(const void *const *bufs, int world, void *out, size_t bytes_per_rank, void *stream,
                                  const tccl_launch_cfg *cfg)
{
    if (bufs == nullptr || out == nullptr || world < 1 || world > TCCL_MAX_WORLD) return TCCL_EINVAL;
    if (bytes_per_rank % kVecBytes != 0 || !aligned16(out)) return TCCL_EALIGN;
    RowTable rows = {};
    for (int i = 0; i < world; ++i) {
        if (bufs[i] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[i])) return TCCL_EALIGN;
        rows.p[i] = static_cast<const char *>(bufs[i]);
    }
    if (bytes_per_rank == 0) return TCCL_OK;
    const size_t row_vecs = bytes_per_rank / kVecBytes;
    const Shape sh = resolve_shape(cfg, row_vecs, 1, world, true);
    hipStream_t s = static_cast<hipStream_t>(stream);
    char *o = static_cast<char *>(out);
    hipError_t e;
    switch (sh.unroll) {
    case 1: e = launch_pack_nt<1>(rows, world, o, row_vecs, sh, s); break;
    case 2: e = launch_pack_nt<2>(rows, world, o, row_vecs, sh, s); break;
    default: e = launch_pack_nt<4>(rows, world, o, row_vecs, sh, s); break;
    }
    return hip_code(e);
}

extern "C" int tccl_all_gather(const void *const *bufs, int world, void *out, size_t bytes_per_rank, void *stream)
{
    return tccl_all_gather_ex(bufs, world, out, bytes_per_rank, stream, nullptr);
}

extern "C" int tccl_tree_copy_step(const void *src, void *dst0, void *dst1, size_t bytes, void *stream)
{
    if (src == nullptr || dst0 == nullptr) return TCCL_EINVAL;
    if (bytes % kVecBytes != 0 || !aligned16(src) || !aligned16(dst0) || !aligned16(dst1)) return TCCL_EALIGN;
    if (bytes == 0) return TCCL_OK;
    const size_t nvec = bytes / kVecBytes;
    const Shape sh = resolve_shape(nullptr, nvec, 1, 1, true);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const char *in = static_cast<const char *>(src);
    hipError_t e = dst1 ? launch_copy_unroll<2>(in, static_cast<char *>(dst0), static_cast<char *>(dst1), nvec, sh, s)
                        : launch_copy_unroll<1>(in, static_cast<char *>(dst0), nullptr, nvec, sh, s);
    return hip_code(e);
}
