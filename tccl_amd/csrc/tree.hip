// tree.hip -- the double binary tree: a batch of node steps per launch, and the schedule
// that runs the whole collective for all virtual ranks as one launch per tree level.
#include <new>
#include <vector>

#include "host.h"
#include "vec.h"

namespace tccl {

struct JobTable {
    tccl_node_job job[TCCL_MAX_JOBS];
};

// One node step over its element range.  blockIdx.y selects the job; workgroup x of a job
// takes tile x, x + gridDim.x, ...  A tile is a 32 KiB piece of a pipelining chunk (the
// whole chunk when chunks are smaller): its sources are read and reduced into registers,
// then the result is written, the way one message of the tree pipeline would be received,
// reduced and forwarded.  32 KiB is the measured optimum for steps with one to three
// sources (a 128 MiB two-child step: 77 us with 32 KiB tiles, 87 us with 128 KiB tiles);
// the tiles of one chunk are neighbours in the grid, so a chunk still completes as a unit.
constexpr int kLevelU = 2;
constexpr int kLevelKMax = 4;

template <class Sum, int NDST, bool FULL>
__device__ __forceinline__ void run_tile(const tccl_node_job &j, char *const (&dst)[NDST], size_t off, uint32_t valid,
                                         int kcount)
{
    const char *c0 = static_cast<const char *>(j.src[0]);
    const char *c1 = static_cast<const char *>(j.src[1]);
    const char *own = static_cast<const char *>(j.src[2]);
    if (j.is_copy) {
        copy_tile_phased<NDST, kLevelU, kLevelKMax>(c0, dst, off, valid, kcount);
    } else if (c0 != nullptr && c1 != nullptr) {
        const char *const src[3] = {c0, c1, own};
        sum_tile_phased<Sum, 3, NDST, kLevelU, kLevelKMax, FULL>(src, dst, off, valid, kcount);
    } else if (c0 != nullptr || c1 != nullptr) {
        const char *const src[2] = {c0 != nullptr ? c0 : c1, own};
        sum_tile_phased<Sum, 2, NDST, kLevelU, kLevelKMax, FULL>(src, dst, off, valid, kcount);
    } else {
        const char *const src[1] = {own};
        sum_tile_phased<Sum, 1, NDST, kLevelU, kLevelKMax, FULL>(src, dst, off, valid, kcount);
    }
}

template <class Sum, int NDST>
__device__ __forceinline__ void run_tail(const tccl_node_job &j, char *const (&dst)[NDST], size_t first)
{
    const char *c0 = static_cast<const char *>(j.src[0]);
    const char *c1 = static_cast<const char *>(j.src[1]);
    const char *own = static_cast<const char *>(j.src[2]);
    if (c0 != nullptr && c1 != nullptr) {
        const char *const src[3] = {c0, c1, own};
        sum_tail<Sum, 3, NDST>(src, dst, first, j.numel);
    } else if (c0 != nullptr || c1 != nullptr) {
        const char *const src[2] = {c0 != nullptr ? c0 : c1, own};
        sum_tail<Sum, 2, NDST>(src, dst, first, j.numel);
    } else {
        const char *const src[1] = {own};
        sum_tail<Sum, 1, NDST>(src, dst, first, j.numel);
    }
}

template <class Sum, int NDST, bool FULL>
__device__ __forceinline__ void run_job(const tccl_node_job &j, int kcount)
{
    char *dst[NDST];
#pragma unroll
    for (int d = 0; d < NDST; ++d) dst[d] = static_cast<char *>(j.dst[d]);
    char *const(&cdst)[NDST] = dst;
    constexpr size_t per_vec = kVecBytes / Sum::kElemBytes;
    const size_t bytes = j.numel / per_vec * kVecBytes;
    const size_t tile_bytes = static_cast<size_t>(kcount) * (kPhasedBlock * kLevelU * kVecBytes);
    for (size_t off = blockIdx.x * tile_bytes; off < bytes; off += gridDim.x * tile_bytes) {
        const size_t left = bytes - off;
        run_tile<Sum, NDST, FULL>(j, cdst, off, static_cast<uint32_t>(left < tile_bytes ? left : tile_bytes), kcount);
    }
    // ragged tail of a reduce step (copy steps are whole vectors)
    if (blockIdx.x == 0 && !j.is_copy && j.numel % per_vec != 0) run_tail<Sum, NDST>(j, cdst, j.numel / per_vec * per_vec);
}

template <class Sum, bool FULL>
__global__ void __launch_bounds__(kPhasedBlock) tree_level_kernel(JobTable jobs, int kcount)
{
    TCCL_STAMP(0, false);
    const tccl_node_job &j = jobs.job[blockIdx.y];
    if (j.dst[1] != nullptr)
        run_job<Sum, 2, FULL>(j, kcount);
    else
        run_job<Sum, 1, FULL>(j, kcount);
}

// A level made of copy steps only (every level of the down-sweep): the jobs are walked one
// after the other by a small persistent grid, 16 KiB per workgroup per step, loads and
// stores streaming.  The whole GPU then works on one source window and its destination
// windows at a time; for copies that beats read-then-write tiles by 5-6 % and running the
// jobs side by side by more.
constexpr int kCopyU = 4;

__global__ void __launch_bounds__(kPhasedBlock) tree_copy_level_kernel(JobTable jobs, int njobs, int esize)
{
    TCCL_STAMP(0, false);
    constexpr size_t span_bytes = static_cast<size_t>(kPhasedBlock) * kCopyU * kVecBytes;
    size_t spans[TCCL_MAX_JOBS];
    size_t total = 0;
#pragma unroll
    for (int i = 0; i < TCCL_MAX_JOBS; ++i) {
        spans[i] = i < njobs ? (jobs.job[i].numel * esize + span_bytes - 1) / span_bytes : 0;
        total += spans[i];
    }
    const uint32_t lane_off = threadIdx.x * kVecBytes;
    for (size_t g = blockIdx.x; g < total; g += gridDim.x) {
        int ji = 0;
        size_t local = g;
#pragma unroll
        for (int i = 0; i < TCCL_MAX_JOBS - 1; ++i) {
            if (ji == i && local >= spans[i]) {
                local -= spans[i];
                ji = i + 1;
            }
        }
        const tccl_node_job &j = jobs.job[ji];
        const size_t bytes = j.numel * esize;
        const size_t off = local * span_bytes;
        const size_t left = bytes - off;
        const uint32_t valid = static_cast<uint32_t>(left < span_bytes ? left : span_bytes);
        const __amdgpu_buffer_rsrc_t rs = tile_rsrc(static_cast<const char *>(j.src[0]) + off, valid);
        u32x4 v[kCopyU];
#pragma unroll
        for (int u = 0; u < kCopyU; ++u)
            v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, u * (kPhasedBlock * kVecBytes) + lane_off, 0, kAuxLoadStream);
        const __amdgpu_buffer_rsrc_t r0 = tile_rsrc(static_cast<char *>(j.dst[0]) + off, valid);
#pragma unroll
        for (int u = 0; u < kCopyU; ++u)
            __builtin_amdgcn_raw_buffer_store_b128(v[u], r0, u * (kPhasedBlock * kVecBytes) + lane_off, 0, kAuxStoreNt);
        if (j.dst[1] != nullptr) {
            const __amdgpu_buffer_rsrc_t r1 = tile_rsrc(static_cast<char *>(j.dst[1]) + off, valid);
#pragma unroll
            for (int u = 0; u < kCopyU; ++u)
                __builtin_amdgcn_raw_buffer_store_b128(v[u], r1, u * (kPhasedBlock * kVecBytes) + lane_off, 0,
                                                       kAuxStoreNt);
        }
    }
    TCCL_STAMP(3, true);
}

int launch_level(const tccl_node_job *jobs, int njobs, int dtype, size_t chunk_elems, hipStream_t stream)
{
    const int esize = dtype_size(dtype);
    if (esize == 0 || jobs == nullptr || njobs < 0 || njobs > TCCL_MAX_JOBS) return TCCL_EINVAL;
    if (njobs == 0) return TCCL_OK;
    const size_t per_vec = kVecBytes / esize;
    if (chunk_elems == 0) chunk_elems = (128u * 1024u) / esize;
    const size_t span = static_cast<size_t>(kPhasedBlock) * kLevelU; // vectors per iteration
    size_t kcount = (chunk_elems / per_vec + span - 1) / span;
    if (kcount < 1) kcount = 1;
    if (kcount > kLevelKMax) kcount = kLevelKMax; // larger chunks are walked in 32 KiB tiles

    JobTable t = {};
    size_t max_tiles = 0;
    bool all_copies = true;
    size_t copy_spans = 0;
    for (int i = 0; i < njobs; ++i) {
        const tccl_node_job &j = jobs[i];
        if (j.dst[0] == nullptr) return TCCL_EINVAL;
        if (j.is_copy ? (j.src[0] == nullptr) : (j.src[2] == nullptr)) return TCCL_EINVAL;
        for (int k = 0; k < 3; ++k)
            if (!aligned16(j.src[k])) return TCCL_EALIGN;
        if (!aligned16(j.dst[0]) || !aligned16(j.dst[1])) return TCCL_EALIGN;
        if (j.is_copy && (j.numel % per_vec) != 0) return TCCL_EALIGN;
        t.job[i] = j;
        all_copies = all_copies && j.is_copy;
        copy_spans += (j.numel * esize + kPhasedBlock * kCopyU * kVecBytes - 1) / (kPhasedBlock * kCopyU * kVecBytes);
        const size_t nvec = j.numel / per_vec;
        const size_t tiles = (nvec + span * kcount - 1) / (span * kcount);
        if (tiles > max_tiles) max_tiles = tiles;
    }
    if (all_copies) {
        if (copy_spans == 0) return TCCL_OK;
        size_t wgs = static_cast<size_t>(compute_units());
        if (wgs > copy_spans) wgs = copy_spans;
        hipLaunchKernelGGL(tree_copy_level_kernel, dim3(static_cast<unsigned>(wgs)), dim3(kPhasedBlock), 0, stream, t,
                           njobs, esize);
        return hip_code(hipGetLastError());
    }
    if (max_tiles == 0) max_tiles = 1; // ragged tails only
    if (max_tiles > 0x7FFFFFFFu) max_tiles = 0x7FFFFFFFu;
    const dim3 grid(static_cast<unsigned>(max_tiles), njobs);
    const int kc = static_cast<int>(kcount);
    const bool full = kcount == static_cast<size_t>(kLevelKMax);
    if (dtype == TCCL_BF16) {
        if (full)
            hipLaunchKernelGGL((tree_level_kernel<Bf16Sum, true>), grid, dim3(kPhasedBlock), 0, stream, t, kc);
        else
            hipLaunchKernelGGL((tree_level_kernel<Bf16Sum, false>), grid, dim3(kPhasedBlock), 0, stream, t, kc);
    } else {
        if (full)
            hipLaunchKernelGGL((tree_level_kernel<F32Sum, true>), grid, dim3(kPhasedBlock), 0, stream, t, kc);
        else
            hipLaunchKernelGGL((tree_level_kernel<F32Sum, false>), grid, dim3(kPhasedBlock), 0, stream, t, kc);
    }
    return hip_code(hipGetLastError());
}

} // namespace tccl

using namespace tccl;

extern "C" int tccl_tree_level(const tccl_node_job *jobs, int njobs, int dtype, size_t chunk_elems, void *stream)
{
    return launch_level(jobs, njobs, dtype, chunk_elems, static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------------ tree index math
// Closed form of the heap-ordered array that tree.py:5-31 builds row by row: position
// idx >= 1 sits on level L = floor(log2 idx) at column c = idx - 2^L, and holds the
// in-order label (2c + 1) * world / 2^(L+1); position 0 holds the extra node 0.

static bool pow2_world(int world) { return world >= 2 && world <= TCCL_MAX_TREE_WORLD && (world & (world - 1)) == 0; }

extern "C" int tccl_double_tree_arrays(int world, int *tree_a, int *tree_b)
{
    if (!pow2_world(world)) return TCCL_EPOW2;
    if (tree_a == nullptr || tree_b == nullptr) return TCCL_EINVAL;
    tree_a[0] = 0;
    for (int level_first = 1; level_first < world; level_first *= 2)
        for (int c = 0; c < level_first; ++c)
            tree_a[level_first + c] = (2 * c + 1) * (world / (2 * level_first));
    // tree.py:83-91: the second tree is the first with every label lowered by one, the
    // subroot wrapping round to world-1.
    for (int i = 0; i < world; ++i) tree_b[i] = (tree_a[i] + world - 1) % world;
    return TCCL_OK;
}

// Neighbours of `r` in tree a without building the array (tree.py:130-146 looks the rank
// up in the array).  For r >= 1 let t = number of trailing zero bits: the node sits t
// levels above the leaves, its children are r -/+ 2^(t-1), and its parent is r - 2^t when
// bit t+1 of r is set, r + 2^t otherwise; the top interior node world/2 hangs under the
// extra node 0, whose single child it is (tree.py:133-136).
static void tree_a_neighbours(int world, int r, int *out3)
{
    if (r == 0) {
        out3[0] = -1;
        out3[1] = world / 2;
        out3[2] = -1;
        return;
    }
    const int low = r & -r;
    if (r == world / 2)
        out3[0] = 0;
    else
        out3[0] = (r & (low << 1)) ? r - low : r + low;
    if (low == 1) {
        out3[1] = -1;
        out3[2] = -1;
    } else {
        out3[1] = r - low / 2;
        out3[2] = r + low / 2;
    }
}

extern "C" int tccl_double_tree_indices(int world, int rank, int *out6)
{
    if (!pow2_world(world)) return TCCL_EPOW2;
    if (out6 == nullptr || rank < 0 || rank >= world) return TCCL_EINVAL;
    tree_a_neighbours(world, rank, out6);
    // Rank r plays in tree b the part that rank r+1 (mod world) plays in tree a; its
    // neighbours are that node's neighbours lowered by one, mod world.  -1 stays -1.
    tree_a_neighbours(world, (rank + 1) % world, out6 + 3);
    for (int k = 3; k < 6; ++k)
        if (out6[k] >= 0) out6[k] = (out6[k] + world - 1) % world;
    return TCCL_OK;
}

extern "C" size_t tccl_double_tree_split(size_t numel, size_t esize)
{
    if (esize == 0 || esize > kVecBytes) return 0;
    const size_t per_vec = kVecBytes / esize;
    return (numel / 2) / per_vec * per_vec;
}

// ------------------------------------------------------------------ the whole collective
// Levels of one tree, by height above the leaves: a rank r >= 1 of tree a is at height
// ctz(r); the extra node 0 sits above the top interior node.  The up-sweep runs heights
// 1 .. log2(world)-1 and then the extra node; leaves run no step of their own: their step
// is "own <- 0 + own", which changes nothing a parent can see (the parent's accumulator
// also starts at +0) and nothing the caller can see (the down-sweep overwrites the leaf's
// buffer).  The down-sweep runs the same levels top to bottom, every rank pulling from its
// parent.

extern "C" int tccl_double_tree_all_reduce(void *const *bufs, void *const *outs, int world, size_t numel, int dtype,
                                           size_t chunk_elems, void *stream)
{
    const int esize = dtype_size(dtype);
    if (esize == 0 || bufs == nullptr) return TCCL_EINVAL;
    if (!pow2_world(world)) return TCCL_EPOW2;
    if (world > TCCL_MAX_TREE_RANKS) return TCCL_EINVAL;
    for (int r = 0; r < world; ++r) {
        if (bufs[r] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[r]) || (outs && !aligned16(outs[r]))) return TCCL_EALIGN;
    }
    const size_t per_vec = kVecBytes / esize;
    if (numel % per_vec != 0) return TCCL_EALIGN;
    if (numel == 0) return TCCL_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);

    const size_t split = tccl_double_tree_split(numel, esize);
    const size_t lo[2] = {0, split};
    const size_t len[2] = {split, numel - split};

    int height = 0;
    while ((1 << height) < world) ++height;

    // node_height[tree][rank]: 0 = leaf, 1..height-1 = interior, height = the extra node.
    int nbr[2][TCCL_MAX_TREE_RANKS][3];
    int node_height[2][TCCL_MAX_TREE_RANKS];
    for (int r = 0; r < world; ++r) {
        int six[6];
        int rc = tccl_double_tree_indices(world, r, six);
        if (rc != TCCL_OK) return rc;
        for (int t = 0; t < 2; ++t) {
            for (int k = 0; k < 3; ++k) nbr[t][r][k] = six[3 * t + k];
            const int ra = (t == 0) ? r : (r + 1) % world;
            node_height[t][r] = (ra == 0) ? height : __builtin_ctz(ra);
        }
    }

    auto at = [&](int rank, int tree) { return static_cast<char *>(bufs[rank]) + lo[tree] * esize; };
    auto out_at = [&](int rank, int tree) -> char * {
        return (outs && outs[rank]) ? static_cast<char *>(outs[rank]) + lo[tree] * esize : nullptr;
    };

    std::vector<tccl_node_job> batch;
    auto flush = [&]() -> int {
        for (size_t i = 0; i < batch.size(); i += TCCL_MAX_JOBS) {
            const int n = static_cast<int>(batch.size() - i < TCCL_MAX_JOBS ? batch.size() - i : TCCL_MAX_JOBS);
            int rc = launch_level(batch.data() + i, n, dtype, chunk_elems, s);
            if (rc != TCCL_OK) return rc;
        }
        batch.clear();
        return TCCL_OK;
    };

    // Up-sweep.
    for (int h = 1; h <= height; ++h) {
        for (int t = 0; t < 2; ++t) {
            if (len[t] == 0) continue;
            for (int r = 0; r < world; ++r) {
                if (node_height[t][r] != h) continue;
                tccl_node_job j = {};
                const int c0 = nbr[t][r][1], c1 = nbr[t][r][2];
                j.src[0] = c0 >= 0 ? at(c0, t) : nullptr;
                j.src[1] = c1 >= 0 ? at(c1, t) : nullptr;
                j.src[2] = at(r, t);
                j.dst[0] = at(r, t);
                // the extra node's step produces the final result: it goes to that rank's
                // output in the same pass (the result is also what its buffer keeps)
                j.dst[1] = (h == height) ? out_at(r, t) : nullptr;
                j.numel = len[t];
                j.is_copy = 0;
                batch.push_back(j);
            }
        }
        int rc = flush();
        if (rc != TCCL_OK) return rc;
    }

    // Down-sweep: the extra node already holds the result (and has written its output);
    // every other rank copies its parent's buffer into its own buffer and its output.
    for (int h = height - 1; h >= 0; --h) {
        for (int t = 0; t < 2; ++t) {
            if (len[t] == 0) continue;
            for (int r = 0; r < world; ++r) {
                if (node_height[t][r] != h) continue;
                tccl_node_job j = {};
                j.is_copy = 1;
                j.numel = len[t];
                j.src[0] = at(nbr[t][r][0], t);
                j.dst[0] = at(r, t);
                j.dst[1] = out_at(r, t);
                batch.push_back(j);
            }
        }
        int rc = flush();
        if (rc != TCCL_OK) return rc;
    }
    return TCCL_OK;
}

// ------------------------------------------------------------------ the whole tree in one launch
namespace tccl {

// Labels are ranks of tree a; tree b is tree a with every label lowered by one (mod W), so
// the lane handling a vector of the second half simply loads label l from rank (l-1) mod W.

// Result of the subtree rooted at interior-or-leaf label R (R >= 1), LOW = lowest set bit of
// R: round(0 + node(R - LOW/2) + node(R + LOW/2) + x[R]); a leaf (LOW == 1) is
// round(0 + x[R]) -- the step every rank runs on its own buffer.
template <class Sum, int W, int R, int LOW>
__device__ __forceinline__ u32x4 subtree(const u32x4 (&x)[W])
{
    Sum acc;
    acc.zero();
    if constexpr (LOW > 1) {
        acc.add(subtree<Sum, W, R - LOW / 2, LOW / 2>(x));
        acc.add(subtree<Sum, W, R + LOW / 2, LOW / 2>(x));
    }
    acc.add(x[R]);
    return acc.result();
}

// The extra node 0 on top: round(0 + node(W/2) + x[0]).
template <class Sum, int W>
__device__ __forceinline__ u32x4 whole_tree(const u32x4 (&x)[W])
{
    Sum acc;
    acc.zero();
    acc.add(subtree<Sum, W, W / 2, W / 2>(x));
    acc.add(x[0]);
    return acc.result();
}

template <int W>
struct TreePtrs {
    char *buf[W];
    char *out[W]; // entries may be null
};

// Vectors [begin, end) of one half; SHIFT = 0 for tree a, W-1 for tree b (label l lives in
// rank (l + SHIFT) mod W), a compile-time constant so that every pointer stays in SGPRs.
template <class Sum, int W, int SHIFT, bool NT>
__device__ __forceinline__ void fused_half(const TreePtrs<W> &p, size_t begin, size_t end)
{
    const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
    for (size_t i = begin + static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < end; i += stride) {
        u32x4 x[W];
#pragma unroll
        for (int l = 0; l < W; ++l) x[l] = load_vec<NT>(p.buf[(l + SHIFT) % W], i);
        const u32x4 s = whole_tree<Sum, W>(x);
#pragma unroll
        for (int r = 0; r < W; ++r) store_vec<NT>(p.buf[r], i, s);
#pragma unroll
        for (int r = 0; r < W; ++r)
            if (p.out[r] != nullptr) store_vec<NT>(p.out[r], i, s);
    }
}

// NT = streaming loads and stores, for inputs too large to stay in the caches.
template <class Sum, int W, bool NT>
__global__ void __launch_bounds__(kPhasedBlock) tree_fused_kernel(TreePtrs<W> p, size_t nvec, size_t split_vec)
{
    fused_half<Sum, W, 0, NT>(p, 0, split_vec);
    fused_half<Sum, W, W - 1, NT>(p, split_vec, nvec);
}

template <class Sum, int W>
static hipError_t launch_fused(void *const *bufs, void *const *outs, size_t nvec, size_t split_vec, hipStream_t stream)
{
    TreePtrs<W> p;
    for (int r = 0; r < W; ++r) {
        p.buf[r] = static_cast<char *>(bufs[r]);
        p.out[r] = outs ? static_cast<char *>(outs[r]) : nullptr;
    }
    // Small inputs: every lane its own vector, cached accesses.  Large inputs (beyond the caches):
    // one workgroup per compute unit walking the range, streaming accesses -- the shape that
    // measured best for write-heavy streams on this GPU.
    const bool big = nvec * kVecBytes * W >= (static_cast<size_t>(256) << 20);
    size_t grid = (nvec + kPhasedBlock - 1) / kPhasedBlock;
    const size_t cap = static_cast<size_t>(compute_units()) * (big ? 1 : 8);
    if (grid > cap) grid = cap;
    if (grid == 0) grid = 1;
    if (big)
        hipLaunchKernelGGL((tree_fused_kernel<Sum, W, true>), dim3(static_cast<unsigned>(grid)), dim3(kPhasedBlock), 0,
                           stream, p, nvec, split_vec);
    else
        hipLaunchKernelGGL((tree_fused_kernel<Sum, W, false>), dim3(static_cast<unsigned>(grid)), dim3(kPhasedBlock), 0,
                           stream, p, nvec, split_vec);
    return hipGetLastError();
}

template <class Sum>
static hipError_t launch_fused_world(void *const *bufs, void *const *outs, int world, size_t nvec, size_t split_vec,
                                     hipStream_t stream)
{
    switch (world) {
    case 2: return launch_fused<Sum, 2>(bufs, outs, nvec, split_vec, stream);
    case 4: return launch_fused<Sum, 4>(bufs, outs, nvec, split_vec, stream);
    case 8: return launch_fused<Sum, 8>(bufs, outs, nvec, split_vec, stream);
    default: return hipErrorInvalidValue;
    }
}

} // namespace tccl

extern "C" int tccl_double_tree_all_reduce_fused(void *const *bufs, void *const *outs, int world, size_t numel,
                                                 int dtype, void *stream)
{
    const int esize = dtype_size(dtype);
    if (esize == 0 || bufs == nullptr) return TCCL_EINVAL;
    if (!pow2_world(world)) return TCCL_EPOW2;
    if (world > 8) return TCCL_EINVAL;
    for (int r = 0; r < world; ++r) {
        if (bufs[r] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[r]) || (outs && !aligned16(outs[r]))) return TCCL_EALIGN;
    }
    const size_t per_vec = kVecBytes / esize;
    if (numel % per_vec != 0) return TCCL_EALIGN;
    if (numel == 0) return TCCL_OK;
    const size_t nvec = numel / per_vec;
    const size_t split_vec = tccl_double_tree_split(numel, esize) / per_vec;
    hipStream_t s = static_cast<hipStream_t>(stream);
    hipError_t e = (dtype == TCCL_BF16) ? launch_fused_world<Bf16Sum>(bufs, outs, world, nvec, split_vec, s)
                                        : launch_fused_world<F32Sum>(bufs, outs, world, nvec, split_vec, s);
    return hip_code(e);
}

// ------------------------------------------------------------------ recorded plans

struct tccl_plan {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
};

extern "C" int tccl_double_tree_plan_create(void *const *bufs, void *const *outs, int world, size_t numel, int dtype,
                                            size_t chunk_elems, tccl_plan **plan_out)
{
    if (plan_out == nullptr) return TCCL_EINVAL;
    *plan_out = nullptr;
    (void)compute_units(); // device query now, not while a stream is being captured
    hipStream_t cap = nullptr;
    hipError_t e = hipStreamCreateWithFlags(&cap, hipStreamNonBlocking);
    if (e != hipSuccess) return hip_code(e);
    e = hipStreamBeginCapture(cap, hipStreamCaptureModeRelaxed);
    if (e != hipSuccess) {
        (void)hipStreamDestroy(cap);
        return hip_code(e);
    }
    const int rc = tccl_double_tree_all_reduce(bufs, outs, world, numel, dtype, chunk_elems, cap);
    hipGraph_t graph = nullptr;
    e = hipStreamEndCapture(cap, &graph); // always end the capture, also after an argument error
    (void)hipStreamDestroy(cap);
    if (rc != TCCL_OK || e != hipSuccess || graph == nullptr) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc != TCCL_OK ? rc : (e != hipSuccess ? hip_code(e) : TCCL_EINVAL);
    }
    tccl_plan *plan = new (std::nothrow) tccl_plan;
    if (plan == nullptr) {
        (void)hipGraphDestroy(graph);
        return hip_code(hipErrorOutOfMemory);
    }
    plan->graph = graph;
    e = hipGraphInstantiate(&plan->exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        delete plan;
        return hip_code(e);
    }
    *plan_out = plan;
    return TCCL_OK;
}

extern "C" int tccl_plan_launch(tccl_plan *plan, void *stream)
{
    if (plan == nullptr || plan->exec == nullptr) return TCCL_EINVAL;
    return hip_code(hipGraphLaunch(plan->exec, static_cast<hipStream_t>(stream)));
}

extern "C" int tccl_plan_destroy(tccl_plan *plan)
{
    if (plan == nullptr) return TCCL_EINVAL;
    hipError_t e1 = plan->exec ? hipGraphExecDestroy(plan->exec) : hipSuccess;
    hipError_t e2 = plan->graph ? hipGraphDestroy(plan->graph) : hipSuccess;
    delete plan;
    return hip_code(e1 != hipSuccess ? e1 : e2);
}
