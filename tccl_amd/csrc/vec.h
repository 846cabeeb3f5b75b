// vec.h -- 16-byte vector access and the bf16/fp32 sum arithmetic shared by every kernel.
//
// Everything here is written for gfx950 wave64: one lane moves one 16-byte vector per
// access (global_load_dwordx4 / global_store_dwordx4), so a wave instruction covers one
// contiguous KiB.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace tccl {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kVecBytes = 16;
constexpr int kMaxBlock = 512;
constexpr int kNumXcd = 8;

// Time stamps for measurement builds.  The library itself is built without TCCL_STAMPS and
// TCCL_STAMP() is nothing there.  benchlib/stamped.hip defines it and includes every source of
// the library as one translation unit: each workgroup then records the 100 MHz wall clock at
// four points of its work, in stamp_words[4 * b + slot] for workgroup b (y-major):
//   slot 0  the workgroup's first instruction            (its first wave)
//   slot 1  the loads of its first iteration have arrived (latest wave)
//   slot 2  its last load has arrived and been reduced    (latest wave)
//   slot 3  its last store has been acknowledged          (latest wave)
// The host clears the words before a launch and reads them after it.
#ifdef TCCL_STAMPS
constexpr int kStampSlots = 4;
constexpr int kStampMaxWorkgroups = 1 << 16;
__device__ long long stamp_words[kStampSlots * kStampMaxWorkgroups];

template <int SLOT, bool DRAIN>
__device__ __forceinline__ void stamp()
{
    // SLOT 1 sits inside the read loop: loads of later iterations may still be moved across
    // it (mask 0x20 = memory reads), the adds that consume this iteration's loads may not
    __builtin_amdgcn_sched_barrier(SLOT == 1 ? 0x20 : 0);
    if constexpr (DRAIN) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const long long t = wall_clock64();
    const size_t b = static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x;
    if (b < kStampMaxWorkgroups && (threadIdx.x & 63) == 0) {
        if constexpr (SLOT == 0) {
            if (threadIdx.x == 0) stamp_words[kStampSlots * b] = t;
        } else {
            __hip_atomic_fetch_max(stamp_words + kStampSlots * b + SLOT, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __builtin_amdgcn_sched_barrier(SLOT == 1 ? 0x20 : 0);
}
#define TCCL_STAMP(slot, drain) ::tccl::stamp<slot, drain>()
#else
#define TCCL_STAMP(slot, drain) ((void)0)
#endif

template <bool NT>
__device__ __forceinline__ u32x4 load_vec(const char *base, size_t vec_index)
{
    const u32x4 *p = reinterpret_cast<const u32x4 *>(base) + vec_index;
    if constexpr (NT)
        return __builtin_nontemporal_load(p);
    else
        return *p;
}

template <bool NT>
__device__ __forceinline__ void store_vec(char *base, size_t vec_index, u32x4 v)
{
    u32x4 *p = reinterpret_cast<u32x4 *>(base) + vec_index;
    if constexpr (NT)
        __builtin_nontemporal_store(v, p);
    else
        *p = v;
}

__device__ __forceinline__ float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// Two fp32 -> two bf16 packed in a dword (element 0 in the low half), round to nearest
// even: one v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    f32x2 f = {lo, hi};
    bf16x2 b = __builtin_convertvector(f, bf16x2);
    return __builtin_bit_cast(uint32_t, b);
}

// bf16 sums: eight fp32 accumulators per 16-byte vector.
struct Bf16Sum {
    static constexpr int kElemBytes = 2;
    // large tiles: sixteen conversions and adds per vector pace the loads already (5-10
    // outstanding per lane as compiled); forcing the barrier measured the same within noise
    static constexpr bool kPaceLoads = false;
    float a[8];

    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int k = 0; k < 8; ++k) a[k] = 0.0f;
    }
    // Widening bf16 -> fp32 is a 16-bit shift (exact).
    __device__ __forceinline__ void add(u32x4 v)
    {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            a[2 * k] = a[2 * k] + bits_to_f32(v[k] << 16);
            a[2 * k + 1] = a[2 * k + 1] + bits_to_f32(v[k] & 0xFFFF0000u);
        }
    }
    __device__ __forceinline__ u32x4 result() const
    {
        u32x4 r;
#pragma unroll
        for (int k = 0; k < 4; ++k) r[k] = pack_bf16(a[2 * k], a[2 * k + 1]);
        return r;
    }
    // One element at a time, for the ragged tail.
    static __device__ __forceinline__ float widen(const char *p, size_t i)
    {
        return bits_to_f32(static_cast<uint32_t>(reinterpret_cast<const uint16_t *>(p)[i]) << 16);
    }
    static __device__ __forceinline__ void narrow(char *p, size_t i, float f)
    {
        reinterpret_cast<uint16_t *>(p)[i] = static_cast<uint16_t>(pack_bf16(f, 0.0f) & 0xFFFFu);
    }
};

// fp32 sums: four accumulators per vector, no final rounding.
struct F32Sum {
    static constexpr int kElemBytes = 4;
    static constexpr bool kPaceLoads = true; // large tiles: see sum_tile_phased
    float a[4];

    __device__ __forceinline__ void zero()
    {
#pragma unroll
        for (int k = 0; k < 4; ++k) a[k] = 0.0f;
    }
    __device__ __forceinline__ void add(u32x4 v)
    {
#pragma unroll
        for (int k = 0; k < 4; ++k) a[k] = a[k] + bits_to_f32(v[k]);
    }
    __device__ __forceinline__ u32x4 result() const
    {
        u32x4 r;
#pragma unroll
        for (int k = 0; k < 4; ++k) r[k] = f32_to_bits(a[k]);
        return r;
    }
    static __device__ __forceinline__ float widen(const char *p, size_t i)
    {
        return reinterpret_cast<const float *>(p)[i];
    }
    static __device__ __forceinline__ void narrow(char *p, size_t i, float f)
    {
        reinterpret_cast<float *>(p)[i] = f;
    }
};

// The order in which a workgroup visits tiles.  Workgroups are handed to the 8 XCDs
// round-robin (workgroup b runs on XCD b % 8).  Plain order: workgroup b takes tiles
// b, b + grid, b + 2*grid, ... so neighbouring tiles land on different XCDs.
// XCD-contiguous order: each XCD owns one contiguous eighth of the tiles and its
// workgroups stride through that eighth, so each XCD's L2 and TLBs see one dense address
// range per source (the host makes the grid a multiple of 8 for this order).
struct TileWalk {
    size_t k, step, limit, offset, ntiles;
    __device__ __forceinline__ TileWalk(bool xcd_contiguous, size_t ntiles_) : ntiles(ntiles_)
    {
        const size_t b = blockIdx.x;
        if (xcd_contiguous) {
            limit = (ntiles + kNumXcd - 1) / kNumXcd;
            offset = (b % kNumXcd) * limit;
            k = b / kNumXcd;
            step = gridDim.x / kNumXcd;
            if (step == 0) step = 1; // cannot happen with a host-sized grid; keeps the walk finite
        } else {
            limit = ntiles;
            offset = 0;
            k = b;
            step = gridDim.x;
        }
    }
    __device__ __forceinline__ bool valid() const { return k < limit && offset + k < ntiles; }
    __device__ __forceinline__ size_t tile() const { return offset + k; }
    __device__ __forceinline__ void next() { k += step; }
};

// Sum NSRC sources into NDST destinations over the vector range [0, nvec), then the
// ragged tail elements [nvec*per_vec, numel).  Work is cut into tiles of
// tile_iters * blockDim.x * UNROLL vectors; a workgroup walks one tile front to back and
// then jumps gridDim.x tiles ahead.  Inside an iteration a lane issues all NSRC*UNROLL
// loads before the first add, so up to NSRC*UNROLL*16 bytes per lane are in flight.
// Sources are added in index order into an accumulator that starts at +0.  A destination
// may alias a source: every vector is read and written by the same lane in the same
// iteration, reads first.
template <class Sum, int NSRC, int NDST, int UNROLL, bool NTL, bool NTS>
__device__ __forceinline__ void sum_range(const char *const (&src)[NSRC], char *const (&dst)[NDST],
                                          size_t numel, int tile_iters, bool xcd_contiguous)
{
    constexpr size_t per_vec = kVecBytes / Sum::kElemBytes;
    const size_t nvec = numel / per_vec;
    const size_t span = static_cast<size_t>(blockDim.x) * UNROLL;
    const size_t tile = span * static_cast<size_t>(tile_iters);
    const size_t ntiles = (nvec + tile - 1) / tile;

    for (TileWalk w(xcd_contiguous, ntiles); w.valid(); w.next()) {
        const size_t t0 = w.tile() * tile;
        const size_t t1 = (t0 + tile < nvec) ? t0 + tile : nvec;
        for (size_t base = t0; base < t1; base += span) {
            u32x4 v[UNROLL][NSRC];
            if (base + span <= t1) {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                    for (int s = 0; s < NSRC; ++s)
                        v[u][s] = load_vec<NTL>(src[s], base + static_cast<size_t>(u) * blockDim.x + threadIdx.x);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    Sum acc;
                    acc.zero();
#pragma unroll
                    for (int s = 0; s < NSRC; ++s) acc.add(v[u][s]);
                    const u32x4 r = acc.result();
#pragma unroll
                    for (int d = 0; d < NDST; ++d)
                        store_vec<NTS>(dst[d], base + static_cast<size_t>(u) * blockDim.x + threadIdx.x, r);
                }
            } else {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const size_t i = base + static_cast<size_t>(u) * blockDim.x + threadIdx.x;
                    if (i < t1) {
                        Sum acc;
                        acc.zero();
#pragma unroll
                        for (int s = 0; s < NSRC; ++s) acc.add(load_vec<NTL>(src[s], i));
                        const u32x4 r = acc.result();
#pragma unroll
                        for (int d = 0; d < NDST; ++d) store_vec<NTS>(dst[d], i, r);
                    }
                }
            }
        }
    }

    // Ragged tail: fewer than per_vec elements, handled by the first lanes of workgroup 0.
    const size_t tail0 = nvec * per_vec;
    if (blockIdx.x == 0 && tail0 + threadIdx.x < numel) {
        const size_t i = tail0 + threadIdx.x;
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < NSRC; ++s) acc = acc + Sum::widen(src[s], i);
#pragma unroll
        for (int d = 0; d < NDST; ++d) Sum::narrow(dst[d], i, acc);
    }
}

// ---------------------------------------------------------------------------------
// Phased tiles.  HBM serves reads and writes over one data bus and loses time on every
// turn-around, so a kernel that interleaves its output stores with its input loads runs
// well below the sum of a pure read pass and a pure write pass.  A phased workgroup owns
// one contiguous tile: it reads and reduces the whole tile into registers first
// (K iterations of U vectors per lane) and only then writes the tile's results, back to
// back.  When all workgroups of a launch are resident at once and run at the same pace,
// the launch as a whole turns into one long read phase followed by one write burst.
//
// Tiles are addressed through buffer descriptors whose size is the exact number of valid
// bytes left in the tile: loads beyond the end return zero and stores beyond the end are
// dropped by the hardware, so a partial tile needs no branches.

constexpr int kPhasedBlock = 256; // lanes per workgroup
constexpr int kPhasedVecs = 32;   // result vectors a lane holds before it writes (128 VGPRs)
constexpr int kAuxLoadStream = 2;   // cache policy of the loads: nt (stream through L2)
constexpr int kAuxStoreStream = 16; // cache policy of a tile's result stores: sc1 (write through to memory)
constexpr int kAuxStoreNt = 2;      // cache policy of the stores of streaming copies: nt
constexpr int kAuxLoadDevice = 18;  // sc1 nt: device-scope loads, coherent with sc1 stores of other XCDs

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_rsrc(const char *tile_start, uint32_t valid_bytes)
{
    // stride 0 (raw buffer), 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(tile_start), 0, static_cast<int>(valid_bytes),
                                             0x00020000);
}

// Vectors per lane per iteration for a given number of sources (two candidates each,
// the first is the default).
template <int NSRC>
struct PhasedUnroll {
    static constexpr int value = NSRC <= 2 ? 4 : (NSRC <= 4 ? 2 : 1);
    static constexpr int alt = value * 2;
};

// One tile: sources [tile_off, tile_off + valid) -> destinations, `kcount` <= KMAX
// iterations of kPhasedBlock * U vectors.  valid is a multiple of 16 (may be 0).
// FULL = the tile has exactly KMAX iterations: straight-line code, which lets the
// compiler start the loads of the next iteration before the adds of this one.
// LAUX = cache policy of the loads.  PIECE maps an iteration to the place of its
// kPhasedBlock * U vectors inside the tile (in units of that many vectors): the identity
// for a contiguous tile, something else when workgroups interleave their tiles.
struct PieceInOrder {
    static constexpr uint32_t at(int k) { return static_cast<uint32_t>(k); }
};
template <class Sum, int NSRC, int NDST, int U, int KMAX, bool FULL, bool PACE = false, int LAUX = kAuxLoadStream,
          class PIECE = PieceInOrder>
__device__ __forceinline__ void sum_tile_phased(const char *const (&src)[NSRC], char *const (&dst)[NDST],
                                                size_t tile_off, uint32_t valid_bytes, int kcount)
{
    __amdgpu_buffer_rsrc_t rs[NSRC];
#pragma unroll
    for (int s = 0; s < NSRC; ++s) rs[s] = tile_rsrc(src[s] + tile_off, valid_bytes);
    constexpr uint32_t span_bytes = kPhasedBlock * U * kVecBytes;
    const uint32_t lane_off = threadIdx.x * kVecBytes;

    u32x4 r[KMAX][U];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        if (FULL || k < kcount) {
            u32x4 v[U][NSRC];
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int s = 0; s < NSRC; ++s)
                    v[u][s] = __builtin_amdgcn_raw_buffer_load_b128(
                        rs[s], PIECE::at(k) * span_bytes + u * (kPhasedBlock * kVecBytes) + lane_off, 0, LAUX);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                Sum acc;
                acc.zero();
#pragma unroll
                for (int s = 0; s < NSRC; ++s) acc.add(v[u][s]);
                r[k][u] = acc.result();
            }
            // PACE: keep the loads of later iterations behind this iteration's adds.  With
            // 128 KiB tiles at two waves per SIMD the memory system runs best with about
            // 8-16 loads of 16 bytes outstanding per lane; left alone, the compiler hoists
            // as many loads as it has registers for (30+ with the four adds per vector of
            // fp32), which measured 7 % slower there.  (With the 32 KiB tiles of the tree
            // level kernel the barrier measured 1-5 % slower, so it is not used there.)
            if constexpr (PACE) __builtin_amdgcn_sched_barrier(0);
            if (k == 0) TCCL_STAMP(1, false);
        }
    }
    TCCL_STAMP(2, false);
#pragma unroll
    for (int d = 0; d < NDST; ++d) {
        const __amdgpu_buffer_rsrc_t rd = tile_rsrc(dst[d] + tile_off, valid_bytes);
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
            if (FULL || k < kcount) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    __builtin_amdgcn_raw_buffer_store_b128(r[k][u], rd,
                                                           PIECE::at(k) * span_bytes + u * (kPhasedBlock * kVecBytes) + lane_off,
                                                           0, kAuxStoreStream);
            }
        }
    }
    TCCL_STAMP(3, true);
}

// Same walk for a plain copy of one source into NDST destinations.
template <int NDST, int U, int KMAX, int LAUX = kAuxLoadStream>
__device__ __forceinline__ void copy_tile_phased(const char *src, char *const (&dst)[NDST], size_t tile_off,
                                                 uint32_t valid_bytes, int kcount)
{
    const __amdgpu_buffer_rsrc_t rs = tile_rsrc(src + tile_off, valid_bytes);
    constexpr uint32_t span_bytes = kPhasedBlock * U * kVecBytes;
    const uint32_t lane_off = threadIdx.x * kVecBytes;
    u32x4 r[KMAX][U];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        if (k < kcount) {
#pragma unroll
            for (int u = 0; u < U; ++u)
                r[k][u] = __builtin_amdgcn_raw_buffer_load_b128(
                    rs, k * span_bytes + u * (kPhasedBlock * kVecBytes) + lane_off, 0, LAUX);
        }
    }
#pragma unroll
    for (int d = 0; d < NDST; ++d) {
        const __amdgpu_buffer_rsrc_t rd = tile_rsrc(dst[d] + tile_off, valid_bytes);
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
            if (k < kcount) {
#pragma unroll
                for (int u = 0; u < U; ++u)
                    __builtin_amdgcn_raw_buffer_store_b128(
                        r[k][u], rd, k * span_bytes + u * (kPhasedBlock * kVecBytes) + lane_off, 0, kAuxStoreStream);
            }
        }
    }
    TCCL_STAMP(3, true);
}

// The ragged tail: elements [first, numel), fewer than one vector, one lane each.
template <class Sum, int NSRC, int NDST>
__device__ __forceinline__ void sum_tail(const char *const (&src)[NSRC], char *const (&dst)[NDST], size_t first,
                                         size_t numel)
{
    const size_t i = first + threadIdx.x;
    if (i < numel) {
        float acc = 0.0f;
#pragma unroll
        for (int s = 0; s < NSRC; ++s) acc = acc + Sum::widen(src[s], i);
#pragma unroll
        for (int d = 0; d < NDST; ++d) Sum::narrow(dst[d], i, acc);
    }
}

// Copy one source into NDST destinations over [0, nvec) vectors; same tiling as sum_range.
template <int NDST, int UNROLL, bool NTL, bool NTS>
__device__ __forceinline__ void copy_range(const char *src, char *const (&dst)[NDST], size_t nvec,
                                           int tile_iters, bool xcd_contiguous)
{
    const size_t span = static_cast<size_t>(blockDim.x) * UNROLL;
    const size_t tile = span * static_cast<size_t>(tile_iters);
    const size_t ntiles = (nvec + tile - 1) / tile;
    for (TileWalk w(xcd_contiguous, ntiles); w.valid(); w.next()) {
        const size_t t0 = w.tile() * tile;
        const size_t t1 = (t0 + tile < nvec) ? t0 + tile : nvec;
        for (size_t base = t0; base < t1; base += span) {
            if (base + span <= t1) {
                u32x4 v[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u)
                    v[u] = load_vec<NTL>(src, base + static_cast<size_t>(u) * blockDim.x + threadIdx.x);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u)
#pragma unroll
                    for (int d = 0; d < NDST; ++d)
                        store_vec<NTS>(dst[d], base + static_cast<size_t>(u) * blockDim.x + threadIdx.x, v[u]);
            } else {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const size_t i = base + static_cast<size_t>(u) * blockDim.x + threadIdx.x;
                    if (i < t1) {
                        const u32x4 v = load_vec<NTL>(src, i);
#pragma unroll
                        for (int d = 0; d < NDST; ++d) store_vec<NTS>(dst[d], i, v);
                    }
                }
            }
        }
    }
}

// Pack copy: `rows` sources of row_vecs vectors each into one output, row after row.  The
// tile index runs over all rows in row-major order, so at any moment the whole grid works
// on one dense window of one source and one dense window of the output (two DRAM streams,
// not 2 x rows).
template <int UNROLL, bool NTL, bool NTS>
__device__ __forceinline__ void pack_rows(const char *const *rows_base, int rows, char *out, size_t row_vecs,
                                          int tile_iters, bool xcd_contiguous)
{
    const size_t span = static_cast<size_t>(blockDim.x) * UNROLL;
    const size_t tile = span * static_cast<size_t>(tile_iters);
    const size_t tiles_per_row = (row_vecs + tile - 1) / tile;
    const size_t ntiles = tiles_per_row * static_cast<size_t>(rows);
    for (TileWalk w(xcd_contiguous, ntiles); w.valid(); w.next()) {
        const size_t row = w.tile() / tiles_per_row;
        const size_t t0 = (w.tile() - row * tiles_per_row) * tile;
        const size_t t1 = (t0 + tile < row_vecs) ? t0 + tile : row_vecs;
        const char *src = rows_base[row];
        char *dst = out + row * row_vecs * kVecBytes;
        for (size_t base = t0; base < t1; base += span) {
            if (base + span <= t1) {
                u32x4 v[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u)
                    v[u] = load_vec<NTL>(src, base + static_cast<size_t>(u) * blockDim.x + threadIdx.x);
#pragma unroll
                for (int u = 0; u < UNROLL; ++u)
                    store_vec<NTS>(dst, base + static_cast<size_t>(u) * blockDim.x + threadIdx.x, v[u]);
            } else {
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const size_t i = base + static_cast<size_t>(u) * blockDim.x + threadIdx.x;
                    if (i < t1) store_vec<NTS>(dst, i, load_vec<NTL>(src, i));
                }
            }
        }
    }
}

} // namespace tccl
