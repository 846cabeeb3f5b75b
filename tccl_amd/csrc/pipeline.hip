// pipeline.hip -- the double tree as ONE persistent launch in which every virtual rank's
// workgroups hand pipelining chunks to each other through signal flags, the way the
// reference's per-rank kernel is designed to (triton_double_tree_allreduce.py:254-335:
// wait for the children, reduce, signal the parent, wait for the parent, copy, signal
// the children), with its wait/send pair (triton_double_tree_allreduce.py:175-225) and its
// signal-pad addressing (a sender writes slot `block * world + sender` of the receiver's
// pad; triton_barrier.py:39-142) rewritten for gfx950.
//
// Differences from the reference's protocol, on purpose:
//  * one slot per (chunk, sender) instead of one per (block, sender), so a sender never has
//    to wait for the receiver to drain the previous chunk's signal (the reference's send
//    spins on a compare-and-swap 0 -> 1 for that); every slot has exactly one writer and
//    one reader per call, so a plain store raises a flag (the wait is still the reference's
//    compare-and-swap 1 -> 0);
//  * the reader writes the slot back to 0 after it has seen the signal, so a pad that starts
//    zero-filled is zero-filled again after every completed call (the property that makes the
//    reference's barrier usable under graph replay);
//  * every wait is bounded: a workgroup that polls `spin_limit` times without seeing its
//    signal counts one time-out in the control words of pad 0 (and raises the caller's host
//    flag, if it gave one) and leaves the kernel; whoever waits for that workgroup then times
//    out the same way, so the grid always drains.
//
// Forward progress.  With the default binding of places to workgroups (by hardware index) a
// workgroup waits for workgroups anywhere in the grid, so every workgroup of the launch must
// be resident at once: the grid never exceeds the occupancy the runtime reports for the
// kernel, and a wait that still expires is reported, never hidden.  With
// TCCL_PIPE_DRAW_PLACES forward progress does not depend on residency at all: a workgroup
// takes its place -- which rank it works for and which index g it has among that rank's
// workgroups -- from a counter it draws from when it starts to run (take_place), so places are
// handed out in the order in which workgroups really begin to run; and a workgroup only ever
// waits for the workgroups with the same g of the other ranks, whose places are drawn right
// before and after its own from the same counter.  So of all groups of W workgroups with
// equal g that still have work to do, all but at most one per counter (the one being drawn)
// have every member running: they can finish, their slots go to workgroups that have not
// started, and those draw the missing places first.  At most 8 * (W - 1) = 56 workgroups can
// sit waiting for members that have not started, fewer than the slots of any one XCD (32
// compute units x at least 2 workgroups), so a slot for the next starter is always there,
// whatever else runs on the GPU.
#include <mutex>

#include "host.h"
#include "vec.h"

namespace tccl {

constexpr int kPipeMaxWorld = TCCL_MAX_WORLD;
constexpr uint32_t kPipeDefaultSpins = 1u << 21;
// Most workgroups per compute unit a grid whose workgroups wait for each other may have (see
// resident_for).
constexpr int kMaxSignallingPerUnit = 6;
// Most workgroups per rank of a per-rank launch of the double tree that carries its own barriers
// (its pads have two rows of barrier slots for that many).
constexpr size_t kTreeBarrierWorkgroups = 512;

// Two signalling kernels that overlap on one GPU could each hold part of the workgroup slots
// and (with places bound by hardware index) starve each other until their waits expire; with
// drawn places they would only slow each other down.  Launches of this process are therefore
// chained: each one first makes its stream wait for the previous signalling kernel of the same
// device (an event wait, no host blocking), whatever stream that one ran on.  A stream that is
// being captured into a graph is left alone (an outside event cannot be waited for inside a
// capture); keeping replays of such graphs apart is then the caller's business.
class SignallingLaunch {
public:
    explicit SignallingLaunch(hipStream_t stream) : stream_(stream), lock_(mutex())
    {
        hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &status) != hipSuccess || status != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return;
        }
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return;
        hipEvent_t &ev = events()[dev];
        if (ev == nullptr) {
            if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) {
                ev = nullptr;
                return;
            }
        } else if (hipStreamWaitEvent(stream, ev, 0) != hipSuccess) {
            return;
        }
        event_ = ev;
    }
    // after the kernel has been enqueued
    void launched()
    {
        if (event_ != nullptr) (void)hipEventRecord(event_, stream_);
    }

private:
    static constexpr int kMaxDevices = 64;
    static std::mutex &mutex()
    {
        static std::mutex m;
        return m;
    }
    static hipEvent_t *events()
    {
        static hipEvent_t e[kMaxDevices] = {};
        return e;
    }
    hipStream_t stream_;
    std::unique_lock<std::mutex> lock_;
    hipEvent_t event_ = nullptr;
};

struct PipeArgs {
    char *buf[kPipeMaxWorld];
    char *out[kPipeMaxWorld]; // entries may be null
    uint32_t *pad[kPipeMaxWorld];
    signed char nbr[2][kPipeMaxWorld][3]; // parent, child0, child1 (-1 = none)
    signed char height[2][kPipeMaxWorld]; // 0 = leaf ... tree_height = the extra node on top
    size_t half_off[2];                   // byte offset of each tree's half inside a buffer
    size_t half_bytes[2];
    uint32_t nchunks[2];
    uint32_t chunk_bytes; // multiple of 16
    uint32_t slots;       // chunk slots per tree in a pad (>= both nchunks)
    uint32_t spin_limit;
    int world, wgs_per_rank, lag, tree_height;
    int draw;         // 1 = workgroups draw their places when they start, 0 = places follow the hardware index
    int only_rank;    // >= 0: the launch holds this rank's workgroups only (one launch per rank); -1: all ranks'
    int own_barriers; // one launch per rank: the kernel also begins and ends with the blockwise barrier
    uint32_t barrier_base; // first word of the barriers' slots in a pad (behind the chunk slots)
    uint32_t *ctl;    // the control words at the end of pad 0 (place counters ... time-outs)
    uint32_t *report; // optional word in host memory that is set to 1 when a wait expires
};

// The last kCtlWords 32-bit words of pad 0: eight place counters (one per list, a cache line
// apart so that draws from different lists do not queue behind each other in the memory-side
// atomic unit: draws from one counter take about 10 ns each), the count of lists that have
// been drawn completely, and -- the very last word -- the count of time-outs.
constexpr int kCtlStride = 32; // words between two place counters
constexpr int kCtlListsDone = kNumXcd * kCtlStride;
constexpr int kCtlWords = kCtlListsDone + kCtlStride;
constexpr int kCtlTimeouts = kCtlWords - 1;
constexpr uint32_t kNoPlace = 0xFFFFFFFFu;
static_assert(kCtlWords == TCCL_PAD_CONTROL_WORDS, "header and library disagree");

// The XCD this wave runs on (0..7): bits 3:0 of the XCC_ID hardware register.  Only a hint
// for locality; nothing depends on its value being right.
__device__ __forceinline__ uint32_t xcd_of_this_wave()
{
    // s_getreg_b32 hwreg(HW_REG_XCC_ID = 20, offset 0, width 4): id | offset << 6 | (width - 1) << 11
    return __builtin_amdgcn_s_getreg(20 | (0 << 6) | (3 << 11)) & (kNumXcd - 1);
}

// A workgroup's place in the collective is (rank, g) with g < wgs_per_rank.  Two ways to get it.
//
// By hardware index (the default): workgroup b of the grid is rank b / wgs_per_rank, index
// b % wgs_per_rank.  This is the faster binding on large inputs (which compute unit runs
// which place matters to the memory system: the same kernel with places bound to workgroups
// in any other way measured 4-15 % slower at 64-256 MiB per buffer), but a workgroup then
// waits for workgroups far away in the grid, so the whole grid must be resident at once.
//
// By drawing (TCCL_PIPE_DRAW_PLACES): the place is drawn from a counter when the workgroup
// starts to run.  The places are kept in 8 lists, list x holding the places with g % 8 == x
// in the order (g, rank); a workgroup draws the next place of the list of the XCD it runs on,
// and goes on to the following lists when that one has been drawn completely (there are
// exactly as many workgroups as places, so it always finds one).  Two things follow.
// (1) Within a list places are drawn in order, so the W places with the same g -- the only
// workgroups that ever wait for each other -- are drawn one after the other, and once any
// later place of the list has been drawn all W of them are running.  (2) Workgroups with the
// same g of all ranks run on the same XCD (as far as the hardware spreads the grid evenly),
// so a chunk one of them wrote a moment ago is read by the next from that XCD's L2 -- as with
// the default binding when wgs_per_rank is a multiple of 8.
// The counters start at zero (the pads are zero-filled before the first call).  The workgroup
// that draws the last place of a list counts the list as done; the one that completes the
// count knows that every workgroup of the launch has drawn its place -- nobody will touch
// the counters again -- and puts all of them back to zero for the next launch.
__device__ __forceinline__ void take_place(uint32_t *ctl, bool draw, uint32_t world, uint32_t wgs_per_rank, int *rank,
                                           uint32_t *g, uint32_t *lds_place)
{
    if (!draw) {
        *rank = static_cast<int>(blockIdx.x / wgs_per_rank);
        *g = blockIdx.x % wgs_per_rank;
        return;
    }
    if (threadIdx.x == 0) {
        const uint32_t first = xcd_of_this_wave();
        uint32_t r = 0, gg = kNoPlace; // no place: cannot happen, there are as many places as workgroups
        for (uint32_t k = 0; k < kNumXcd; ++k) {
            const uint32_t x = (first + k) & (kNumXcd - 1);
            if (x >= wgs_per_rank) continue; // an empty list
            const uint32_t places = world * ((wgs_per_rank - x + kNumXcd - 1) / kNumXcd);
            const uint32_t u =
                __hip_atomic_fetch_add(ctl + x * kCtlStride, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (u >= places) continue; // that list has been drawn completely
            gg = x + kNumXcd * (u / world);
            r = u % world;
            if (u + 1 == places) {
                const uint32_t lists = wgs_per_rank < kNumXcd ? wgs_per_rank : kNumXcd;
                const uint32_t done =
                    __hip_atomic_fetch_add(ctl + kCtlListsDone, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (done + 1 == lists) {
                    for (uint32_t y = 0; y < kNumXcd; ++y)
                        __hip_atomic_store(ctl + y * kCtlStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(ctl + kCtlListsDone, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            break;
        }
        lds_place[0] = r;
        lds_place[1] = gg;
    }
    __syncthreads();
    // the same for every lane: say so, so that everything derived from them (buffer addresses,
    // descriptors, loop bounds) stays in scalar registers
    *rank = __builtin_amdgcn_readfirstlane(static_cast<int>(lds_place[0]));
    *g = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(lds_place[1])));
}

// A wait expired: count it, and tell the host if it gave us a word to tell it through.
__device__ __forceinline__ void report_timeout(uint32_t *ctl, uint32_t *report)
{
    __hip_atomic_fetch_add(ctl + kCtlTimeouts, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (report != nullptr) __hip_atomic_store(report, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// Take a raised flag: polls the slot with a compare-and-swap 1 -> 0, the reference's own wait
// (triton_barrier.py:108-118), until it succeeds or the wait's budget is used up.  A device-scope
// read-modify-write is carried out where all XCDs meet, so the poll sees the flag wherever its
// sender ran, and seeing and lowering it are one step.
//
// The polls back off.  A launch that begins with a barrier may have a thousand workgroups
// waiting for a rank that is still busy with the kernel before its collective, and every poll
// goes to the few memory channels that hold the pads -- channels which that rank's kernel needs
// as well.  So the first 64 polls come about 0.2 us apart, and the pause doubles with every
// further 64 polls up to about 30 us: a flag is still taken within a fraction of the time it
// has been waited for.  The budget counts pauses, not polls: spin_limit units of about 0.2 us.
__device__ __forceinline__ bool take_flag(uint32_t *slot, uint32_t spin_limit, uint32_t *spent)
{
    uint32_t nap = 1, round = 0;
    for (;;) {
        uint32_t expect = 1u;
        if (__hip_atomic_compare_exchange_strong(slot, &expect, 0u, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT))
            return true;
        *spent += nap;
        if (*spent >= spin_limit) return false;
        for (uint32_t i = 0; i < nap; ++i) __builtin_amdgcn_s_sleep(8);
        if (++round == 64) {
            round = 0;
            if (nap < 128) nap *= 2;
        }
    }
}

// Coherence between workgroups on different XCDs (each XCD has its own L2) without flushing
// or invalidating whole caches: every store of this kernel is a device-scope store (sc1: it
// is written through to memory and acknowledged from there) and every load of data that a
// peer may have rewritten during the kernel is a device-scope load (sc1: it never hits a
// stale line of the local L2).  What is left is ordering: a wave waits until all its stores
// have been acknowledged, the workgroup meets, then one lane raises the flag.
__device__ __forceinline__ void send_signals(uint32_t *slot0, uint32_t *slot1)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        if (slot0 != nullptr) __hip_atomic_store(slot0, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (slot1 != nullptr) __hip_atomic_store(slot1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Wait until every non-null slot has been raised, and lower it again.  One lane polls (with
// take_flag); the result reaches the other lanes through LDS, and the barrier keeps
// every lane's later loads behind the poll that saw the flag.  Returns false after
// spin_limit polls without success (counted in the control words); the caller then leaves the
// kernel.
__device__ __forceinline__ bool wait_signals(uint32_t *slot0, uint32_t *slot1, uint32_t spin_limit, uint32_t *ctl,
                                             uint32_t *report, int *lds_ok)
{
    if (slot0 == nullptr && slot1 == nullptr) return true; // uniform over the workgroup
    if (threadIdx.x == 0) {
        bool ok = true;
        uint32_t *const slots[2] = {slot0, slot1};
        uint32_t polls = 0;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            uint32_t *s = slots[i];
            if (s == nullptr || !ok) continue;
            ok = take_flag(s, spin_limit, &polls);
        }
        if (!ok) report_timeout(ctl, report);
        *lds_ok = ok ? 1 : 0;
    }
    __syncthreads();
    const int ok = *lds_ok;
    __syncthreads(); // lds_ok may be rewritten by the next wait only after everyone has read it
    return ok != 0;
}

// The reference's blockwise barrier (triton_barrier.py:39-142) between the workgroups with the
// same index of all W ranks, on the W slots that start at word `base` of every pad: lane i < W of
// the first wave raises slot `base + rank` in rank i's pad and takes slot `base + i` of the own
// pad (each slot has one writer and one reader, so the sender's compare-and-swap 0 -> 1 of the
// reference becomes a plain store; the wait is its compare-and-swap 1 -> 0, take_flag).
// Everything the workgroup stored before the barrier is visible to its peers' device-scope loads
// after it.  *lds_ok must be 1 on entry; returns false when a wait expired (counted in the
// control words).
__device__ __forceinline__ bool barrier_on_slots(uint32_t *const *pad, int world, int rank, uint32_t base,
                                                 uint32_t spin_limit, uint32_t *ctl, uint32_t *report, int *lds_ok)
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int lane = threadIdx.x;
    if (lane < world && lane != rank) {
        __hip_atomic_store(pad[lane] + base + rank, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t spent = 0;
        if (!take_flag(pad[rank] + base + lane, spin_limit, &spent)) {
            report_timeout(ctl, report);
            *lds_ok = 0; // any lane that failed clears the flag
        }
    }
    __syncthreads();
    return *lds_ok != 0;
}

// One chunk of a reduce step: sources -> destinations, in tiles of VECS vectors per lane
// (256 lanes: 32 KiB for VECS = 8, 128 KiB for VECS = 32), each read and reduced into
// registers and then written.
template <class Sum, int VECS, int NSRC, int NDST>
__device__ __forceinline__ void reduce_chunk(const char *const (&src)[NSRC], char *const (&dst)[NDST], size_t off,
                                             uint32_t bytes)
{
    constexpr int U = VECS >= 32 ? PhasedUnroll<NSRC>::value : 2;
    constexpr int KMAX = VECS / U;
    constexpr uint32_t span = kPhasedBlock * U * kVecBytes;
    constexpr uint32_t kPipeTileBytes = kPhasedBlock * VECS * kVecBytes;
    for (uint32_t done = 0; done < bytes; done += kPipeTileBytes) {
        const uint32_t valid = bytes - done < kPipeTileBytes ? bytes - done : kPipeTileBytes;
        const int kcount = static_cast<int>((valid + span - 1) / span);
        if (valid == kPipeTileBytes)
            sum_tile_phased<Sum, NSRC, NDST, U, KMAX, true, false, kAuxLoadDevice>(src, dst, off + done, valid, KMAX);
        else
            sum_tile_phased<Sum, NSRC, NDST, U, KMAX, false, false, kAuxLoadDevice>(src, dst, off + done, valid, kcount);
    }
}

template <int VECS, int NDST>
__device__ __forceinline__ void copy_chunk(const char *src, char *const (&dst)[NDST], size_t off, uint32_t bytes)
{
    constexpr int U = 4;
    constexpr int KMAX = VECS / U;
    constexpr uint32_t span = kPhasedBlock * U * kVecBytes;
    constexpr uint32_t kPipeTileBytes = kPhasedBlock * VECS * kVecBytes;
    for (uint32_t done = 0; done < bytes; done += kPipeTileBytes) {
        const uint32_t valid = bytes - done < kPipeTileBytes ? bytes - done : kPipeTileBytes;
        copy_tile_phased<NDST, U, KMAX, kAuxLoadDevice>(src, dst, off + done, valid, static_cast<int>((valid + span - 1) / span));
    }
}

// Up-sweep step of `rank` in tree t for chunk c: own <- 0 + child0 + child1 + own (absent
// children skipped), in place; the extra node on top also writes its output, because its
// sum is the final result.  Returns false on a time-out.
template <class Sum, int VECS>
__device__ __forceinline__ bool up_step(const PipeArgs &a, int rank, int t, uint32_t c, int *lds_ok)
{
    const int h = a.height[t][rank];
    if (h == 0) return true; // a leaf's own step changes nothing anyone can see
    const int parent = a.nbr[t][rank][0], c0 = a.nbr[t][rank][1], c1 = a.nbr[t][rank][2];
    const uint32_t slot = (static_cast<uint32_t>(t) * a.slots + c) * a.world;
    // children that are leaves have nothing to signal: their buffers are the inputs
    uint32_t *w0 = (c0 >= 0 && a.height[t][c0] > 0) ? a.pad[rank] + slot + c0 : nullptr;
    uint32_t *w1 = (c1 >= 0 && a.height[t][c1] > 0) ? a.pad[rank] + slot + c1 : nullptr;
    if (!wait_signals(w0, w1, a.spin_limit, a.ctl, a.report, lds_ok)) return false;

    const size_t off = a.half_off[t] + static_cast<size_t>(c) * a.chunk_bytes;
    const size_t left = a.half_bytes[t] - static_cast<size_t>(c) * a.chunk_bytes;
    const uint32_t bytes = left < a.chunk_bytes ? static_cast<uint32_t>(left) : a.chunk_bytes;
    char *own = a.buf[rank];
    const bool top = h == a.tree_height;
    char *out = top ? a.out[rank] : nullptr;
    if (!top) {
        // an interior node of the perfect tree has both children
        const char *const src[3] = {a.buf[c0], a.buf[c1], own};
        char *const dst[1] = {own};
        reduce_chunk<Sum, VECS, 3, 1>(src, dst, off, bytes);
    } else {
        // the extra node has one child (tree.py:133-136)
        const char *const src[2] = {a.buf[c0], own};
        if (out != nullptr) {
            char *const dst[2] = {own, out};
            reduce_chunk<Sum, VECS, 2, 2>(src, dst, off, bytes);
        } else {
            char *const dst[1] = {own};
            reduce_chunk<Sum, VECS, 2, 1>(src, dst, off, bytes);
        }
    }
    if (!top) {
        send_signals(a.pad[parent] + slot + rank, nullptr);
    } else {
        // the result is final: start the down-sweep
        send_signals(a.pad[c0] + slot + rank, nullptr);
    }
    return true;
}

// Down-sweep step: own, output <- parent (triton_double_tree_allreduce.py:306-326), then
// tell the children.
template <int VECS>
__device__ __forceinline__ bool down_step(const PipeArgs &a, int rank, int t, uint32_t c, int *lds_ok)
{
    const int h = a.height[t][rank];
    if (h == a.tree_height) return true; // the extra node already holds and has written the result
    const int parent = a.nbr[t][rank][0], c0 = a.nbr[t][rank][1], c1 = a.nbr[t][rank][2];
    const uint32_t slot = (static_cast<uint32_t>(t) * a.slots + c) * a.world;
    if (!wait_signals(a.pad[rank] + slot + parent, nullptr, a.spin_limit, a.ctl, a.report, lds_ok)) return false;

    const size_t off = a.half_off[t] + static_cast<size_t>(c) * a.chunk_bytes;
    const size_t left = a.half_bytes[t] - static_cast<size_t>(c) * a.chunk_bytes;
    const uint32_t bytes = left < a.chunk_bytes ? static_cast<uint32_t>(left) : a.chunk_bytes;
    if (a.out[rank] != nullptr) {
        char *const dst[2] = {a.buf[rank], a.out[rank]};
        copy_chunk<VECS, 2>(a.buf[parent], dst, off, bytes);
    } else {
        char *const dst[1] = {a.buf[rank]};
        copy_chunk<VECS, 1>(a.buf[parent], dst, off, bytes);
    }
    if (c0 >= 0 || c1 >= 0)
        send_signals(c0 >= 0 ? a.pad[c0] + slot + rank : nullptr, c1 >= 0 ? a.pad[c1] + slot + rank : nullptr);
    return true;
}

// Workgroup g of a rank's wgs_per_rank takes chunks g, g + wgs_per_rank, ... of both trees.
// In round i it runs the up-sweep steps of its i-th chunk and the down-sweep steps of its
// (i - lag)-th.  Every rank's workgroup g walks the same chunks in the same order, and a
// step only waits for steps of the same chunk that sit at the same or an earlier place in
// the other ranks' order (up-sweep: lower tree levels; down-sweep: the levels above, ending
// at the extra node's up-sweep step), so among the workgroups with the same g nothing waits in
// a circle, and those are the only workgroups a workgroup ever waits for (see take_place).
template <class Sum, int VECS>
__device__ __forceinline__ void tree_pipelined_walk(const PipeArgs &a, int rank, uint32_t g, int *lds_ok)
{
    const uint32_t G = a.wgs_per_rank;
    const uint32_t most = a.nchunks[0] > a.nchunks[1] ? a.nchunks[0] : a.nchunks[1];
    if (g >= most) return; // (the same workgroups in every rank's launch)
    // One launch per rank with the reference's leading barrier inside (the double tree's kernel
    // begins with blockwise_barrier, triton_double_tree_allreduce.py:239): every rank's input is
    // in place before anybody reads a leaf's buffer.  The trailing barrier (row 512 + g) tells the
    // peers that this workgroup has taken every flag and read every chunk it ever will, so buffers
    // and pads are free for the next collective when the kernel has ended.  Two rows in turn, as
    // in the one-shot kernels.
    const bool own_barriers = a.only_rank >= 0 && a.own_barriers != 0;
    if (own_barriers) {
        if (threadIdx.x == 0) *lds_ok = 1;
        if (!barrier_on_slots(a.pad, a.world, rank, a.barrier_base + g * a.world, a.spin_limit, a.ctl, a.report, lds_ok))
            return;
        __syncthreads(); // wait_signals rewrites lds_ok
    }
    const uint32_t rounds = (most - g + G - 1) / G;
    const uint32_t lag = a.lag;
    for (uint32_t i = 0; i < rounds + lag; ++i) {
        if (i < rounds) {
            const uint32_t c = g + i * G;
            for (int t = 0; t < 2; ++t)
                if (c < a.nchunks[t] && !up_step<Sum, VECS>(a, rank, t, c, lds_ok)) return;
        }
        if (i >= lag) {
            const uint32_t c = g + (i - lag) * G;
            for (int t = 0; t < 2; ++t)
                if (c < a.nchunks[t] && !down_step<VECS>(a, rank, t, c, lds_ok)) return;
        }
    }
    if (own_barriers) {
        __syncthreads();
        if (threadIdx.x == 0) *lds_ok = 1;
        // (the second block of rows starts at a fixed row, not at G: calls with different G share the pads)
        const uint32_t row = static_cast<uint32_t>(kTreeBarrierWorkgroups) + g;
        (void)barrier_on_slots(a.pad, a.world, rank, a.barrier_base + row * a.world, a.spin_limit, a.ctl, a.report, lds_ok);
    }
}

template <class Sum, int VECS>
__global__ void __launch_bounds__(kPhasedBlock) tree_pipelined_kernel(PipeArgs a)
{
    __shared__ int lds_ok;
    __shared__ uint32_t lds_place[2];
    int rank;
    uint32_t g;
    if (a.only_rank >= 0) {
        // one launch per rank (the reference's form: every rank runs its own kernel and meets the
        // others through the pads): the grid is this rank's workgroups
        rank = a.only_rank;
        g = blockIdx.x;
    } else {
        take_place(a.ctl, a.draw != 0, a.world, a.wgs_per_rank, &rank, &g, lds_place);
    }
    if (g != kNoPlace) tree_pipelined_walk<Sum, VECS>(a, rank, g, &lds_ok);
}

// Workgroups per rank for `units` units of work (chunks, tiles) per rank, at most `most`.
// Workgroup g takes units g, g + G, ...
//
// First choice: a count that gives every compute unit the same number of workgroups (G * world a
// multiple of the units: 96, 128 or 160 per rank for a world of 8 on 256 units), at least three
// per unit.  The hardware deals a grid out to the units evenly, so with any other count some
// units carry one workgroup more than the rest and the launch lasts as long as they do: for the
// two-shot all-reduce of 8 x 64 MiB, 128 per rank took 208 us, 120 took 222, 112 230, 104 241
// and 103 (which wastes no workgroup-round on 513 tiles) 260.  Among the balanced counts the
// one with the fewest unit-slots on the busiest compute unit wins -- per unit, workgroups x
// full rounds, plus the partial last round -- then one that divides `units` exactly (128 for
// 1,024 chunks), then the smaller or the larger as the kernel likes it (the two-shot kernel is
// as fast with three workgroups per unit as with four and loses less in a partial last round:
// 213 against 224 us for 513 tiles; the pipelined tree wants the most workgroups it can get: 96
// per rank measured 10-15 % slower than 128 or 160).  Such counts are multiples of 8 per rank for worlds of 2, 4
// and 8, so workgroup g of every rank shares an XCD and its L2 (workgroups go to the 8 XCDs
// round-robin), and part of what a rank reads from a peer right after the peer wrote it never
// leaves the XCD (8 % of the pipelined tree's reads and 29 % of the two-shot's, by the fetch
// counters).
// Where no balanced count fits (worlds of 5 and 7): the count from 60 % of `most` upwards that
// wastes the fewest workgroup-rounds, ties to a multiple of 8 and then to the larger.
static size_t workgroups_per_rank(size_t units, size_t most, int world, bool ties_to_larger)
{
    if (most < 1) most = 1;
    if (units <= most) return units < 1 ? 1 : units;
    const size_t cus = static_cast<size_t>(compute_units());
    const size_t w = static_cast<size_t>(world < 1 ? 1 : world);
    size_t a = w, b = cus; // greatest common divisor
    while (b != 0) {
        const size_t t = a % b;
        a = b;
        b = t;
    }
    const size_t step = cus / (a > 0 ? a : 1);
    size_t best = 0, best_cost = static_cast<size_t>(-1);
    bool best_exact = false;
    for (size_t g = step; step > 0 && g <= most; g += step) {
        const size_t per_cu = g * w / cus;
        if (per_cu < 3 && g + step <= most) continue; // too few waves to keep the memory system busy
        const size_t full = units / g, rem = units % g;
        const size_t last = (rem * w + cus - 1) / cus;
        const size_t cost = per_cu * full + (last < per_cu ? last : per_cu);
        const bool exact = rem == 0;
        if (cost < best_cost || (cost == best_cost && (exact != best_exact ? exact : ties_to_larger))) {
            best = g;
            best_cost = cost;
            best_exact = exact;
        }
    }
    if (best != 0) return best;
    best = most;
    size_t best_score = static_cast<size_t>(-1);
    const size_t least = most * 6 / 10 > 0 ? most * 6 / 10 : 1;
    for (size_t g = most; g >= least; --g) {
        const size_t rounds = (units + g - 1) / g;
        const size_t score = (rounds * g - units) * 2 + (g % kNumXcd != 0 ? 1 : 0);
        if (score < best_score) {
            best_score = score;
            best = g;
        }
    }
    return best;
}

// Workgroups of kernel `k` that fit the device at once.
// The hardware hands a grid's workgroups to the 8 XCDs round-robin and, inside an XCD, to its
// 32 compute units round-robin (read back from the hardware-id register of every workgroup
// of grids of 4 and 6 per unit: every unit got exactly its share), so a grid of
// per_cu * units workgroups is resident as a whole once earlier work has left the units.
// With the registers the signalling kernels need that is 2 to 5 per unit.  Never more than 6:
// a signalling grid of 8 per unit once timed out for a reason that was never established, so
// that shape stays unreachable whatever a kernel's register use becomes.
//
// separate_launches: the workgroups that wait for each other belong to different launches (one
// per rank, from different processes), which arrive at different times behind other kernels.  Then
// the occupancy the runtime reports cannot be relied on.  Measured with 8 processes at the
// reported 4 per unit, each rank's collective behind an elementwise kernel of its own: the last
// rank's launch got 2 of its 128 workgroups placed, and the other 896, which left room for 126
// more by the runtime's count, waited for the rest until their waits expired.  The explanation
// that fits: a wave's registers are one contiguous block of its SIMD's 512, the short-lived waves
// of the other kernels that come and go between the arrivals leave the waiting waves scattered
// over the file, and the holes between them may each be too small for the late launch's waves
// although their sum is not.  With n waves of v
// registers per SIMD wanted, n - 1 badly placed ones leave a hole of at least
// (512 - (n - 1) v) / n, which holds the n-th for n <= (512 + v) / (2 v): half the reported
// figure, rounded up.  Only as many workgroups as that are launched, so the last arrival
// always finds room.
template <class K>
static int resident_for(K kernel, bool separate_launches = false)
{
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kPhasedBlock, 0) != hipSuccess || per_cu < 1) return 0;
    if (per_cu > kMaxSignallingPerUnit) per_cu = kMaxSignallingPerUnit;
    if (separate_launches) per_cu = (per_cu + 1) / 2;
    return per_cu * compute_units();
}

template <class Sum, int VECS>
static int launch_pipelined(const PipeArgs &a, int wgs_wanted, int world, size_t slots, hipStream_t s)
{
    // asked once per kernel: the answer depends on the kernel's register use only
    static std::once_flag once;
    static int resident_one = 0, resident_per_rank = 0;
    std::call_once(once, [] {
        resident_one = resident_for(tree_pipelined_kernel<Sum, VECS>);
        resident_per_rank = resident_for(tree_pipelined_kernel<Sum, VECS>, true);
    });
    // Every workgroup must be resident: the grid never exceeds what the runtime says fits -- or, where
    // the ranks' launches come from different processes at different times, what always finds room.
    const int resident = a.only_rank >= 0 ? resident_per_rank : resident_one;
    if (resident < world) return hip_code(hipErrorLaunchOutOfResources);
    int per_rank;
    if (wgs_wanted > 0) {
        per_rank = (wgs_wanted < resident ? wgs_wanted : resident) / world;
        if (per_rank < 1) per_rank = 1;
        if (static_cast<size_t>(per_rank) > slots) per_rank = static_cast<int>(slots);
    } else {
        per_rank = static_cast<int>(workgroups_per_rank(slots, static_cast<size_t>(resident / world), world, true));
    }
    if (a.own_barriers && static_cast<size_t>(per_rank) > kTreeBarrierWorkgroups) per_rank = static_cast<int>(kTreeBarrierWorkgroups);
    PipeArgs args = a;
    args.wgs_per_rank = per_rank;
    SignallingLaunch guard(s);
    const int ranks_in_launch = a.only_rank >= 0 ? 1 : world;
    hipLaunchKernelGGL((tree_pipelined_kernel<Sum, VECS>), dim3(static_cast<unsigned>(per_rank * ranks_in_launch)),
                       dim3(kPhasedBlock), 0, s, args);
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) guard.launched();
    return hip_code(e);
}

template <class Sum>
static int launch_pipelined_tile(const PipeArgs &a, int tile_kib, int wgs_wanted, int world, size_t slots,
                                 hipStream_t s)
{
    switch (tile_kib) {
    case 128: return launch_pipelined<Sum, 32>(a, wgs_wanted, world, slots, s);
    default: return launch_pipelined<Sum, 8>(a, wgs_wanted, world, slots, s);
    }
}

static bool pow2_small_world(int world) { return world == 2 || world == 4 || world == 8; }

struct PipeGeometry {
    size_t per_vec, split, chunk_bytes;
    size_t half_bytes[2];
    size_t nchunks[2];
    size_t slots; // chunk slots per tree
};

static int pipe_geometry(int world, size_t numel, int dtype, size_t chunk_elems, PipeGeometry *g)
{
    const int esize = dtype_size(dtype);
    if (esize == 0) return TCCL_EINVAL;
    if (!pow2_small_world(world)) return (world >= 2 && (world & (world - 1)) == 0) ? TCCL_EINVAL : TCCL_EPOW2;
    g->per_vec = kVecBytes / esize;
    if (numel % g->per_vec != 0) return TCCL_EALIGN;
    g->split = tccl_double_tree_split(numel, esize);
    g->half_bytes[0] = g->split * esize;
    g->half_bytes[1] = (numel - g->split) * esize;
    if (chunk_elems == 0) {
        // 32 KiB (one tile per signal: 1.58 ms against 1.67 ms with 128 KiB chunks for
        // 8 x 256 MiB; 16 KiB chunks lose again), halved (down to 4 KiB) while a tree has
        // fewer than 256 chunks: a chunk crosses up to 2*log2(world) dependent steps, so a
        // small input needs many small chunks in flight, not a few large ones
        size_t bytes = 32u * 1024u;
        while (bytes > 4096 && g->half_bytes[1] / bytes < 256) bytes /= 2;
        chunk_elems = bytes / esize;
    }
    if (chunk_elems % g->per_vec != 0) return TCCL_EALIGN;
    g->chunk_bytes = chunk_elems * esize;
    if (g->chunk_bytes > (static_cast<size_t>(1) << 30)) return TCCL_EINVAL;
    for (int t = 0; t < 2; ++t) g->nchunks[t] = (g->half_bytes[t] + g->chunk_bytes - 1) / g->chunk_bytes;
    g->slots = g->nchunks[0] > g->nchunks[1] ? g->nchunks[0] : g->nchunks[1];
    if (g->slots > 0x0FFFFFFFu) return TCCL_EINVAL;
    return TCCL_OK;
}

} // namespace tccl

using namespace tccl;

extern "C" size_t tccl_double_tree_signal_pad_bytes(int world, size_t numel, int dtype, size_t chunk_elems)
{
    PipeGeometry g;
    if (pipe_geometry(world, numel, dtype, chunk_elems, &g) != TCCL_OK) return 0;
    // two trees x slots x world flags, two rows of barrier slots for up to kTreeBarrierWorkgroups
    // workgroups per rank (used by the per-rank launch with TCCL_PIPE_OWN_BARRIERS), then the control
    // words; rounded up to 16 bytes
    const size_t words = (2 * g.slots + 2 * kTreeBarrierWorkgroups) * static_cast<size_t>(world) + kCtlWords;
    return (words * sizeof(uint32_t) + 15) / 16 * 16;
}

// Both forms of the pipelined double tree: only_rank < 0 -- one launch holding every rank's
// workgroups, outs = W outputs or null; only_rank >= 0 -- that rank's launch, outs[only_rank]
// its output (the other entries are not read).
static int pipelined_double_tree(void *const *bufs, void *const *outs, void *const *signal_pads, size_t pad_bytes,
                                 int world, int only_rank, size_t numel, int dtype, size_t chunk_elems,
                                 const tccl_pipeline_cfg *cfg, void *stream)
{
    if (bufs == nullptr || signal_pads == nullptr) return TCCL_EINVAL;
    PipeGeometry g;
    int rc = pipe_geometry(world, numel, dtype, chunk_elems, &g);
    if (rc != TCCL_OK) return rc;
    const size_t need = tccl_double_tree_signal_pad_bytes(world, numel, dtype, chunk_elems);
    if (pad_bytes < need) return TCCL_EINVAL;
    for (int r = 0; r < world; ++r) {
        if (bufs[r] == nullptr || signal_pads[r] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[r]) || !aligned16(signal_pads[r]) || (outs && !aligned16(outs[r]))) return TCCL_EALIGN;
    }
    if (numel == 0) return TCCL_OK;

    PipeArgs a = {};
    int height = 0;
    while ((1 << height) < world) ++height;
    a.tree_height = height;
    for (int r = 0; r < world; ++r) {
        a.buf[r] = static_cast<char *>(bufs[r]);
        a.out[r] = outs ? static_cast<char *>(outs[r]) : nullptr;
        a.pad[r] = static_cast<uint32_t *>(signal_pads[r]);
        int six[6];
        rc = tccl_double_tree_indices(world, r, six);
        if (rc != TCCL_OK) return rc;
        for (int t = 0; t < 2; ++t) {
            for (int k = 0; k < 3; ++k) a.nbr[t][r][k] = static_cast<signed char>(six[3 * t + k]);
            const int ra = (t == 0) ? r : (r + 1) % world; // the rank's label in tree a's numbering
            a.height[t][r] = static_cast<signed char>(ra == 0 ? height : __builtin_ctz(ra));
        }
    }
    const int esize = dtype_size(dtype);
    a.half_off[0] = 0;
    a.half_off[1] = g.split * esize;
    for (int t = 0; t < 2; ++t) {
        a.half_bytes[t] = g.half_bytes[t];
        a.nchunks[t] = static_cast<uint32_t>(g.nchunks[t]);
    }
    a.chunk_bytes = static_cast<uint32_t>(g.chunk_bytes);
    a.slots = static_cast<uint32_t>(g.slots);
    a.world = world;
    a.only_rank = only_rank;
    a.own_barriers = (only_rank >= 0 && cfg && (cfg->flags & TCCL_PIPE_OWN_BARRIERS)) ? 1 : 0;
    a.barrier_base = static_cast<uint32_t>(2 * g.slots * static_cast<size_t>(world));
    a.draw = (only_rank < 0 && cfg && (cfg->flags & TCCL_PIPE_DRAW_PLACES)) ? 1 : 0;
    a.ctl = a.pad[0] + pad_bytes / sizeof(uint32_t) - kCtlWords; // the last words of pad 0
    a.report = cfg ? cfg->timeout_flag : nullptr;
    a.spin_limit = (cfg && cfg->spin_limit > 0) ? cfg->spin_limit : kPipeDefaultSpins;
    a.lag = (cfg && cfg->lag > 0) ? cfg->lag - 1 : 0; // cfg->lag is 1-based so that 0 means "default"
    if (a.lag > 64) a.lag = 64;

    hipStream_t s = static_cast<hipStream_t>(stream);
    const int tile_kib = cfg ? cfg->tile_kib : 0;
    const int wgs = cfg ? cfg->workgroups : 0;
    return dtype == TCCL_BF16 ? launch_pipelined_tile<Bf16Sum>(a, tile_kib, wgs, world, g.slots, s)
                              : launch_pipelined_tile<F32Sum>(a, tile_kib, wgs, world, g.slots, s);
}

extern "C" int tccl_double_tree_all_reduce_pipelined(void *const *bufs, void *const *outs, void *const *signal_pads,
                                                     size_t pad_bytes, int world, size_t numel, int dtype,
                                                     size_t chunk_elems, const tccl_pipeline_cfg *cfg, void *stream)
{
    return pipelined_double_tree(bufs, outs, signal_pads, pad_bytes, world, -1, numel, dtype, chunk_elems, cfg, stream);
}

extern "C" int tccl_double_tree_all_reduce_pipelined_rank(void *const *bufs, void *out, void *const *signal_pads,
                                                          size_t pad_bytes, int world, int rank, size_t numel,
                                                          int dtype, size_t chunk_elems, const tccl_pipeline_cfg *cfg,
                                                          void *stream)
{
    if (rank < 0 || rank >= world || world > TCCL_MAX_WORLD) return TCCL_EINVAL;
    if (cfg && (cfg->flags & TCCL_PIPE_DRAW_PLACES)) return TCCL_EINVAL; // places are fixed by the rank's own launch
    void *outs[TCCL_MAX_WORLD] = {};
    outs[rank] = out;
    return pipelined_double_tree(bufs, out ? outs : nullptr, signal_pads, pad_bytes, world, rank, numel, dtype,
                                 chunk_elems, cfg, stream);
}

extern "C" int tccl_signal_pad_timeouts(const void *pad0, size_t pad_bytes, unsigned *timeouts_out, void *stream)
{
    if (pad0 == nullptr || timeouts_out == nullptr || pad_bytes < 16 || pad_bytes % 16 != 0) return TCCL_EINVAL;
    const uint32_t *status = static_cast<const uint32_t *>(pad0) + pad_bytes / sizeof(uint32_t) - 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    uint32_t v = 0;
    hipError_t e = hipMemcpyAsync(&v, status, sizeof(v), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_code(e);
    *timeouts_out = v;
    return TCCL_OK;
}

// ------------------------------------------------------------------ two-shot all-reduce, one launch
namespace tccl {

struct TwoShotArgs {
    char *buf[kPipeMaxWorld];
    char *out[kPipeMaxWorld]; // entries may be null
    uint32_t *pad[kPipeMaxWorld];
    size_t share_bytes; // bytes of one rank's share (multiple of 16)
    uint32_t spin_limit;
    int world, wgs_per_rank;
    int draw;         // 1 = workgroups draw their places when they start, 0 = places follow the hardware index
    int only_rank;    // >= 0: the launch holds this rank's workgroups only (one launch per rank); -1: all ranks'
    int own_barriers; // one launch per rank: the kernel also begins and ends with the blockwise barrier
    uint32_t rows;    // own_barriers: rows of one barrier's block of the pad (fixed by the pad's size, not by G)
    uint32_t *ctl;    // control words at the end of pad 0 (place counters ... time-outs)
    uint32_t *report; // optional host word set to 1 when a wait expires
};

// The blockwise barrier of workgroup g on row `row` of the pads (barrier_on_slots).
__device__ __forceinline__ bool blockwise_barrier(const TwoShotArgs &a, int rank, uint32_t row, int *lds_ok)
{
    return barrier_on_slots(a.pad, a.world, rank, row * static_cast<uint32_t>(a.world), a.spin_limit, a.ctl, a.report, lds_ok);
}

// Rank r's workgroup g of G:
//   shot 1  reduces tiles g, g+G, ... of share r from all W buffers, in rank order, into its
//           own buffer in place (and its output);
//   barrier with workgroup g of every other rank;
//   shot 2  copies the same tiles of every other share s from rank s's buffer -- exactly the
//           tiles that rank s's workgroup g reduced, which is why a barrier between
//           workgroups of equal index is enough -- into its own buffer and its output.
// Every buffer ends up holding the whole all-reduce, as after the double tree.
// Tiles are 16 KiB (4 vectors per lane): with four workgroups per compute unit that measured
// 2-10 % faster than 128 KiB tiles at 64 MiB per buffer and several times faster on small
// inputs, whose shares it spreads over many more workgroups.
constexpr int kTwoShotVecs = 4;

//
// PEERS_MAY_STILL_WRITE (one launch per rank): the kernel may have started before a peer's
// producer kernel ended, so shot 1 reads with device-scope loads too; and with a.own_barriers
// the kernel begins with the barrier that says "every rank's input is in place" (row R + g of
// the pads) and ends with the one that says "every rank has read what it needs from every
// buffer" (row 2 R + g) -- three barriers in a row on three different rows, so a flag is never
// raised over one that its reader has not consumed, within a call and from call to call.  R is
// a third of the pad's rows whatever G is: a call with more workgroups than the one before it
// (a larger input) must find workgroup g's rows where the last call left them, or its leading
// flags would land on trailing flags of the last call that a slower peer has yet to take.
template <class Sum, int W, bool PEERS_MAY_STILL_WRITE>
__device__ __forceinline__ void two_shot_body(const TwoShotArgs &a, int rank, uint32_t g, int &lds_ok)
{
    constexpr int VECS = kTwoShotVecs;
    constexpr int LAUX = PEERS_MAY_STILL_WRITE ? kAuxLoadDevice : kAuxLoadStream;
    constexpr int U = PhasedUnroll<W>::value < VECS ? PhasedUnroll<W>::value : VECS;
    constexpr int KMAX = VECS / U;
    constexpr uint32_t span = kPhasedBlock * U * kVecBytes;
    constexpr uint32_t tile_bytes = kPhasedBlock * VECS * kVecBytes;
    const uint32_t G = a.wgs_per_rank;
    if (threadIdx.x == 0) lds_ok = 1;
    // (the barrier's first __syncthreads orders this store before any lane's clear)
    const bool own_barriers = PEERS_MAY_STILL_WRITE && W > 1 && a.own_barriers != 0;
    if (own_barriers && !blockwise_barrier(a, rank, a.rows + g, &lds_ok)) return;

    const char *src[W];
#pragma unroll
    for (int i = 0; i < W; ++i) src[i] = a.buf[i];
    const char *const(&csrc)[W] = src;
    const size_t share_off = static_cast<size_t>(rank) * a.share_bytes;
    for (size_t t = static_cast<size_t>(g) * tile_bytes; t < a.share_bytes; t += static_cast<size_t>(G) * tile_bytes) {
        const size_t left = a.share_bytes - t;
        const uint32_t valid = left < tile_bytes ? static_cast<uint32_t>(left) : tile_bytes;
        const int kcount = static_cast<int>((valid + span - 1) / span);
        const bool full = valid == tile_bytes;
        if (a.out[rank] != nullptr) {
            char *const dst[2] = {a.buf[rank], a.out[rank]};
            if (full)
                sum_tile_phased<Sum, W, 2, U, KMAX, true, Sum::kPaceLoads, LAUX>(csrc, dst, share_off + t, valid, KMAX);
            else
                sum_tile_phased<Sum, W, 2, U, KMAX, false, Sum::kPaceLoads, LAUX>(csrc, dst, share_off + t, valid, kcount);
        } else {
            char *const dst[1] = {a.buf[rank]};
            if (full)
                sum_tile_phased<Sum, W, 1, U, KMAX, true, Sum::kPaceLoads, LAUX>(csrc, dst, share_off + t, valid, KMAX);
            else
                sum_tile_phased<Sum, W, 1, U, KMAX, false, Sum::kPaceLoads, LAUX>(csrc, dst, share_off + t, valid, kcount);
        }
    }
    if (W == 1) return;
    if (!blockwise_barrier(a, rank, g, &lds_ok)) return;

    for (int i = 1; i < W; ++i) {
        const int s = (rank + i) % W; // start at a different peer per rank
        const size_t off = static_cast<size_t>(s) * a.share_bytes;
        for (size_t t = static_cast<size_t>(g) * tile_bytes; t < a.share_bytes;
             t += static_cast<size_t>(G) * tile_bytes) {
            const size_t left = a.share_bytes - t;
            const uint32_t valid = left < tile_bytes ? static_cast<uint32_t>(left) : tile_bytes;
            constexpr uint32_t cspan = kPhasedBlock * 4 * kVecBytes;
            const int kcount = static_cast<int>((valid + cspan - 1) / cspan);
            if (a.out[rank] != nullptr) {
                char *const dst[2] = {a.buf[rank], a.out[rank]};
                copy_tile_phased<2, 4, VECS / 4, kAuxLoadDevice>(a.buf[s], dst, off + t, valid, kcount);
            } else {
                char *const dst[1] = {a.buf[rank]};
                copy_tile_phased<1, 4, VECS / 4, kAuxLoadDevice>(a.buf[s], dst, off + t, valid, kcount);
            }
        }
    }
    if (own_barriers) (void)blockwise_barrier(a, rank, 2 * a.rows + g, &lds_ok);
}

template <class Sum, int W>
__global__ void __launch_bounds__(kPhasedBlock) two_shot_kernel(TwoShotArgs a)
{
    __shared__ int lds_ok;
    __shared__ uint32_t lds_place[2];
    int rank;
    uint32_t g;
    take_place(a.ctl, a.draw != 0, W, a.wgs_per_rank, &rank, &g, lds_place);
    if (g != kNoPlace) two_shot_body<Sum, W, false>(a, rank, g, lds_ok);
}

// One launch per rank: the barrier between the shots is then the reference's own construct, a
// barrier between the kernels of different owners.
template <class Sum, int W>
__global__ void __launch_bounds__(kPhasedBlock) two_shot_rank_kernel(TwoShotArgs a)
{
    __shared__ int lds_ok;
    two_shot_body<Sum, W, true>(a, a.only_rank, blockIdx.x, lds_ok);
}

// What the entry point without caller-owned pads asks for before its kernel: zero the first
// flag_words words of each of `pads` pads of pad_words words starting at base, and the
// control words.
struct ClearRequest {
    uint32_t *base;
    uint32_t pad_words, flag_words;
    int pads;
};

// Zeroes the first `flag_words` words of each of the gridDim.y pads and the control words at
// the end of pad 0.  (A fill kernel, not a memset node: this entry point is meant to be
// recorded into graphs.)
__global__ void __launch_bounds__(kPhasedBlock) clear_pads_kernel(uint32_t *base, uint32_t pad_words, uint32_t flag_words)
{
    uint32_t *pad = base + static_cast<size_t>(blockIdx.y) * pad_words;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < flag_words; i += gridDim.x * blockDim.x)
        __hip_atomic_store(pad + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (blockIdx.x == 0 && blockIdx.y == 0)
        for (uint32_t i = threadIdx.x; i < kCtlWords; i += blockDim.x)
            __hip_atomic_store(base + pad_words - kCtlWords + i, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <class Sum, int W>
static int launch_two_shot(TwoShotArgs a, int wgs_wanted, size_t pad_words, const ClearRequest *clear, hipStream_t s)
{
    static std::once_flag once;
    static int resident_one = 0, resident_rank = 0;
    std::call_once(once, [] {
        resident_one = resident_for(two_shot_kernel<Sum, W>);
        resident_rank = resident_for(two_shot_rank_kernel<Sum, W>, true);
    });
    const int resident = a.only_rank < 0 ? resident_one : resident_rank;
    if (resident < W) return hip_code(hipErrorLaunchOutOfResources);
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * kTwoShotVecs * kVecBytes;
    const size_t tiles = (a.share_bytes + tile_bytes - 1) / tile_bytes;
    // one slot per (workgroup index, sender) in every pad -- three with the kernel's own leading and
    // trailing barriers; the last words of pad 0 are the control words
    const size_t fit = (pad_words - kCtlWords) / (static_cast<size_t>(W) * (a.own_barriers ? 3 : 1));
    if (fit < 1) return TCCL_EINVAL;
    a.rows = static_cast<uint32_t>(fit);
    size_t per_rank;
    if (wgs_wanted > 0) {
        per_rank = static_cast<size_t>((wgs_wanted < resident ? wgs_wanted : resident) / W);
        if (per_rank < 1) per_rank = 1;
        if (per_rank > tiles) per_rank = tiles;
        if (per_rank > fit) per_rank = fit;
    } else {
        const size_t most = static_cast<size_t>(resident / W);
        per_rank = workgroups_per_rank(tiles, most < fit ? most : fit, W, false);
    }
    a.wgs_per_rank = static_cast<int>(per_rank);
    SignallingLaunch guard(s); // from here on the stream is behind the device's previous signalling kernel
    if (clear != nullptr) {
        const dim3 cgrid((clear->flag_words + kPhasedBlock * 4 - 1) / (kPhasedBlock * 4), clear->pads);
        hipLaunchKernelGGL(clear_pads_kernel, cgrid, dim3(kPhasedBlock), 0, s, clear->base, clear->pad_words,
                           clear->flag_words);
        const hipError_t ce = hipGetLastError();
        if (ce != hipSuccess) return hip_code(ce);
    }
    if (a.only_rank >= 0)
        hipLaunchKernelGGL((two_shot_rank_kernel<Sum, W>), dim3(static_cast<unsigned>(per_rank)), dim3(kPhasedBlock), 0, s, a);
    else
        hipLaunchKernelGGL((two_shot_kernel<Sum, W>), dim3(static_cast<unsigned>(per_rank * W)), dim3(kPhasedBlock), 0, s, a);
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) guard.launched();
    return hip_code(e);
}

template <class Sum>
static int launch_two_shot_world(const TwoShotArgs &a, int wgs_wanted, size_t pad_words, const ClearRequest *clear,
                                 hipStream_t s)
{
    switch (a.world) {
    case 1: return launch_two_shot<Sum, 1>(a, wgs_wanted, pad_words, clear, s);
    case 2: return launch_two_shot<Sum, 2>(a, wgs_wanted, pad_words, clear, s);
    case 3: return launch_two_shot<Sum, 3>(a, wgs_wanted, pad_words, clear, s);
    case 4: return launch_two_shot<Sum, 4>(a, wgs_wanted, pad_words, clear, s);
    case 5: return launch_two_shot<Sum, 5>(a, wgs_wanted, pad_words, clear, s);
    case 6: return launch_two_shot<Sum, 6>(a, wgs_wanted, pad_words, clear, s);
    case 7: return launch_two_shot<Sum, 7>(a, wgs_wanted, pad_words, clear, s);
    case 8: return launch_two_shot<Sum, 8>(a, wgs_wanted, pad_words, clear, s);
    default: return TCCL_EINVAL;
    }
}

// Argument checks shared by the two entry points of the two-shot all-reduce (everything but
// the signal pads).  TCCL_OK means "launch"; *nothing_to_do is set for an empty input.
static int two_shot_check(void *const *bufs, void *const *outs, int world, size_t numel, int dtype, bool *nothing_to_do)
{
    *nothing_to_do = false;
    const int esize = dtype_size(dtype);
    if (esize == 0 || bufs == nullptr || world < 1 || world > TCCL_MAX_WORLD) return TCCL_EINVAL;
    const size_t per_vec = kVecBytes / esize;
    if (numel % (per_vec * world) != 0) return TCCL_EALIGN; // every share is whole vectors
    for (int r = 0; r < world; ++r) {
        if (bufs[r] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[r]) || (outs && !aligned16(outs[r]))) return TCCL_EALIGN;
    }
    *nothing_to_do = numel == 0;
    return TCCL_OK;
}

// The launch itself: `pads` are the W signal pads (device addresses), each of pad_bytes.
static int two_shot_launch(void *const *bufs, void *const *outs, uint32_t *const *pads, size_t pad_bytes, int world,
                           size_t numel, int dtype, const tccl_pipeline_cfg *cfg, const ClearRequest *clear, hipStream_t s,
                           int only_rank = -1)
{
    TwoShotArgs a = {};
    for (int r = 0; r < world; ++r) {
        a.buf[r] = static_cast<char *>(bufs[r]);
        a.out[r] = outs ? static_cast<char *>(outs[r]) : nullptr;
        a.pad[r] = pads[r];
    }
    a.share_bytes = numel / world * dtype_size(dtype);
    a.world = world;
    a.spin_limit = (cfg && cfg->spin_limit > 0) ? cfg->spin_limit : kPipeDefaultSpins;
    const size_t pad_words = pad_bytes / sizeof(uint32_t);
    a.ctl = a.pad[0] + pad_words - kCtlWords;
    a.report = cfg ? cfg->timeout_flag : nullptr;
    a.only_rank = only_rank;
    a.own_barriers = (only_rank >= 0 && cfg && (cfg->flags & TCCL_PIPE_OWN_BARRIERS)) ? 1 : 0;
    a.draw = (only_rank < 0 && cfg && (cfg->flags & TCCL_PIPE_DRAW_PLACES)) ? 1 : 0;
    const int wgs = cfg ? cfg->workgroups : 0;
    return dtype == TCCL_BF16 ? launch_two_shot_world<Bf16Sum>(a, wgs, pad_words, clear, s)
                              : launch_two_shot_world<F32Sum>(a, wgs, pad_words, clear, s);
}

} // namespace tccl

extern "C" int tccl_two_shot_all_reduce(void *const *bufs, void *const *outs, void *const *signal_pads,
                                        size_t pad_bytes, int world, size_t numel, int dtype,
                                        const tccl_pipeline_cfg *cfg, void *stream)
{
    if (signal_pads == nullptr || world < 1 || world > TCCL_MAX_WORLD) return TCCL_EINVAL;
    if (pad_bytes % 16 != 0 || pad_bytes < (static_cast<size_t>(world) + kCtlWords) * sizeof(uint32_t))
        return TCCL_EINVAL;
    bool nothing = false;
    const int rc = two_shot_check(bufs, outs, world, numel, dtype, &nothing);
    if (rc != TCCL_OK) return rc;
    uint32_t *pads[TCCL_MAX_WORLD];
    for (int r = 0; r < world; ++r) {
        if (signal_pads[r] == nullptr) return TCCL_EINVAL;
        if (!aligned16(signal_pads[r])) return TCCL_EALIGN;
        pads[r] = static_cast<uint32_t *>(signal_pads[r]);
    }
    if (nothing) return TCCL_OK;
    return two_shot_launch(bufs, outs, pads, pad_bytes, world, numel, dtype, cfg, nullptr,
                           static_cast<hipStream_t>(stream));
}

extern "C" int tccl_two_shot_all_reduce_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes,
                                             int world, int rank, size_t numel, int dtype,
                                             const tccl_pipeline_cfg *cfg, void *stream)
{
    if (signal_pads == nullptr || world < 1 || world > TCCL_MAX_WORLD || rank < 0 || rank >= world) return TCCL_EINVAL;
    if (cfg && (cfg->flags & TCCL_PIPE_DRAW_PLACES)) return TCCL_EINVAL; // places are fixed by the rank's own launch
    const size_t rows = (cfg && (cfg->flags & TCCL_PIPE_OWN_BARRIERS)) ? 3 : 1;
    if (pad_bytes % 16 != 0 || pad_bytes < (rows * static_cast<size_t>(world) + kCtlWords) * sizeof(uint32_t))
        return TCCL_EINVAL;
    void *outs[TCCL_MAX_WORLD] = {};
    outs[rank] = out;
    bool nothing = false;
    const int rc = two_shot_check(bufs, out ? outs : nullptr, world, numel, dtype, &nothing);
    if (rc != TCCL_OK) return rc;
    uint32_t *pads[TCCL_MAX_WORLD];
    for (int r = 0; r < world; ++r) {
        if (signal_pads[r] == nullptr) return TCCL_EINVAL;
        if (!aligned16(signal_pads[r])) return TCCL_EALIGN;
        pads[r] = static_cast<uint32_t *>(signal_pads[r]);
    }
    if (nothing) return TCCL_OK;
    return two_shot_launch(bufs, out ? outs : nullptr, pads, pad_bytes, world, numel, dtype, cfg, nullptr,
                           static_cast<hipStream_t>(stream), rank);
}

// ------------------------------------------------------------------ one-shot collectives, one launch per rank
namespace tccl {

// The reference's one-shot kernels begin with blockwise_barrier inside the kernel
// (triton_one_shot_all_reduce_no_128.py:46, triton_all_gather.py:43, commented at
// triton_reduce_scatter.py:70): every rank launches its own kernel, whose workgroup g first
// meets workgroup g of every other rank's kernel ("your buffer is filled") and then pulls
// from all W buffers.  Here the same as one launch per rank over IPC-mapped buffers and pads,
// plus the barrier the reference lacks at the end ("I have read your buffer, refill it").
//
// The two barriers of a call use different rows of slots: row g for the leading one, row
// R + g for the trailing one, R = half the rows the pad holds -- fixed by the pad, not by the
// launch, so that workgroup g finds its rows in the same place in every call on the same pads
// whatever the calls' sizes and kinds.  (With R = this launch's workgroup count, a call with
// more workgroups than the one before it would raise leading flags on rows where a slower
// peer has yet to take the last call's trailing flags, and one of the two would be lost.)
// A rank raises its flag for barrier k+1 of a row only after
// it has passed barrier k of the other row, which its peer raises only after it has lowered
// the flag of barrier k of this row -- so a flag is never raised over one that has not been
// consumed, within a call and from call to call, without the sender having to wait for the
// slot to be lowered.
struct RankArgs {
    const char *src[kPipeMaxWorld]; // sums: every rank's buffer at the first byte this launch reduces; gather: every rank's buffer
    char *out;
    uint32_t *pad[kPipeMaxWorld];
    size_t bytes; // sums: bytes to reduce; gather: bytes per rank
    uint32_t spin_limit;
    int world, rank, wgs;
    uint32_t rows;    // R: the trailing barrier's first row
    uint32_t *ctl;    // control words at the end of pad 0 (time-outs)
    uint32_t *report; // optional host word set to 1 when a wait expires
};

// triton_barrier.py:39-142 between workgroup g of this launch and workgroup g of every other
// rank's launch, on row `row` of the pads.
__device__ __forceinline__ bool rank_barrier(const RankArgs &a, uint32_t row, int *lds_ok)
{
    return barrier_on_slots(a.pad, a.world, a.rank, row * static_cast<uint32_t>(a.world), a.spin_limit, a.ctl, a.report, lds_ok);
}

// 16 KiB tiles, as in the two-shot kernel: a rank has 1/W of the GPU's workgroup slots, and
// small tiles spread a small input over all of them.  (Tiles of 32, 64 and 128 KiB measured within
// 10 % of these either way at 1 to 256 MiB per buffer with 8 processes, which is the spread between
// two runs.)
constexpr int kRankVecs = 4;

// All-reduce (bytes = the whole buffer) and reduce-scatter (src offset to this rank's share,
// bytes = the share): out = sum over the W sources in rank order.  Loads are device-scope: a
// peer's producer kernel may have finished after this kernel started, so nothing read here
// may come from a line this XCD's L2 already holds.
template <class Sum, int W>
__global__ void __launch_bounds__(kPhasedBlock) sum_rank_kernel(RankArgs a)
{
    __shared__ int lds_ok;
    constexpr int VECS = kRankVecs;
    constexpr int U = PhasedUnroll<W>::value < VECS ? PhasedUnroll<W>::value : VECS;
    constexpr int KMAX = VECS / U;
    constexpr uint32_t span = kPhasedBlock * U * kVecBytes;
    constexpr uint32_t tile_bytes = kPhasedBlock * VECS * kVecBytes;
    const uint32_t g = blockIdx.x, G = a.wgs;
    if (threadIdx.x == 0) lds_ok = 1;
    if (W > 1 && !rank_barrier(a, g, &lds_ok)) return;

    const char *src[W];
#pragma unroll
    for (int i = 0; i < W; ++i) src[i] = a.src[i];
    const char *const(&csrc)[W] = src;
    char *const dst[1] = {a.out};
    for (size_t t = static_cast<size_t>(g) * tile_bytes; t < a.bytes; t += static_cast<size_t>(G) * tile_bytes) {
        const size_t left = a.bytes - t;
        const uint32_t valid = left < tile_bytes ? static_cast<uint32_t>(left) : tile_bytes;
        if (valid == tile_bytes)
            sum_tile_phased<Sum, W, 1, U, KMAX, true, false, kAuxLoadDevice>(csrc, dst, t, valid, KMAX);
        else
            sum_tile_phased<Sum, W, 1, U, KMAX, false, false, kAuxLoadDevice>(csrc, dst, t, valid,
                                                                              static_cast<int>((valid + span - 1) / span));
    }
    if (W > 1) (void)rank_barrier(a, a.rows + g, &lds_ok);
}

// All-gather: out[s] = rank s's buffer for every s, starting at a different peer per rank.
__global__ void __launch_bounds__(kPhasedBlock) gather_rank_kernel(RankArgs a)
{
    __shared__ int lds_ok;
    constexpr int VECS = kRankVecs;
    constexpr uint32_t span = kPhasedBlock * 4 * kVecBytes;
    constexpr uint32_t tile_bytes = kPhasedBlock * VECS * kVecBytes;
    const uint32_t g = blockIdx.x, G = a.wgs;
    if (threadIdx.x == 0) lds_ok = 1;
    if (a.world > 1 && !rank_barrier(a, g, &lds_ok)) return;
    for (int i = 0; i < a.world; ++i) {
        const int s = (a.rank + i) % a.world;
        char *const dst[1] = {a.out + static_cast<size_t>(s) * a.bytes};
        for (size_t t = static_cast<size_t>(g) * tile_bytes; t < a.bytes; t += static_cast<size_t>(G) * tile_bytes) {
            const size_t left = a.bytes - t;
            const uint32_t valid = left < tile_bytes ? static_cast<uint32_t>(left) : tile_bytes;
            copy_tile_phased<1, 4, VECS / 4, kAuxLoadDevice>(a.src[s], dst, t, valid, static_cast<int>((valid + span - 1) / span));
        }
    }
    if (a.world > 1) (void)rank_barrier(a, a.rows + g, &lds_ok);
}

// Every rank computes the same count from the same arguments: its launch takes 1/W of the
// workgroups that fit the device, so that all W launches can be resident together.
template <class K>
static int launch_rank_kernel(K kernel, int resident, RankArgs a, size_t tiles, int wgs_wanted, size_t pad_words,
                              hipStream_t s)
{
    if (resident < a.world) return hip_code(hipErrorLaunchOutOfResources);
    // two rows of slots (leading and trailing barrier), one slot per (workgroup, sender)
    const size_t fit = (pad_words - kCtlWords) / (2 * static_cast<size_t>(a.world));
    if (fit < 1) return TCCL_EINVAL;
    a.rows = static_cast<uint32_t>(fit);
    size_t most = static_cast<size_t>(resident / a.world);
    if (most > fit) most = fit;
    size_t per_rank;
    if (wgs_wanted > 0) { // as everywhere in tccl_pipeline_cfg: the total over all ranks
        per_rank = static_cast<size_t>(wgs_wanted) / static_cast<size_t>(a.world);
        if (per_rank > most) per_rank = most;
        if (per_rank > tiles) per_rank = tiles;
    } else {
        per_rank = workgroups_per_rank(tiles, most, a.world, false);
    }
    if (per_rank < 1) per_rank = 1;
    a.wgs = static_cast<int>(per_rank);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(per_rank)), dim3(kPhasedBlock), 0, s, a);
    return hip_code(hipGetLastError());
}

template <class Sum, int W>
static int launch_sum_rank_w(const RankArgs &a, size_t tiles, int wgs, size_t pad_words, hipStream_t s)
{
    // asked once per kernel: the answer depends on the kernel's register use only
    static std::once_flag once;
    static int resident = 0;
    std::call_once(once, [] { resident = resident_for(sum_rank_kernel<Sum, W>, true); });
    return launch_rank_kernel(sum_rank_kernel<Sum, W>, resident, a, tiles, wgs, pad_words, s);
}

template <class Sum>
static int launch_sum_rank(const RankArgs &a, size_t tiles, int wgs, size_t pad_words, hipStream_t s)
{
    switch (a.world) {
    case 1: return launch_sum_rank_w<Sum, 1>(a, tiles, wgs, pad_words, s);
    case 2: return launch_sum_rank_w<Sum, 2>(a, tiles, wgs, pad_words, s);
    case 3: return launch_sum_rank_w<Sum, 3>(a, tiles, wgs, pad_words, s);
    case 4: return launch_sum_rank_w<Sum, 4>(a, tiles, wgs, pad_words, s);
    case 5: return launch_sum_rank_w<Sum, 5>(a, tiles, wgs, pad_words, s);
    case 6: return launch_sum_rank_w<Sum, 6>(a, tiles, wgs, pad_words, s);
    case 7: return launch_sum_rank_w<Sum, 7>(a, tiles, wgs, pad_words, s);
    case 8: return launch_sum_rank_w<Sum, 8>(a, tiles, wgs, pad_words, s);
    default: return TCCL_EINVAL;
    }
}

// Checks and argument block shared by the three entry points.  `first_byte`: where in every
// buffer this launch starts to read.
static int rank_args(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes, int world, int rank,
                     size_t first_byte, size_t bytes, const tccl_pipeline_cfg *cfg, RankArgs *a)
{
    if (bufs == nullptr || out == nullptr || signal_pads == nullptr || world < 1 || world > TCCL_MAX_WORLD || rank < 0 ||
        rank >= world)
        return TCCL_EINVAL;
    if (cfg && (cfg->flags & TCCL_PIPE_DRAW_PLACES)) return TCCL_EINVAL; // places are fixed by the rank's own launch
    if (pad_bytes % 16 != 0 || pad_bytes < (2 * static_cast<size_t>(world) + kCtlWords) * sizeof(uint32_t)) return TCCL_EINVAL;
    if (!aligned16(out)) return TCCL_EALIGN;
    *a = RankArgs{};
    for (int r = 0; r < world; ++r) {
        if (bufs[r] == nullptr || signal_pads[r] == nullptr) return TCCL_EINVAL;
        if (!aligned16(bufs[r]) || !aligned16(signal_pads[r])) return TCCL_EALIGN;
        a->src[r] = static_cast<const char *>(bufs[r]) + first_byte;
        a->pad[r] = static_cast<uint32_t *>(signal_pads[r]);
    }
    a->out = static_cast<char *>(out);
    a->bytes = bytes;
    a->spin_limit = (cfg && cfg->spin_limit > 0) ? cfg->spin_limit : kPipeDefaultSpins;
    a->world = world;
    a->rank = rank;
    a->ctl = a->pad[0] + pad_bytes / sizeof(uint32_t) - kCtlWords;
    a->report = cfg ? cfg->timeout_flag : nullptr;
    return TCCL_OK;
}

static int sum_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes, int world, int rank,
                    size_t first_elem, size_t numel, int dtype, const tccl_pipeline_cfg *cfg, void *stream)
{
    const int esize = dtype_size(dtype);
    if (esize == 0) return TCCL_EINVAL;
    if ((numel * esize) % kVecBytes != 0 || (first_elem * esize) % kVecBytes != 0) return TCCL_EALIGN;
    RankArgs a;
    const int rc = rank_args(bufs, out, signal_pads, pad_bytes, world, rank, first_elem * esize, numel * esize, cfg, &a);
    if (rc != TCCL_OK) return rc;
    // an empty input still meets the peers: the barriers are the collective's ordering
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * kRankVecs * kVecBytes;
    size_t tiles = (a.bytes + tile_bytes - 1) / tile_bytes;
    if (tiles < 1) tiles = 1;
    const int wgs = cfg ? cfg->workgroups : 0;
    const size_t pad_words = pad_bytes / sizeof(uint32_t);
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == TCCL_BF16 ? launch_sum_rank<Bf16Sum>(a, tiles, wgs, pad_words, s)
                              : launch_sum_rank<F32Sum>(a, tiles, wgs, pad_words, s);
}

} // namespace tccl

extern "C" int tccl_all_reduce_sum_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes,
                                        int world, int rank, size_t numel, int dtype, const tccl_pipeline_cfg *cfg,
                                        void *stream)
{
    return sum_rank(bufs, out, signal_pads, pad_bytes, world, rank, 0, numel, dtype, cfg, stream);
}

extern "C" int tccl_reduce_scatter_sum_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes,
                                            int world, int rank, size_t numel_total, int dtype,
                                            const tccl_pipeline_cfg *cfg, void *stream)
{
    if (world < 1 || world > TCCL_MAX_WORLD || rank < 0 || rank >= world) return TCCL_EINVAL;
    // every rank's share is the same whole number of vectors (triton_reduce_scatter.py:101-104)
    if (numel_total % static_cast<size_t>(world) != 0) return TCCL_EALIGN;
    const size_t per_rank = numel_total / static_cast<size_t>(world);
    return sum_rank(bufs, out, signal_pads, pad_bytes, world, rank, static_cast<size_t>(rank) * per_rank, per_rank, dtype,
                    cfg, stream);
}

extern "C" int tccl_all_gather_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes, int world,
                                    int rank, size_t bytes_per_rank, const tccl_pipeline_cfg *cfg, void *stream)
{
    if (bytes_per_rank % kVecBytes != 0) return TCCL_EALIGN;
    RankArgs a;
    const int rc = rank_args(bufs, out, signal_pads, pad_bytes, world, rank, 0, bytes_per_rank, cfg, &a);
    if (rc != TCCL_OK) return rc;
    constexpr size_t tile_bytes = static_cast<size_t>(kPhasedBlock) * kRankVecs * kVecBytes;
    size_t tiles = (a.bytes + tile_bytes - 1) / tile_bytes;
    if (tiles < 1) tiles = 1;
    static std::once_flag once;
    static int resident = 0;
    std::call_once(once, [] { resident = resident_for(gather_rank_kernel, true); });
    return launch_rank_kernel(gather_rank_kernel, resident, a, tiles, cfg ? cfg->workgroups : 0,
                              pad_bytes / sizeof(uint32_t), static_cast<hipStream_t>(stream));
}

// ------------------------------------------------------------------ the entry point that allocates nothing
namespace tccl {

// Signal pads of the two-shot all-reduce for callers that cannot bring their own: W pads of
// kStaticPadBytes each, side by side in one array that every GPU holds from the moment the
// library is loaded until the process ends.  A pad has room for TCCL_STATIC_MAX_WORKGROUPS
// workgroups per rank in a world of TCCL_MAX_WORLD, plus the control words.
constexpr size_t kStaticPadBytes =
    (static_cast<size_t>(TCCL_STATIC_MAX_WORKGROUPS) * TCCL_MAX_WORLD + kCtlWords) * sizeof(uint32_t);
static_assert(kStaticPadBytes % 16 == 0, "pads must stay 16-byte aligned");
static_assert(kStaticPadBytes * TCCL_MAX_WORLD == TCCL_STATIC_SCRATCH_BYTES, "header and library disagree");

static __device__ __align__(256) unsigned char scratch[TCCL_STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current device (every GPU has its own copy of the array
// at its own address).  Looked up once per device; nullptr with *err set when that fails.
static unsigned char *scratch_on_current_device(hipError_t *err)
{
    constexpr int kMaxDevices = 64;
    static std::mutex m;
    static unsigned char *ptrs[kMaxDevices] = {};
    int dev = 0;
    *err = hipGetDevice(&dev);
    if (*err != hipSuccess) return nullptr;
    if (dev < 0 || dev >= kMaxDevices) {
        *err = hipErrorInvalidDevice;
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(m);
    if (ptrs[dev] == nullptr) {
        void *p = nullptr;
        *err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (*err != hipSuccess || p == nullptr) {
            if (*err == hipSuccess) *err = hipErrorInvalidSymbol;
            return nullptr;
        }
        ptrs[dev] = static_cast<unsigned char *>(p);
    }
    return ptrs[dev];
}

} // namespace tccl

extern "C" int tccl_two_shot_all_reduce_static(void *const *bufs, void *const *outs, int world, size_t numel,
                                               int dtype, const tccl_pipeline_cfg *cfg, void *stream)
{
    bool nothing = false;
    const int rc = two_shot_check(bufs, outs, world, numel, dtype, &nothing);
    if (rc != TCCL_OK) return rc;
    // more workgroups per rank than a static pad has flags for: say so instead of clamping
    if (cfg != nullptr && cfg->workgroups > TCCL_STATIC_MAX_WORKGROUPS * world) return TCCL_ESCRATCH;
    if (nothing) return TCCL_OK;
    hipError_t e = hipSuccess;
    unsigned char *base = scratch_on_current_device(&e);
    if (base == nullptr) return hip_code(e);
    uint32_t *pads[TCCL_MAX_WORLD];
    for (int r = 0; r < world; ++r) pads[r] = reinterpret_cast<uint32_t *>(base + static_cast<size_t>(r) * kStaticPadBytes);
    // The array keeps whatever the last call left: flags of a call whose waits expired would let
    // this call's waits pass too early.  Clear what this call can touch, in stream order, behind
    // the device's previous signalling kernel.
    ClearRequest clear;
    clear.base = reinterpret_cast<uint32_t *>(base);
    clear.pad_words = static_cast<uint32_t>(kStaticPadBytes / sizeof(uint32_t));
    // every flag word a launch on these pads can touch, whatever count of workgroups it settles on
    clear.flag_words = clear.pad_words - kCtlWords;
    clear.pads = world;
    return two_shot_launch(bufs, outs, pads, kStaticPadBytes, world, numel, dtype, cfg, &clear,
                           static_cast<hipStream_t>(stream));
}

// A 32-bit word in pinned host memory that the GPU can write: a caller without HIP bindings
// gets the `timeout_flag` of tccl_pipeline_cfg from here and reads it through the pointer.
extern "C" int tccl_timeout_flag_create(uint32_t **flag_out)
{
    if (flag_out == nullptr) return TCCL_EINVAL;
    *flag_out = nullptr;
    void *p = nullptr;
    const hipError_t e = hipHostMalloc(&p, 64, hipHostMallocMapped | hipHostMallocCoherent);
    if (e != hipSuccess) return hip_code(e);
    *static_cast<volatile uint32_t *>(p) = 0u;
    *flag_out = static_cast<uint32_t *>(p);
    return TCCL_OK;
}

extern "C" int tccl_timeout_flag_destroy(uint32_t *flag)
{
    if (flag == nullptr) return TCCL_EINVAL;
    return hip_code(hipHostFree(flag));
}
