// ipc.hip -- buffers that several processes on one GPU can map, and the reference's blockwise
// barrier as a kernel of its own that each owner launches for itself.
//
// The reference allocates its peer-mappable buffers with _SymmetricMemory.empty_strided_p2p
// (triton_one_shot_all_reduce_no_128.py:116-122), exchanges them with rendezvous (:82), and
// every rank's kernel begins with blockwise_barrier (triton_barrier.py:39-142), which meets
// the other ranks' kernels through signal pads in peer memory.  Here the owners are separate
// processes sharing one MI355X: an allocation is exported as a 64-byte handle
// (hipIpcGetMemHandle), carried to the peers by whatever the host side uses (files, pipes), and
// opened there (hipIpcOpenMemHandle); the addresses that come out go into the same pointer
// tables every other entry point of the library takes.
#include <cstring>

#include "host.h"
#include "vec.h"

namespace tccl {

constexpr uint32_t kBarrierDefaultSpins = 1u << 22;

// Rank `rank`'s side of the barrier, for `blocks` independent rows of slots: lane i < world of
// workgroup g raises slot g * world + rank in rank i's pad (a system-scope store: the pad
// belongs to another process) and waits until slot g * world + i of its own pad has been
// raised by rank i, then lowers it again, so a pad that starts zero-filled is zero-filled after
// every completed barrier (triton_barrier.py:49-54).  A slot has one writer of 1 (the sender)
// and one writer of 0 (the owner), so the reference's compare-and-swap loops become "wait until
// the slot reads 0, store 1" on the sending side and "wait until it reads 1, store 0" on the
// receiving side.  The sender's wait matters: a rank may enter its next barrier while a peer
// has seen, but not yet lowered, the flag of the previous one, and a flag raised then would be
// wiped out with the old one.  Waits are bounded: a lane that polls spin_limit times in vain
// sets *timeout_flag (if given) and gives up; the kernel always ends.
struct PadTable {
    uint32_t *p[TCCL_MAX_WORLD];
};

__global__ void __launch_bounds__(64) blockwise_barrier_kernel(PadTable pads, int world, int rank, uint32_t spin_limit,
                                                               uint32_t *timeout_flag)
{
    uint32_t *const(&pad)[TCCL_MAX_WORLD] = pads.p;
    const int lane = threadIdx.x;
    if (lane >= world || lane == rank) return;
    const uint32_t base = blockIdx.x * static_cast<uint32_t>(world);
    uint32_t *theirs = nullptr, *mine = pad[0];
#pragma unroll
    for (int i = 0; i < TCCL_MAX_WORLD; ++i) {
        if (i == lane) theirs = pad[i] + base + rank;
        if (i == rank) mine = pad[i] + base + lane;
    }
    uint32_t polls = 0;
    bool expired = false;
    // send: the slot must have been lowered by its owner since this rank last raised it
    while (__hip_atomic_load(theirs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) != 0u) {
        if (++polls >= spin_limit) {
            expired = true;
            break;
        }
        __builtin_amdgcn_s_sleep(8);
    }
    if (!expired) {
        __hip_atomic_store(theirs, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
        // wait: the peer's flag in this rank's pad
        while (__hip_atomic_load(mine, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM) == 0u) {
            if (++polls >= spin_limit) {
                expired = true;
                break;
            }
            __builtin_amdgcn_s_sleep(8);
        }
    }
    if (expired) {
        if (timeout_flag != nullptr) __hip_atomic_store(timeout_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        return;
    }
    __hip_atomic_store(mine, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

} // namespace tccl

using namespace tccl;

extern "C" int tccl_symm_alloc(size_t bytes, void **ptr_out)
{
    if (ptr_out == nullptr || bytes == 0) return TCCL_EINVAL;
    *ptr_out = nullptr;
    // an allocation that is mapped into other processes stays below 2 GiB
    if (bytes >= (static_cast<size_t>(2) << 30)) return TCCL_EINVAL;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes);
    if (e != hipSuccess) return hip_code(e);
    // hipMemset on device memory may return before the fill has run (it is queued on the null
    // stream, behind whatever this process has in flight there).  The caller exports the
    // allocation next, and a peer that maps it may raise flags in it straight away: the zeros
    // must be in place before this call returns, or the late fill would wipe those flags out.
    e = hipMemset(p, 0, bytes);
    if (e == hipSuccess) e = hipStreamSynchronize(nullptr);
    if (e != hipSuccess) {
        (void)hipFree(p);
        return hip_code(e);
    }
    *ptr_out = p;
    return TCCL_OK;
}

extern "C" int tccl_symm_free(void *ptr)
{
    if (ptr == nullptr) return TCCL_EINVAL;
    return hip_code(hipFree(ptr));
}

static_assert(sizeof(hipIpcMemHandle_t) == TCCL_IPC_HANDLE_BYTES, "handle size");

extern "C" int tccl_ipc_export(void *ptr, unsigned char *handle_out)
{
    if (ptr == nullptr || handle_out == nullptr) return TCCL_EINVAL;
    hipIpcMemHandle_t h;
    const hipError_t e = hipIpcGetMemHandle(&h, ptr);
    if (e != hipSuccess) return hip_code(e);
    std::memcpy(handle_out, &h, sizeof(h));
    return TCCL_OK;
}

extern "C" int tccl_ipc_open(const unsigned char *handle, void **ptr_out)
{
    if (handle == nullptr || ptr_out == nullptr) return TCCL_EINVAL;
    *ptr_out = nullptr;
    hipIpcMemHandle_t h;
    std::memcpy(&h, handle, sizeof(h));
    void *p = nullptr;
    const hipError_t e = hipIpcOpenMemHandle(&p, h, hipIpcMemLazyEnablePeerAccess);
    if (e != hipSuccess) return hip_code(e);
    *ptr_out = p;
    return TCCL_OK;
}

extern "C" int tccl_ipc_close(void *ptr)
{
    if (ptr == nullptr) return TCCL_EINVAL;
    return hip_code(hipIpcCloseMemHandle(ptr));
}

extern "C" int tccl_blockwise_barrier(void *const *signal_pads, size_t pad_bytes, int world, int rank, int blocks,
                                      unsigned spin_limit, uint32_t *timeout_flag, void *stream)
{
    if (signal_pads == nullptr || world < 1 || world > TCCL_MAX_WORLD || rank < 0 || rank >= world || blocks < 1)
        return TCCL_EINVAL;
    if (pad_bytes < static_cast<size_t>(blocks) * world * sizeof(uint32_t)) return TCCL_EINVAL;
    PadTable t = {};
    for (int i = 0; i < world; ++i) {
        if (signal_pads[i] == nullptr) return TCCL_EINVAL;
        if (!aligned16(signal_pads[i])) return TCCL_EALIGN;
        t.p[i] = static_cast<uint32_t *>(signal_pads[i]);
    }
    if (world == 1) return TCCL_OK;
    hipLaunchKernelGGL(blockwise_barrier_kernel, dim3(static_cast<unsigned>(blocks)), dim3(64), 0,
                       static_cast<hipStream_t>(stream), t, world, rank, spin_limit > 0 ? spin_limit : kBarrierDefaultSpins,
                       timeout_flag);
    return hip_code(hipGetLastError());
}
