// stamped.hip -- the library's own kernels with time stamps, for bench.py --stamps
// (benchlib/libtccl_amd_stamped.so; no part of the product).  Every source of the library is
// compiled here as ONE translation unit with TCCL_STAMPS defined, which turns the TCCL_STAMP()
// marks in the kernels into wall-clock readings per workgroup (see tccl_amd/csrc/vec.h); the
// result exports the library's whole C ABI plus tccl_stamp_buffer() below, so the benchmark
// runs an operation through the same wrappers and entry points and then reads when each
// workgroup started, got its first data, finished reading and finished writing.
#define TCCL_STAMPS 1
#include "../tccl_amd/csrc/util.hip"
#include "../tccl_amd/csrc/sum.hip"
#include "../tccl_amd/csrc/gather.hip"
#include "../tccl_amd/csrc/tree.hip"
#include "../tccl_amd/csrc/pipeline.hip"
#include "../tccl_amd/csrc/ipc.hip"

// Device address of the stamp words on the current device, how many 64-bit words a workgroup has
// and how many workgroups there is room for.
extern "C" int tccl_stamp_buffer(void **ptr_out, int *slots_out, int *max_workgroups_out)
{
    if (ptr_out == nullptr) return TCCL_EINVAL;
    void *p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(tccl::stamp_words));
    if (e != hipSuccess) return tccl::hip_code(e);
    *ptr_out = p;
    if (slots_out) *slots_out = tccl::kStampSlots;
    if (max_workgroups_out) *max_workgroups_out = tccl::kStampMaxWorkgroups;
    return TCCL_OK;
}
