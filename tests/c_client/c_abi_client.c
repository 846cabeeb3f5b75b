/*
 * A plain C client of libtccl_amd.so: no Python, no torch -- only the HIP runtime for
 * device memory and the entry points of include/tccl_amd.h.  It repeats the reference's
 * own known-answer test (every rank fills its buffer with its rank; the all-reduce is
 * W(W-1)/2 everywhere, triton_one_shot_all_reduce_no_128.py:116-127) for every operation.
 * Prints "c client ok" and exits 0 on success.
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tccl_amd.h"

#define W 8
#define N (8 * 8 * 4099) /* elements per rank, a multiple of 8*W */

#define HIP_OK(x)                                                                          \
    do {                                                                                   \
        hipError_t e_ = (x);                                                               \
        if (e_ != hipSuccess) {                                                            \
            fprintf(stderr, "%s failed: %s\n", #x, hipGetErrorString(e_));                 \
            return 2;                                                                      \
        }                                                                                  \
    } while (0)
#define TCCL_OK_(x)                                                                        \
    do {                                                                                   \
        int rc_ = (x);                                                                     \
        if (rc_ != TCCL_OK) {                                                              \
            fprintf(stderr, "%s -> %d (%s)\n", #x, rc_, tccl_error_string(rc_));           \
            return 3;                                                                      \
        }                                                                                  \
    } while (0)

static uint16_t bf16_of_small_int(int v)
{
    float f = (float)v; /* small integers are exact in bf16: truncation is the conversion */
    uint32_t u;
    memcpy(&u, &f, 4);
    return (uint16_t)(u >> 16);
}

static int all_equal(const uint16_t *p, size_t n, uint16_t want, const char *what)
{
    for (size_t i = 0; i < n; ++i)
        if (p[i] != want) {
            fprintf(stderr, "%s: element %zu is 0x%04x, want 0x%04x\n", what, i, p[i], want);
            return 0;
        }
    return 1;
}

int main(void)
{
    if (tccl_abi_version() != TCCL_ABI_VERSION) {
        fprintf(stderr, "ABI version mismatch\n");
        return 1;
    }
    void *bufs[W], *outs[W], *out = NULL, *gathered = NULL, *share = NULL;
    uint16_t *host = (uint16_t *)malloc((size_t)W * N * 2);
    if (!host) return 1;
    for (int r = 0; r < W; ++r) {
        HIP_OK(hipMalloc(&bufs[r], (size_t)N * 2));
        HIP_OK(hipMalloc(&outs[r], (size_t)N * 2));
        for (size_t i = 0; i < N; ++i) host[i] = bf16_of_small_int(r);
        HIP_OK(hipMemcpy(bufs[r], host, (size_t)N * 2, hipMemcpyHostToDevice));
    }
    HIP_OK(hipMalloc(&out, (size_t)N * 2));
    HIP_OK(hipMalloc(&share, (size_t)N / W * 2));
    HIP_OK(hipMalloc(&gathered, (size_t)W * N * 2));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    const uint16_t sum = bf16_of_small_int(W * (W - 1) / 2);

    TCCL_OK_(tccl_all_reduce_sum((const void *const *)bufs, W, out, N, TCCL_BF16, stream));
    TCCL_OK_(tccl_reduce_scatter_sum((const void *const *)bufs, W, 3, share, N, TCCL_BF16, stream));
    TCCL_OK_(tccl_all_gather((const void *const *)bufs, W, gathered, (size_t)N * 2, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(host, out, (size_t)N * 2, hipMemcpyDeviceToHost));
    if (!all_equal(host, N, sum, "all-reduce")) return 4;
    HIP_OK(hipMemcpy(host, share, (size_t)N / W * 2, hipMemcpyDeviceToHost));
    if (!all_equal(host, N / W, sum, "reduce-scatter")) return 4;
    HIP_OK(hipMemcpy(host, gathered, (size_t)W * N * 2, hipMemcpyDeviceToHost));
    for (int r = 0; r < W; ++r)
        if (!all_equal(host + (size_t)r * N, N, bf16_of_small_int(r), "all-gather row")) return 4;

    /* tree indices of rank 3 in a world of 8: tree.py:163 */
    int six[6];
    const int want6[6] = {2, -1, -1, 7, 1, 5};
    TCCL_OK_(tccl_double_tree_indices(W, 3, six));
    if (memcmp(six, want6, sizeof six) != 0) {
        fprintf(stderr, "tree indices of rank 3 differ\n");
        return 4;
    }

    /* the double tree overwrites the buffers with the result and fills every output */
    TCCL_OK_(tccl_double_tree_all_reduce(bufs, outs, W, N, TCCL_BF16, 0, stream));
    HIP_OK(hipStreamSynchronize(stream));
    for (int r = 0; r < W; ++r) {
        HIP_OK(hipMemcpy(host, outs[r], (size_t)N * 2, hipMemcpyDeviceToHost));
        if (!all_equal(host, N, sum, "double-tree output")) return 4;
        HIP_OK(hipMemcpy(host, bufs[r], (size_t)N * 2, hipMemcpyDeviceToHost));
        if (!all_equal(host, N, sum, "double-tree buffer")) return 4;
    }
    /* every buffer now holds 28: one tree reduce step own + 2 children gives 84 */
    TCCL_OK_(tccl_tree_reduce_step(bufs[0], bufs[1], bufs[2], bufs[0], N, TCCL_BF16, stream));
    TCCL_OK_(tccl_tree_copy_step(bufs[0], bufs[3], bufs[4], (size_t)N * 2, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipMemcpy(host, bufs[4], (size_t)N * 2, hipMemcpyDeviceToHost));
    if (!all_equal(host, N, bf16_of_small_int(84), "tree step + copy")) return 4;

    /* the signalling kernels: refill with the ranks, zero-filled pads from hipMalloc + hipMemset */
    void *pads[W];
    size_t pad_bytes = tccl_double_tree_signal_pad_bytes(W, N, TCCL_BF16, 0);
    if (pad_bytes < 4096) pad_bytes = 4096;
    for (int r = 0; r < W; ++r) {
        HIP_OK(hipMalloc(&pads[r], pad_bytes));
        HIP_OK(hipMemset(pads[r], 0, pad_bytes));
        for (size_t i = 0; i < N; ++i) host[i] = bf16_of_small_int(r);
        HIP_OK(hipMemcpy(bufs[r], host, (size_t)N * 2, hipMemcpyHostToDevice));
    }
    unsigned expired = 1;
    TCCL_OK_(tccl_double_tree_all_reduce_pipelined(bufs, outs, pads, pad_bytes, W, N, TCCL_BF16, 0, NULL, stream));
    TCCL_OK_(tccl_signal_pad_timeouts(pads[0], pad_bytes, &expired, stream));
    if (expired != 0) {
        fprintf(stderr, "pipelined double tree: %u waits expired\n", expired);
        return 4;
    }
    for (int r = 0; r < W; ++r) {
        HIP_OK(hipMemcpy(host, outs[r], (size_t)N * 2, hipMemcpyDeviceToHost));
        if (!all_equal(host, N, sum, "pipelined double-tree output")) return 4;
    }
    /* every buffer holds 28 now: the in-place two-shot all-reduce of eight of them gives 224 */
    TCCL_OK_(tccl_two_shot_all_reduce(bufs, NULL, pads, pad_bytes, W, N, TCCL_BF16, NULL, stream));
    TCCL_OK_(tccl_signal_pad_timeouts(pads[0], pad_bytes, &expired, stream));
    if (expired != 0) {
        fprintf(stderr, "two-shot all-reduce: %u waits expired\n", expired);
        return 4;
    }
    for (int r = 0; r < W; ++r) {
        HIP_OK(hipMemcpy(host, bufs[r], (size_t)N * 2, hipMemcpyDeviceToHost));
        if (!all_equal(host, N, bf16_of_small_int(224), "two-shot buffer")) return 4;
        hipFree(pads[r]);
    }

    /* error codes instead of faults */
    if (tccl_all_reduce_sum((const void *const *)bufs, 9, out, N, TCCL_BF16, stream) != TCCL_EINVAL) return 5;
    if (tccl_all_gather((const void *const *)bufs, W, gathered, 24, stream) != TCCL_EALIGN) return 5;

    for (int r = 0; r < W; ++r) {
        hipFree(bufs[r]);
        hipFree(outs[r]);
    }
    hipFree(out);
    hipFree(share);
    hipFree(gathered);
    hipStreamDestroy(stream);
    free(host);
    printf("c client ok\n");
    return 0;
}
