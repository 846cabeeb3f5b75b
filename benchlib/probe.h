/*
 * probe.h -- measuring kernels used by bench.py only (benchlib/libtccl_probe.so).  Not part of
 * the product library or its ABI; none of them has a counterpart in the reference.
 */
#ifndef TCCL_PROBE_H
#define TCCL_PROBE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The read half of the large all-reduce on its own: reads and reduces `world` buffers of
 * bytes_per_buffer each (bf16 arithmetic, the sum kernel's launch shape) and stores nothing
 * (`sink`: 4,096 bytes of device memory that receives a checksum in one case out of 2^32,
 * which is what keeps the loads alive). */
int tccl_probe_read(const void *const *bufs, int world, size_t bytes_per_buffer, void *sink, void *stream);
/* The write half: fills `bytes` at dst with a pattern, 32 stores per lane back to back. */
int tccl_probe_write(void *dst, size_t bytes, void *stream);
/* The same fill in 32 KiB tiles: the fastest way found to write HBM in tiles. */
int tccl_probe_write_small(void *dst, size_t bytes, void *stream);
/* pure write, one workgroup per compute unit, 4 KiB per workgroup per step: one dense window */
int tccl_probe_write_dense(void *dst, size_t bytes, void *stream);
/* One contiguous range read front to back by the whole GPU (grid-stride, streaming loads): the
 * fastest way found to read HBM, the reference point for every read rate in the benchmark. */
int tccl_probe_read_dense(const void *buf, size_t bytes, void *sink, void *stream);
/* A plain copy in the launch shape that is fastest on uncached data: the reference point for the
 * copies (all-gather, tree copy step). */
int tccl_probe_copy(const void *src, void *dst, size_t bytes, void *stream);
/* The large all-reduce's kernel shape (8 bf16 sources, one 128 KiB tile per workgroup) with time
 * stamps: stamps[3*b + 0..2] = 100 MHz wall clock of workgroup b at its start, at the end of its
 * read phase and at the end of its writes. */
int tccl_probe_sum_timed(const void *const *bufs, void *out, size_t bytes_per_buffer, long long *stamps, void *stream);
/* One empty kernel: what a timed single launch costs when the kernel does nothing. */
int tccl_probe_empty(void *stream);
/* A one-lane kernel that stores the GPU's 100 MHz wall clock at `slot` (device memory): where a
 * stream has got to, on a clock that all processes sharing the GPU read alike. */
int tccl_probe_stamp(long long *slot, void *stream);
/* An empty kernel of `workgroups` x 256 lanes, and the same grid with every lane loading one
 * 16-byte vector from src and storing it to dst (both workgroups x 4 KiB): what a short
 * streaming kernel costs whatever it moves. */
int tccl_probe_empty_grid(int workgroups, void *stream);
int tccl_probe_touch(const void *src, void *dst, int workgroups, void *stream);
/* out[2*b] = HW_REG_HW_ID, out[2*b+1] = HW_REG_XCC_ID of workgroup b of a grid of `workgroups`
 * x 256 lanes, each holding its slot for hold_us microseconds. */
int tccl_probe_placement(uint32_t *out, int workgroups, int hold_us, void *stream);

#ifdef __cplusplus
}
#endif
#endif
