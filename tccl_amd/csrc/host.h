// host.h -- host-side helpers shared by the entry points: argument checks, launch-shape
// selection and error mapping.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/tccl_amd.h"

namespace tccl {

inline int hip_code(hipError_t e) { return e == hipSuccess ? TCCL_OK : TCCL_EHIP_BASE - static_cast<int>(e); }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int dtype_size(int dtype)
{
    switch (dtype) {
    case TCCL_BF16: return 2;
    case TCCL_F32: return 4;
    default: return 0;
    }
}

// Number of compute units of the current device (cached per process; 256 on MI355X).
int compute_units();

// A resolved launch shape.
struct Shape {
    int block, unroll, grid, tile_iters;
    bool nt_load, nt_store, xcd_contiguous;
};

// Fill in whatever the caller left at 0.
//   nvec      -- 16-byte vectors of output the launch produces (per row for the gather)
//   nsrc      -- source streams read per output vector
//   rows      -- rows of nvec vectors each that share the grid (gather), else 1
//   is_copy   -- a pure copy: from 8 MiB they get their own defaults (one or two workgroups per
//                compute unit, four vectors per lane, streaming loads and stores)
Shape resolve_shape(const tccl_launch_cfg *cfg, size_t nvec, int nsrc, int rows, bool is_copy = false);

} // namespace tccl
