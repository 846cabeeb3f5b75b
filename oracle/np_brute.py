"""numpy brute force of the float-sum contract, independent of torch and of the C oracle.

Test infrastructure only.  bf16 values are carried as uint16 bit patterns; widening and
rounding are done with integer arithmetic written differently from tccl_oracle.c (explicit
remainder comparison instead of the bias trick), so a mistake in either shows up as a
mismatch.  Meant for inputs of a few thousand elements.
"""
from __future__ import annotations

from typing import Optional, Sequence

import numpy as np


def widen(bits: np.ndarray) -> np.ndarray:
    """bf16 bit patterns (uint16) -> float32, exact."""
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def narrow(x: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round to nearest, ties to even; NaN -> 0x7FC0."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    upper = u >> np.uint64(16)
    rem = u & np.uint64(0xFFFF)
    up = (rem > 0x8000) | ((rem == 0x8000) & ((upper & np.uint64(1)) == 1))
    out = (upper + up.astype(np.uint64)).astype(np.uint16)
    isnan = (u & np.uint64(0x7FFFFFFF)) > np.uint64(0x7F800000)
    out[isnan] = 0x7FC0
    return out


def all_reduce_bf16(bufs: Sequence[np.ndarray]) -> np.ndarray:
    """AR:53-64 under the contract arithmetic, one element at a time."""
    n = bufs[0].size
    out = np.empty(n, dtype=np.float32)
    wide = [widen(b) for b in bufs]
    with np.errstate(all="ignore"):
        for j in range(n):
            acc = np.float32(0.0)
            for w in wide:
                acc = np.float32(acc + w[j])
            out[j] = acc
    return narrow(out)


def all_reduce_f32(bufs: Sequence[np.ndarray]) -> np.ndarray:
    n = bufs[0].size
    out = np.empty(n, dtype=np.float32)
    with np.errstate(all="ignore"):
        for j in range(n):
            acc = np.float32(0.0)
            for b in bufs:
                acc = np.float32(acc + b[j])
            out[j] = acc
    return out


def tree_reduce_step_bf16(own: np.ndarray, child0: Optional[np.ndarray],
                          child1: Optional[np.ndarray]) -> np.ndarray:
    """DT:274-294 + DT:276-288: order (child0, child1, own), absent children skipped."""
    srcs = [c for c in (child0, child1) if c is not None] + [own]
    return all_reduce_bf16(srcs)
