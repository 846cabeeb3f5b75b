"""Shared input generators and comparisons for the tests."""
from __future__ import annotations

from typing import List

import numpy as np
import torch


def seeded_randn(world: int, numel: int, dtype=torch.bfloat16, seed_base: int = 0) -> List[torch.Tensor]:
    """The reference's recipe (triton_reduce_scatter.py:185-195): rank r's buffer is
    ``torch.manual_seed(r); torch.randn(numel, dtype=...)`` made on the CPU."""
    out = []
    for r in range(world):
        torch.manual_seed(seed_base + r)
        out.append(torch.randn(numel, dtype=dtype))
    return out


def seeded_uniform(world: int, numel: int, seed_base: int = 0) -> List[torch.Tensor]:
    """fp32 ~U(-1, 1), seed = rank."""
    out = []
    for r in range(world):
        torch.manual_seed(seed_base + r)
        out.append(torch.rand(numel, dtype=torch.float32) * 2 - 1)
    return out


def seeded_int8(world: int, numel: int, seed_base: int = 0) -> List[torch.Tensor]:
    out = []
    for r in range(world):
        torch.manual_seed(seed_base + r)
        out.append(torch.randint(-128, 128, (numel,), dtype=torch.int8))
    return out


def bits(t: torch.Tensor) -> torch.Tensor:
    """Integer view of a tensor's bytes, so that comparisons are bit comparisons."""
    t = t.detach().cpu().contiguous()
    view = {1: torch.int8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()]
    return t.view(view)


def np_bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 numpy array; fp32 tensor -> float32 numpy array."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def from_np_bits(a: np.ndarray) -> torch.Tensor:
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return torch.from_numpy(a.copy())


def assert_bit_equal(got: torch.Tensor, want: torch.Tensor, what: str = "") -> None:
    g, w = bits(got), bits(want)
    assert g.shape == w.shape, f"{what}: shape {tuple(g.shape)} != {tuple(w.shape)}"
    if not torch.equal(g, w):
        bad = (g != w).reshape(-1).nonzero().reshape(-1)
        i = int(bad[0])
        raise AssertionError(f"{what}: {bad.numel()} of {g.numel()} elements differ; first at {i}: "
                             f"got {int(g.reshape(-1)[i]):#x} want {int(w.reshape(-1)[i]):#x}")


def assert_bit_equal_nan_aware(got: torch.Tensor, want: torch.Tensor, what: str = "") -> None:
    """Bit equality everywhere except that any NaN matches any NaN (NaN sign and payload
    are not part of the contract)."""
    gf, wf = got.detach().cpu().float(), want.detach().cpu().float()
    gn, wn = torch.isnan(gf), torch.isnan(wf)
    assert torch.equal(gn, wn), f"{what}: NaN positions differ"
    g, w = bits(got).clone(), bits(want).clone()
    g[gn] = 0
    w[wn] = 0
    assert torch.equal(g, w), f"{what}: non-NaN elements differ"


def bf16_bits_equal_nan_aware(a: np.ndarray, b: np.ndarray) -> bool:
    """uint16 bf16 patterns: equal bit for bit, except that any NaN equals any NaN."""
    an = (a & 0x7FFF) > 0x7F80
    bn = (b & 0x7FFF) > 0x7F80
    return bool(np.array_equal(an, bn) and np.array_equal(a[~an], b[~bn]))
