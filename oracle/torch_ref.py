"""torch CPU reference of the collectives' per-rank data path.

Test infrastructure only (see the package docstring).  Each function cites the lines of
the reference it restates; AR/RS/AG/DT/TREE are the reference's
triton_one_shot_all_reduce_no_128.py, triton_reduce_scatter.py, triton_all_gather.py,
triton_double_tree_allreduce.py and tree.py.

Float sums follow the contract arithmetic: widen to fp32, accumulate from +0 in rank
order 0..W-1 (zero start AR:57, order AR:58), round once to the input dtype.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch


def _acc_dtype(dtype: torch.dtype) -> torch.dtype:
    if dtype in (torch.bfloat16, torch.float16, torch.float32):
        return torch.float32
    raise TypeError(f"unsupported dtype for a sum: {dtype}")


def all_reduce(bufs: Sequence[torch.Tensor], acc: Optional[torch.Tensor] = None) -> torch.Tensor:
    """AR:53-64.  ``out[j] = round(0 + buf_0[j] + buf_1[j] + ... )`` in fp32, rank order.

    ``acc`` is an optional pre-allocated fp32 accumulator (used when this is timed)."""
    first = bufs[0]
    if acc is None:
        acc = torch.zeros(first.shape, dtype=_acc_dtype(first.dtype))
    else:
        acc.zero_()
    for b in bufs:                       # explicit loop: torch.sum does not promise an order
        acc += b
    return acc.to(first.dtype)


def all_reduce_stepwise(bufs: Sequence[torch.Tensor]) -> torch.Tensor:
    """Information only: the reference's own arithmetic, packed add.bf16x2 (AR:22-23),
    i.e. the running sum re-rounded to bf16 after every rank (what RS:197-200 computes as
    its expected value).  Never a pass/fail gate."""
    acc = torch.zeros_like(bufs[0])
    for b in bufs:
        acc += b
    return acc


def reduce_scatter(bufs: Sequence[torch.Tensor], rank: int) -> torch.Tensor:
    """RS:73-92: rank's share is elements [rank*P, (rank+1)*P), P = numel // W (RS:73,
    RS:86), summed like the all-reduce."""
    world = len(bufs)
    per_rank = bufs[0].numel() // world
    lo = rank * per_rank
    return all_reduce([b.reshape(-1)[lo:lo + per_rank] for b in bufs])


def all_gather(bufs: Sequence[torch.Tensor]) -> torch.Tensor:
    """AG:54-62, AG:82: output [W, *shape], row i is a copy of buf_i (AG:128 builds the
    expected value the same way, with torch.stack)."""
    out = torch.empty((len(bufs),) + tuple(bufs[0].shape), dtype=bufs[0].dtype)
    for i, b in enumerate(bufs):
        out[i].copy_(b)
    return out


def tree_reduce_step(own: torch.Tensor, child0: Optional[torch.Tensor],
                     child1: Optional[torch.Tensor]) -> torch.Tensor:
    """DT:274-294 with the commented child adds DT:276-288: 0 + child0 + child1 + own in
    that order, absent children (the reference's -1) skipped, one rounding."""
    acc = torch.zeros(own.shape, dtype=_acc_dtype(own.dtype))
    if child0 is not None:
        acc += child0
    if child1 is not None:
        acc += child1
    acc += own
    return acc.to(own.dtype)


# ------------------------------------------------------------------ tree index math

def build_tree(n: int) -> List[int]:
    """TREE:5-31, restated recursively instead of row by row: the heap-ordered array of
    the perfect binary tree whose in-order labelling is 1..n-1, with node 0 in front."""
    if n < 2 or n & (n - 1):
        raise AssertionError("len(ranks) is not a power of 2!")
    levels: List[List[int]] = []
    span = n
    while span >= 2:
        # level with subtree span `span`: midpoints span/2, span/2 + span, ...
        levels.append(list(range(span // 2, n, span)))
        span //= 2
    out = [0]
    for row in levels:
        out.extend(row)
    return out


def build_double_tree(n: int) -> Tuple[List[int], List[int]]:
    """TREE:83-91."""
    a = build_tree(n)
    b = [e - 1 for e in a]
    b[0] = n - 1
    return a, b


def get_parents_and_children(n: int, rank: int) -> Tuple[int, int, int, int, int, int]:
    """TREE:93-148."""
    def one(tree: List[int]) -> Tuple[int, int, int]:
        pos = tree.index(rank)
        if pos == 0:
            return -1, tree[1], -1
        c0, c1 = 2 * pos, 2 * pos + 1
        return (tree[pos // 2],
                tree[c0] if c0 < len(tree) else -1,
                tree[c1] if c1 < len(tree) else -1)
    a, b = build_double_tree(n)
    return one(a) + one(b)


def double_tree_split(numel: int, esize: int) -> int:
    """Boundary between the half reduced over tree a and the half over tree b:
    floor(numel/2) rounded down to whole 16-byte vectors."""
    per_vec = 16 // esize
    return (numel // 2) // per_vec * per_vec


def double_tree_all_reduce(bufs: Sequence[torch.Tensor]) -> List[torch.Tensor]:
    """The collective as designed (DT:254-335 plus TREE:39-50), for all W virtual ranks.

    Per tree, on its half of the element range: every node computes
    round(0 + R_child0 + R_child1 + X_own) (children first), so there is one rounding per
    tree level; the subroot's result is then copied to every rank (DT:314-325).  Written
    as a recursion over the rank graph so that it shares no traversal code with the C
    oracle or with the product's level schedule.  Inputs are not modified; returns the W
    outputs (all bit-identical)."""
    world = len(bufs)
    flat = [b.reshape(-1) for b in bufs]
    numel = flat[0].numel()
    split = double_tree_split(numel, flat[0].element_size())
    result = torch.empty_like(flat[0])

    for which, (lo, hi) in enumerate(((0, split), (split, numel))):
        def node_result(rank: int) -> torch.Tensor:
            t = get_parents_and_children(world, rank)[3 * which:3 * which + 3]
            c0 = node_result(t[1]) if t[1] >= 0 else None
            c1 = node_result(t[2]) if t[2] >= 0 else None
            return tree_reduce_step(flat[rank][lo:hi], c0, c1)
        root = build_double_tree(world)[which][0]
        result[lo:hi] = node_result(root)
    return [result.clone().reshape(bufs[0].shape) for _ in range(world)]
