"""Tree index math: product (closed forms in the C library) and the three oracle
restatements against the reference-held known answers and against each other."""
import pytest

import tccl_amd
from oracle import torch_ref

KAT_WORLDS_ARRAYS = ["4", "8", "16", "32"]
KAT_WORLDS_TUPLES = ["4", "8", "32"]


def impls(c_oracle):
    return {
        "product": (tccl_amd.build_double_tree, tccl_amd.get_parents_and_children, tccl_amd.build_tree),
        "c_oracle": (c_oracle.build_double_tree, c_oracle.get_parents_and_children, c_oracle.build_tree),
        "torch_ref": (torch_ref.build_double_tree, torch_ref.get_parents_and_children, torch_ref.build_tree),
    }


@pytest.mark.parametrize("name", ["product", "c_oracle", "torch_ref"])
def test_arrays_known_answers(name, tree_kat, c_oracle):
    double, _, single = impls(c_oracle)[name]
    for n in KAT_WORLDS_ARRAYS:
        a, b = double(int(n))
        assert list(a) == tree_kat["arrays"][n]["a"], (name, n)
        assert list(b) == tree_kat["arrays"][n]["b"], (name, n)
        assert list(single(int(n))) == tree_kat["arrays"][n]["a"]
        # tree.py:156,158: both arrays are permutations
        assert sorted(a) == list(range(int(n))) and sorted(b) == list(range(int(n)))


@pytest.mark.parametrize("name", ["product", "c_oracle", "torch_ref"])
def test_tuples_known_answers(name, tree_kat, c_oracle):
    _, gpc, _ = impls(c_oracle)[name]
    for n in KAT_WORLDS_TUPLES:
        for rank, want in enumerate(tree_kat["tuples"][n]):
            assert tuple(gpc(int(n), rank)) == tuple(want), (name, n, rank)


@pytest.mark.parametrize("name", ["product", "c_oracle", "torch_ref"])
def test_parent_table_w8(name, tree_kat, c_oracle):
    """The W=8 parent table kept in triton_barrier2.py:157-161."""
    _, gpc, _ = impls(c_oracle)[name]
    assert [gpc(8, r)[0] for r in range(8)] == tree_kat["parents_w8"]["tree0"]
    assert [gpc(8, r)[3] for r in range(8)] == tree_kat["parents_w8"]["tree1"]


@pytest.mark.parametrize("n", [2, 4, 8, 16, 32, 64, 128, 256, 512, 1024])
def test_three_implementations_agree(n, c_oracle):
    """Closed form (product) vs row-by-row construction (C oracle) vs level construction
    (torch_ref): three different algorithms, every rank, worlds the reference holds no
    vector for included."""
    a_p, b_p = tccl_amd.build_double_tree(n)
    assert (list(a_p), list(b_p)) == tuple(map(list, c_oracle.build_double_tree(n)))
    assert (list(a_p), list(b_p)) == tuple(map(list, torch_ref.build_double_tree(n)))
    for r in range(n):
        t = tccl_amd.get_parents_and_children(n, r)
        assert t == tuple(c_oracle.get_parents_and_children(n, r)), (n, r)
        if n <= 128:
            assert t == tuple(torch_ref.get_parents_and_children(n, r)), (n, r)


@pytest.mark.parametrize("n", [2, 4, 8, 16, 64, 1024])
def test_structure_invariants(n):
    """What the docstring of build_double_tree promises (tree.py:47-50): each rank is a
    leaf in one tree and interior in the other (the two subroots aside), parent/child
    relations are mutual, each tree is connected and rooted at its subroot."""
    tuples = [tccl_amd.get_parents_and_children(n, r) for r in range(n)]
    a, b = tccl_amd.build_double_tree(n)
    for which, tree in ((0, a), (1, b)):
        root = tree[0]
        for r in range(n):
            parent, c0, c1 = tuples[r][3 * which:3 * which + 3]
            if r == root:
                assert parent == -1 and c0 == tree[1] and c1 == -1
            else:
                assert parent >= 0
                assert r in tuples[parent][3 * which + 1:3 * which + 3]
                assert (c0 == -1) == (c1 == -1)
            for c in (c0, c1):
                if c >= 0:
                    assert tuples[c][3 * which] == r
            # walking up reaches the subroot
            cur, steps = r, 0
            while tuples[cur][3 * which] != -1:
                cur = tuples[cur][3 * which]
                steps += 1
                assert steps <= n
            assert cur == root
    if n >= 4:
        for r in range(n):
            a_leaf = tuples[r][1] == -1
            b_leaf = tuples[r][4] == -1
            if r not in (a[0], b[0]):
                assert a_leaf != b_leaf, r
    # second tree = first tree shifted by one (tree.py:83-89)
    assert [(x + n - 1) % n for x in a] == list(b)


def test_error_behaviour():
    """Same failures as the reference: tree.py:11 (power of two), tree.py:135 (one rank),
    list.index at tree.py:131 (rank outside the world)."""
    for n in (3, 6, 12, 100):
        with pytest.raises(AssertionError):
            tccl_amd.build_tree(n)
        with pytest.raises(AssertionError):
            tccl_amd.get_parents_and_children(n, 0)
    assert tccl_amd.build_tree(1) == [0]
    with pytest.raises(IndexError):
        tccl_amd.get_parents_and_children(1, 0)
    with pytest.raises(ValueError):
        tccl_amd.get_parents_and_children(8, 8)
    with pytest.raises(ValueError):
        tccl_amd.get_parents_and_children(8, -1)


def test_c_abi_error_codes():
    import ctypes
    lib = tccl_amd.load_library()
    out = (ctypes.c_int * 6)()
    assert lib.tccl_double_tree_indices(6, 0, out) == -3
    assert lib.tccl_double_tree_indices(1, 0, out) == -3
    assert lib.tccl_double_tree_indices(8, 8, out) == -1
    assert lib.tccl_double_tree_indices(8, 0, None) == -1
    assert lib.tccl_double_tree_arrays(8, None, None) == -1
    assert lib.tccl_double_tree_split(100, 2) == 48
    assert lib.tccl_double_tree_split(134217728, 2) == 67108864
    assert lib.tccl_double_tree_split(7, 4) == 0
