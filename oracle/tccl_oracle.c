/*
 * tccl_oracle.c -- CPU restatement of the per-rank data path of tccl's collectives.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, __graft_entry__.smoke()
 * and bench.py's cpu_baseline leg may load it, and only as the checker.  The shipped
 * library (tccl_amd/csrc) never links, loads or calls anything in this file.
 *
 * Every function names the lines of the reference it restates (paths relative to the
 * reference checkout):
 *   AR   = triton_one_shot_all_reduce_no_128.py
 *   RS   = triton_reduce_scatter.py
 *   AG   = triton_all_gather.py
 *   DT   = triton_double_tree_allreduce.py
 *   TREE = tree.py
 *
 * Arithmetic contract for float sums: widen each bf16 to fp32 (exact), accumulate in
 * fp32 starting from +0.0f in rank order 0..W-1 (AR:57-61, RS:83-88 give the zero start
 * and the order), round ONCE to bf16 with round-to-nearest-even.  The reference itself
 * re-rounds to bf16 after every rank (packed add.bf16x2, AR:22-23); that variant is kept
 * below as orc_all_reduce_bf16_stepwise for information only and is never a gate.
 *
 * How each function is pinned (see tests/test_oracle*.py):
 *   tree indices        : reference-held known answers TREE:155-243 (arrays N=4,8,16,32;
 *                         6-tuples N=4,8,32), the independent W=8 parent table
 *                         triton_barrier2.py:157-161, permutation/consistency invariants,
 *                         and the product's closed form (a different algorithm).
 *   bf16 rounding       : exhaustive comparison over all 2^16 upper halves x boundary
 *                         lower halves against torch's float->bfloat16, plus RNE ties.
 *   sums                : fill_(rank) -> W(W-1)/2 (AR:116-127), small-integer closed
 *                         forms, the order-sensitivity vector, an independent numpy
 *                         brute force, and torch's own fp32 arithmetic.
 *   gather / copy       : byte equality with the stacked sources (AG:128 recipe).
 *   double-tree values  : the reference never produced a value for this op (its kernel
 *                         is a stub, DT:276-335), so parity WITH THE REFERENCE is
 *                         unpinned by construction; the schedule is pinned by the tree
 *                         tables, fill_(rank) -> W(W-1)/2, "all ranks bit-identical",
 *                         and an independent recursive numpy restatement.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -fopenmp).
 */
#include <stddef.h>
#include <stdint.h>
#include <string.h>

/* ---------------------------------------------------------------- bf16 <-> fp32 */

static inline float orc_widen(uint16_t h)
{
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Round-to-nearest-even fp32 -> bf16.  NaN maps to the canonical quiet NaN 0x7FC0
 * (what torch's CPU conversion produces); sign and payload of a NaN are therefore not
 * part of the contract. */
static inline uint16_t orc_narrow(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u)
        return 0x7FC0;
    uint32_t bias = 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)((u + bias) >> 16);
}

uint16_t orc_bf16_from_f32(float f) { return orc_narrow(f); }
float orc_f32_from_bf16(uint16_t h) { return orc_widen(h); }

/* ---------------------------------------------------------------- one-shot all-reduce
 * AR:53-64: for every element, acc = 0; for i in 0..W-1: acc += buf_i[j]; out[j] = acc.
 * Contract arithmetic: fp32 accumulate, one rounding. */
void orc_all_reduce_bf16(const uint16_t *const *bufs, int world, uint16_t *out, size_t numel)
{
#pragma omp parallel for schedule(static)
    for (ptrdiff_t j = 0; j < (ptrdiff_t)numel; ++j) {
        float acc = 0.0f;
        for (int i = 0; i < world; ++i)
            acc = acc + orc_widen(bufs[i][j]);
        out[j] = orc_narrow(acc);
    }
}

/* fp32 inputs: same loop, no final rounding. */
void orc_all_reduce_f32(const float *const *bufs, int world, float *out, size_t numel)
{
#pragma omp parallel for schedule(static)
    for (ptrdiff_t j = 0; j < (ptrdiff_t)numel; ++j) {
        float acc = 0.0f;
        for (int i = 0; i < world; ++i)
            acc = acc + bufs[i][j];
        out[j] = acc;
    }
}

/* Information only: the reference's own arithmetic (AR:22-23, RS:43-46), running sum
 * re-rounded to bf16 after every rank. */
void orc_all_reduce_bf16_stepwise(const uint16_t *const *bufs, int world, uint16_t *out, size_t numel)
{
#pragma omp parallel for schedule(static)
    for (ptrdiff_t j = 0; j < (ptrdiff_t)numel; ++j) {
        uint16_t acc = 0;
        for (int i = 0; i < world; ++i)
            acc = orc_narrow(orc_widen(acc) + orc_widen(bufs[i][j]));
        out[j] = acc;
    }
}

/* ---------------------------------------------------------------- reduce-scatter
 * RS:73, RS:86: per_rank = numel // world; source of rank r's share is
 * buf_i + r*per_rank; RS:83-88 zero start and rank order.  out has per_rank elements. */
void orc_reduce_scatter_bf16(const uint16_t *const *bufs, int world, int rank, uint16_t *out, size_t numel_total)
{
    size_t per_rank = numel_total / (size_t)world;
    const uint16_t *shifted[64];
    for (int i = 0; i < world; ++i)
        shifted[i] = bufs[i] + (size_t)rank * per_rank;
    orc_all_reduce_bf16(shifted, world, out, per_rank);
}

void orc_reduce_scatter_f32(const float *const *bufs, int world, int rank, float *out, size_t numel_total)
{
    size_t per_rank = numel_total / (size_t)world;
    const float *shifted[64];
    for (int i = 0; i < world; ++i)
        shifted[i] = bufs[i] + (size_t)rank * per_rank;
    orc_all_reduce_f32(shifted, world, out, per_rank);
}

/* ---------------------------------------------------------------- all-gather
 * AG:54-62 with the output laid out [world, numel] row-major (AG:82): row i is a byte
 * copy of buf_i. */
void orc_all_gather(const void *const *bufs, int world, void *out, size_t bytes_per_rank)
{
    for (int i = 0; i < world; ++i)
        memcpy((char *)out + (size_t)i * bytes_per_rank, bufs[i], bytes_per_rank);
}

/* ---------------------------------------------------------------- double-tree node step
 * Reduce step as designed in DT:274-294 with the commented child adds DT:276-288:
 * acc = 0; if child0: acc += child0[j]; if child1: acc += child1[j]; acc += own[j];
 * dst[j] = acc (the reference stores back into own, DT:293-294; dst may alias own).
 * A NULL child is the reference's -1. */
void orc_tree_reduce_step_bf16(const uint16_t *own, const uint16_t *child0, const uint16_t *child1,
                               uint16_t *dst, size_t numel)
{
#pragma omp parallel for schedule(static)
    for (ptrdiff_t j = 0; j < (ptrdiff_t)numel; ++j) {
        float acc = 0.0f;
        if (child0) acc = acc + orc_widen(child0[j]);
        if (child1) acc = acc + orc_widen(child1[j]);
        acc = acc + orc_widen(own[j]);
        dst[j] = orc_narrow(acc);
    }
}

void orc_tree_reduce_step_f32(const float *own, const float *child0, const float *child1,
                              float *dst, size_t numel)
{
#pragma omp parallel for schedule(static)
    for (ptrdiff_t j = 0; j < (ptrdiff_t)numel; ++j) {
        float acc = 0.0f;
        if (child0) acc = acc + child0[j];
        if (child1) acc = acc + child1[j];
        acc = acc + own[j];
        dst[j] = acc;
    }
}

/* Broadcast step DT:314-325 (commented design): own <- parent, output <- parent. */
void orc_tree_copy_step(const void *src, void *dst0, void *dst1, size_t bytes)
{
    if (dst1) memcpy(dst1, src, bytes);
    if (dst0 != src) memmove(dst0, src, bytes);
}

/* ---------------------------------------------------------------- tree index math
 * TREE:5-31.  Rows are built from the leaves up: the leaf row is the odd ranks, every
 * higher row is the midpoint of adjacent pairs of the row below; rows are prepended;
 * finally the extra node 0 is put in front.  Returns 0, or -1 if n is not a power of
 * two >= 2 (the reference asserts the power of two, TREE:11, and fails for n == 1 at
 * TREE:135). */
int orc_build_tree(int n, int *tree /* n entries */)
{
    if (n < 2 || (n & (n - 1)) != 0)
        return -1;
    int height = 0;
    while ((1 << height) < n) ++height;
    int row[n], prev[n];
    int prev_len = 0;
    int end = n;                     /* rows are written right-to-left into tree[1..n-1] */
    for (int h = 0; h < height; ++h) {
        int len = 0;
        if (h == 0) {
            for (int i = 0; i < n; ++i)
                if (i % 2 != 0) row[len++] = i;
        } else {
            for (int i = 0; i + 1 < prev_len; i += 2)
                row[len++] = (prev[i] + prev[i + 1]) / 2;
        }
        end -= len;
        for (int i = 0; i < len; ++i) tree[end + i] = row[i];
        for (int i = 0; i < len; ++i) prev[i] = row[i];
        prev_len = len;
    }
    tree[0] = 0;
    return end == 1 ? 0 : -2;
}

/* TREE:83-91: b is a with 1 subtracted from every entry, the subroot wrapping to n-1. */
int orc_build_double_tree(int n, int *tree_a, int *tree_b)
{
    int rc = orc_build_tree(n, tree_a);
    if (rc) return rc;
    for (int i = 0; i < n; ++i) tree_b[i] = tree_a[i] - 1;
    if (tree_b[0] != -1) return -3;
    tree_b[0] = n - 1;
    return 0;
}

/* TREE:130-146 for one tree: position of rank in the heap-ordered array; the subroot
 * (position 0) has the single child at position 1; otherwise parent = pos/2, children
 * 2pos and 2pos+1 when inside the array. */
static void orc_one_tree(const int *tree, int n, int rank, int *out3)
{
    int pos = -1;
    for (int i = 0; i < n; ++i)
        if (tree[i] == rank) { pos = i; break; }
    if (pos == 0) {
        out3[0] = -1; out3[1] = tree[1]; out3[2] = -1;
        return;
    }
    out3[0] = tree[pos / 2];
    out3[1] = (2 * pos < n) ? tree[2 * pos] : -1;
    out3[2] = (2 * pos + 1 < n) ? tree[2 * pos + 1] : -1;
}

/* TREE:93-148: (a_parent, a_child0, a_child1, b_parent, b_child0, b_child1). */
int orc_get_parents_and_children(int n, int rank, int *out6)
{
    if (rank < 0 || rank >= n) return -4;
    int a[n], b[n];
    int rc = orc_build_double_tree(n, a, b);
    if (rc) return rc;
    orc_one_tree(a, n, rank, out6);
    orc_one_tree(b, n, rank, out6 + 3);
    return 0;
}

/* ---------------------------------------------------------------- full double tree
 * Split point between the half reduced over tree a and the half reduced over tree b:
 * floor(numel/2) rounded down to a whole number of 16-byte vectors. */
size_t orc_double_tree_split(size_t numel, size_t esize)
{
    size_t per_vec = 16 / esize;
    return (numel / 2) / per_vec * per_vec;
}

/* One tree over elements [lo, hi): up-sweep in place (every node applies the reduce
 * step to its own buffer, children first: heap positions n-1 .. 1, then the subroot),
 * then the result held by the subroot is copied into every rank's buffer and output
 * (DT:314-325).  Leaves run the step too (DT:274-294 runs it for every rank). */
static void orc_one_tree_all_reduce_bf16(uint16_t *const *bufs, uint16_t *const *outs, int n,
                                         const int *tree, size_t lo, size_t hi)
{
    size_t len = hi - lo;
    if (len == 0) return;
    for (int pos = n - 1; pos >= 0; --pos) {
        int t[3];
        orc_one_tree(tree, n, tree[pos], t);
        uint16_t *own = bufs[tree[pos]] + lo;
        orc_tree_reduce_step_bf16(own, t[1] >= 0 ? bufs[t[1]] + lo : NULL,
                                  t[2] >= 0 ? bufs[t[2]] + lo : NULL, own, len);
    }
    const uint16_t *res = bufs[tree[0]] + lo;
    for (int r = 0; r < n; ++r) {
        if (outs && outs[r]) memcpy(outs[r] + lo, res, len * 2);
        if (r != tree[0]) memcpy(bufs[r] + lo, res, len * 2);
    }
}

/* Whole collective for all n virtual ranks: bufs are overwritten (as in the reference's
 * design, DT:293-294 and DT:321-323); outs[r] receives rank r's output (DT:324-325). */
int orc_double_tree_all_reduce_bf16(uint16_t *const *bufs, uint16_t *const *outs, int n, size_t numel)
{
    int a[n], b[n];
    int rc = orc_build_double_tree(n, a, b);
    if (rc) return rc;
    size_t split = orc_double_tree_split(numel, 2);
    orc_one_tree_all_reduce_bf16(bufs, outs, n, a, 0, split);
    orc_one_tree_all_reduce_bf16(bufs, outs, n, b, split, numel);
    return 0;
}
