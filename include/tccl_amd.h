/*
 * tccl_amd.h -- C ABI of the MI355X (gfx950) data path for tccl-style collectives.
 *
 * One GPU holds W "virtual ranks": W separate device allocations stand in for the
 * symmetric-memory peer buffers of the reference.  Every entry point below replaces one
 * Triton kernel launch (or one host helper) of the reference; the file:line each one
 * replaces is given with it (paths relative to the reference checkout).
 *
 * Conventions
 *   - plain C: pointers and sizes only, no torch types.
 *   - every device pointer must be 16-byte aligned; `stream` is a hipStream_t passed as
 *     void* (NULL = the null stream).
 *   - calls are asynchronous on `stream`, allocate no device memory, never synchronise and
 *     never throw; the return value is TCCL_OK or a negative code (tccl_error_string()).
 *     Every launching entry point can be recorded into a caller's HIP graph.
 *   - ordering between virtual ranks and between tree levels is stream order; this
 *     replaces the reference's signal-pad barrier (triton_barrier.py:39-142) and its
 *     wait/send flags (triton_double_tree_allreduce.py:175-225).  Two entry points keep the
 *     device-side protocol instead, between the virtual ranks' workgroups of one launch:
 *     tccl_double_tree_all_reduce_pipelined() and tccl_two_shot_all_reduce(); they take
 *     signal pads.  Where every rank is a process of its own on the same GPU (buffers and pads
 *     exchanged with tccl_ipc_export/open), the same protocol runs between one launch per rank,
 *     as in the reference: tccl_blockwise_barrier(), tccl_double_tree_all_reduce_pipelined_rank(),
 *     tccl_two_shot_all_reduce_rank(), and -- with the barrier inside the kernel, as the reference's
 *     kernels have it -- tccl_all_reduce_sum_rank(), tccl_reduce_scatter_sum_rank(), tccl_all_gather_rank().
 *   - float sums: each bf16 is widened to fp32, accumulated from +0.0f in the order the
 *     sources are given, and rounded once (round-to-nearest-even) on store.  NaN sign
 *     and payload are not specified.
 */
#ifndef TCCL_AMD_H
#define TCCL_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TCCL_ABI_VERSION 2

/* Largest number of source buffers one launch can take (virtual world size). */
#define TCCL_MAX_WORLD 8
/* Largest number of node steps one tccl_tree_level() launch can take. */
#define TCCL_MAX_JOBS 8
/* Largest world tccl_double_tree_all_reduce() runs (a node step reads at most 3 buffers, so
 * the tree is not bound by TCCL_MAX_WORLD). */
#define TCCL_MAX_TREE_RANKS 64
/* Largest world the host-side tree index math accepts. */
#define TCCL_MAX_TREE_WORLD (1 << 20)

enum {
    TCCL_OK = 0,
    TCCL_EINVAL = -1,      /* NULL pointer, world/rank/dtype out of range, size mismatch */
    TCCL_EALIGN = -2,      /* a pointer or a row size is not a multiple of 16 bytes */
    TCCL_EPOW2 = -3,       /* tree world size is not a power of two >= 2 */
    TCCL_ESCRATCH = -4,    /* the request needs more scratch memory than the library's static buffer holds */
    TCCL_ETIMEOUT = -5,    /* a wait of a signalling kernel expired (reported by host wrappers, never by a launch) */
    TCCL_EHIP_BASE = -1000 /* -(1000 + hipError_t) */
};

typedef enum {
    TCCL_BF16 = 0, /* bf16 in/out, fp32 accumulate, one RNE rounding */
    TCCL_F32 = 1   /* fp32 in/out, fp32 accumulate */
} tccl_dtype_t;

/* Launch shape override, for tuning and tests.  Any field left 0 is chosen by the
 * library (all fields 0 is the same as passing NULL: the library's own launch plans
 * apply).  The reference hard-codes its shape in each wrapper
 * (triton_one_shot_all_reduce_no_128.py:68-71: 24 blocks x 512 lanes). */
typedef struct {
    int block;      /* threads per workgroup: 64, 128, 256 or 512 */
    int unroll;     /* independent 16-byte vectors per thread per iteration: 1, 2 or 4 */
    int grid;       /* workgroups */
    int tile_iters; /* consecutive iterations a workgroup spends on one contiguous tile */
    int flags;      /* TCCL_CFG_* */
} tccl_launch_cfg;

#define TCCL_CFG_NONTEMPORAL_LOAD 1  /* mark loads as streaming */
#define TCCL_CFG_NONTEMPORAL_STORE 2 /* mark stores as streaming */
#define TCCL_CFG_XCD_CONTIGUOUS 4    /* give each of the 8 XCDs one contiguous eighth of the tiles */
#define TCCL_CFG_TEMPORAL 8          /* force plain (cached) loads and stores */
#define TCCL_CFG_STREAMING 16        /* force the grid-stride kernel (stores interleaved with loads) */
#define TCCL_CFG_PHASED 32           /* force the phased kernel (each workgroup reads its whole tile,
                                        then writes it); there `grid` = workgroups per launch and
                                        `tile_iters` = iterations per tile, `unroll` = vectors per lane per
                                        iteration (iterations * unroll <= 32), block unused */

int tccl_abi_version(void);
const char *tccl_error_string(int code);

/* One-shot all-reduce (sum): out[j] = sum_{i<world} bufs[i][j].
 * Replaces one_shot_all_reduce_kernel, triton_one_shot_all_reduce_no_128.py:35-64
 * (launched at :85-95).  `bufs` is a HOST array of `world` device pointers (the
 * reference's symm_mem.buffer_ptrs_dev, :86, passed here by value into the kernel
 * arguments).  1 <= world <= TCCL_MAX_WORLD.  `numel` may be any value; elements past
 * the last whole 16-byte vector are summed one at a time. */
int tccl_all_reduce_sum(const void *const *bufs, int world, void *out, size_t numel,
                        int dtype, void *stream);
int tccl_all_reduce_sum_ex(const void *const *bufs, int world, void *out, size_t numel,
                           int dtype, void *stream, const tccl_launch_cfg *cfg);

/* One rank's share of a reduce-scatter: out[j] = sum_i bufs[i][rank*P + j],
 * P = numel_total / world, j < P.
 * Replaces one_shot_reduce_scatter_kernel, triton_reduce_scatter.py:59-92 (launched at
 * :116-126).  numel_total must be a multiple of world and P*esize a multiple of 16 (the
 * reference requires numel % (8*world) == 0, :101-104); TCCL_EALIGN otherwise, for every rank
 * alike. */
int tccl_reduce_scatter_sum(const void *const *bufs, int world, int rank, void *out,
                            size_t numel_total, int dtype, void *stream);
int tccl_reduce_scatter_sum_ex(const void *const *bufs, int world, int rank, void *out,
                               size_t numel_total, int dtype, void *stream,
                               const tccl_launch_cfg *cfg);

/* All-gather pack: out is [world, bytes_per_rank] row-major, row i = bufs[i].
 * Replaces one_shot_all_gather_kernel, triton_all_gather.py:32-63 (launched at :84-94;
 * output layout :82).  Typeless byte copy; bytes_per_rank % 16 == 0. */
int tccl_all_gather(const void *const *bufs, int world, void *out, size_t bytes_per_rank,
                    void *stream);
int tccl_all_gather_ex(const void *const *bufs, int world, void *out, size_t bytes_per_rank,
                       void *stream, const tccl_launch_cfg *cfg);

/* Double-tree node step, reduce half: dst[j] = 0 + child0[j] + child1[j] + own[j] in that
 * order; a NULL child is skipped (the reference's -1).  dst may be `own` (the reference
 * stores in place, triton_double_tree_allreduce.py:293-294).
 * Replaces the reduce loop of double_tree_all_reduce_kernel,
 * triton_double_tree_allreduce.py:266-295 including the child adds at :276-288. */
int tccl_tree_reduce_step(const void *own, const void *child0, const void *child1, void *dst,
                          size_t numel, int dtype, void *stream);

/* Double-tree node step, forward/broadcast half: dst0[j] = dst1[j] = src[j]; dst1 may be
 * NULL.  Replaces the broadcast loop sketched at
 * triton_double_tree_allreduce.py:306-326 (own <- parent, output <- parent).
 * bytes % 16 == 0. */
int tccl_tree_copy_step(const void *src, void *dst0, void *dst1, size_t bytes, void *stream);

/* A batch of independent node steps in ONE launch (all nodes of one tree level, both
 * trees).  No counterpart in the reference, where each rank's kernel does its own step;
 * on one GPU the steps of a level are independent and share a launch.  No job may write
 * what another job of the same batch reads or writes.  Reduce steps are worked in tiles of
 * at most 32 KiB (read and reduce the tile, then write it); a batch of copy steps only is
 * walked job after job by one workgroup per compute unit. */
typedef struct {
    const void *src[3]; /* reduce: child0, child1, own (NULL = absent); copy: src[0] only */
    void *dst[2];       /* dst[1] may be NULL */
    size_t numel;       /* elements of `dtype` */
    int is_copy;        /* 0 = reduce step, 1 = copy step (bit-exact, no arithmetic) */
    int pad_;
} tccl_node_job;

int tccl_tree_level(const tccl_node_job *jobs, int njobs, int dtype, size_t chunk_elems,
                    void *stream);

/* Tree index math (host only, no GPU needed).
 * tccl_double_tree_arrays  replaces build_double_tree, tree.py:34-91 (heap-ordered arrays).
 * tccl_double_tree_indices replaces get_parents_and_children, tree.py:93-148:
 *   out6 = (a_parent, a_child0, a_child1, b_parent, b_child0, b_child1), -1 = none.
 * world must be a power of two >= 2 (tree.py:11; world == 1 fails in the reference at
 * tree.py:135). */
int tccl_double_tree_arrays(int world, int *tree_a, int *tree_b);
int tccl_double_tree_indices(int world, int rank, int *out6);

/* First element of the half that tree b reduces: floor(numel/2) rounded down to whole
 * 16-byte vectors.  Tree a owns [0, split), tree b owns [split, numel). */
size_t tccl_double_tree_split(size_t numel, size_t esize);

/* The whole double-tree all-reduce for all `world` virtual ranks, as the sequence of node
 * steps that triton_double_tree_allreduce.py:254-335 (live and commented code) describes,
 * one launch per tree level with both trees in it, ordered by the stream:
 * up-sweep  -- each interior node reduces its children's buffers into its own, in place;
 * down-sweep -- each rank copies its parent's buffer into its own buffer and its output.
 * bufs[r] is overwritten with the result (as in the reference's design, :293-294 and
 * :321-323); outs[r] (nullable entries) receive rank r's output (:324-325).  `world` is a
 * power of two, 2..TCCL_MAX_TREE_RANKS.  chunk_elems = elements per pipelining chunk
 * (0 = 128 KiB worth); a chunk is worked on in tiles of at most 32 KiB, one workgroup each. */
int tccl_double_tree_all_reduce(void *const *bufs, void *const *outs, int world, size_t numel,
                                int dtype, size_t chunk_elems, void *stream);

/* The same collective in ONE launch, for worlds of 2, 4 or 8 whose buffers all live on this
 * GPU: each lane loads its 16-byte vector from all `world` buffers, reduces it in registers
 * in the tree's order with the tree's rounding (one rounding per node, exactly the values
 * the node steps produce), and stores the result into every buffer and every output.  It
 * moves world reads + 2*world writes per element instead of the schedule's level-by-level
 * traffic and needs no ordering between launches, which is what bounds small inputs.  No
 * counterpart in the reference (a rank there cannot read every peer's buffer for free);
 * it leaves memory in the same final state as tccl_double_tree_all_reduce(). */
int tccl_double_tree_all_reduce_fused(void *const *bufs, void *const *outs, int world, size_t numel,
                                      int dtype, void *stream);

/* The same collective recorded once into a HIP graph and replayed with one launch, for
 * callers that repeat it on the same buffers (its 2*log2(world) launches cost more than
 * its kernels below a few MiB).  No counterpart in the reference, whose whole collective
 * is one kernel per rank.  Creating a plan allocates host and driver memory (never device
 * memory) and does not run anything; launching it is asynchronous on `stream`.  A plan
 * holds the addresses it was created with: the buffers must stay allocated. */
typedef struct tccl_plan tccl_plan;
int tccl_double_tree_plan_create(void *const *bufs, void *const *outs, int world, size_t numel,
                                 int dtype, size_t chunk_elems, tccl_plan **plan_out);
int tccl_plan_launch(tccl_plan *plan, void *stream);
int tccl_plan_destroy(tccl_plan *plan);

/* The same collective as ONE persistent launch with device-side signalling, for worlds of
 * 2, 4 or 8: each virtual rank owns a share of the grid's workgroups, which walk the
 * pipelining chunks of both trees and run the per-rank program the reference's kernel is
 * designed as (triton_double_tree_allreduce.py:254-335): wait for the children's chunk,
 * reduce it with the own chunk in place, signal the parent; wait for the parent's result,
 * copy it into the own buffer and the output, signal the children.  Replaces the
 * wait/send pair of triton_double_tree_allreduce.py:175-225 and the signal-pad addressing
 * of triton_barrier.py:39-142 (a sender writes into the RECEIVER's pad, the receiver polls
 * its own pad and resets the slot), with one slot per (tree, chunk, sender) so that a send
 * never blocks.  Leaves memory in the same final state as tccl_double_tree_all_reduce().
 * chunk_elems = elements per pipelining chunk, the unit that is signalled (whole 16-byte
 * vectors); 0 = 32 KiB worth (the measured optimum for large inputs), halved down to 4 KiB
 * while a tree would have fewer than 256 chunks (a chunk crosses up to 2*log2(world)
 * dependent steps, so small inputs want many small chunks in flight).
 *
 * signal_pads: HOST array of `world` device pointers (the reference's
 *   symm_mem.signal_pad_ptrs_dev), each to pad_bytes >= tccl_double_tree_signal_pad_bytes()
 *   bytes, 16-byte aligned and ZERO-FILLED before the first call.  A completed call leaves
 *   them zero-filled again.  The last TCCL_PAD_CONTROL_WORDS 32-bit words of pad 0 are control
 *   words (counters from which the workgroups draw their places, and -- the very last word,
 *   at pad_bytes - 4 -- the count of time-outs).
 * Waits are bounded (cfg->spin_limit pauses of about 0.2 us; polls back off from one pause to 128
 * between two polls while a flag stays away): a workgroup whose signal never comes counts a
 *   time-out and leaves the kernel, and so does everyone who waits for it, so the launch
 *   always ends; the buffers then hold partial results and the pads must be cleared by the
 *   caller.  tccl_signal_pad_timeouts() reads the count (it synchronises the stream); a caller
 *   that must not synchronise passes cfg->timeout_flag, a word in pinned host memory that the
 *   kernel sets to 1 when a wait expires, and looks at it whenever it likes (for instance
 *   before its next call).
 * Forward progress.  By default workgroup b of the grid works as rank b / (workgroups per
 *   rank): that binding is the fastest on large inputs, but a workgroup then waits for
 *   workgroups anywhere in the grid, so the whole grid must be resident at once.  The library
 *   never launches more workgroups than the occupancy HIP reports for the kernel; should other
 *   work keep part of the GPU busy for longer than spin_limit allows, waits expire and are
 *   reported as above.  With TCCL_PIPE_DRAW_PLACES in cfg->flags forward progress does not
 *   depend on residency: a workgroup draws its place (rank, index) from a counter when it starts
 *   to run, and only waits for the workgroups with the same index of the other ranks, whose
 *   places are drawn next to its own -- they are all running once any later place has been
 *   drawn, and at most 56 workgroups can ever sit waiting for one that has not started.  Use
 *   it when these kernels overlap with other kernels on the same GPU; it measured up to 15 %
 *   slower at 64-256 MiB per buffer on an otherwise idle GPU and the same below 16 MiB.
 *   Two signalling launches that overlap on one GPU slow each other down; calls made by one
 *   process are kept apart by the library (each launch makes its stream wait for the previous
 *   signalling kernel of the device, on whatever stream that ran).  Two launches must never
 *   share signal pads at the same time. */
#define TCCL_PAD_CONTROL_WORDS 288
typedef struct {
    int workgroups;      /* total workgroups (all ranks); 0 = chosen by the library */
    int lag;             /* 1 + rounds the down-sweep runs behind the up-sweep; 0 = default (1: none) */
    unsigned spin_limit; /* pauses of about 0.2 us before a wait gives up; 0 = default (about half a second) */
    int tile_kib;        /* a workgroup works a chunk in tiles of 32 (default) or 128 KiB */
    uint32_t *timeout_flag; /* NULL, or a device-visible 32-bit word (pinned host memory, e.g. from
                               tccl_timeout_flag_create) that is set to 1 when a wait expires */
    int flags;           /* TCCL_PIPE_* */
    int pad_;
} tccl_pipeline_cfg;

#define TCCL_PIPE_DRAW_PLACES 1 /* workgroups draw their places when they start (see above) */
#define TCCL_PIPE_OWN_BARRIERS 2 /* tccl_two_shot_all_reduce_rank and tccl_double_tree_all_reduce_pipelined_rank:
                                    the kernel begins and ends with the blockwise barrier itself (see there) */

size_t tccl_double_tree_signal_pad_bytes(int world, size_t numel, int dtype, size_t chunk_elems);
int tccl_double_tree_all_reduce_pipelined(void *const *bufs, void *const *outs,
                                          void *const *signal_pads, size_t pad_bytes, int world,
                                          size_t numel, int dtype, size_t chunk_elems,
                                          const tccl_pipeline_cfg *cfg, void *stream);
/* The same kernel as ONE RANK's launch: the form the reference runs it in
 * (triton_double_tree_allreduce.py:338-370, one kernel per rank, the ranks meeting through
 * wait/send on pads in each other's memory, :175-225).  Every rank -- a process of its own on
 * the same GPU -- makes this call with its own `rank`; bufs and signal_pads are the same tables
 * in every rank's address space (peers' entries as opened with tccl_ipc_open), `out` is this
 * rank's output (may be NULL).  (Ranks that share a process use the one-launch form above: the
 * library runs a process's signalling launches one after the other, so they could never meet.)  The W launches must be able to run
 * at the same time (each holds 1/world of the workgroups that fit the GPU) and must all be given
 * the same numel, dtype, chunk_elems and cfg.  Between two collectives on the same buffers and
 * pads every rank must have finished the first before any rank starts the second (and the inputs
 * must be in place before any rank starts): either TCCL_PIPE_OWN_BARRIERS in cfg->flags -- the
 * kernel then begins with the blockwise barrier, as the reference's does
 * (triton_double_tree_allreduce.py:239), and ends with one, on slots of their own behind the
 * chunks' (the size tccl_double_tree_signal_pad_bytes() returns has room for them; at most 512
 * workgroups per rank) -- or tccl_blockwise_barrier() before and after.  TCCL_PIPE_DRAW_PLACES does
 * not apply (TCCL_EINVAL).  Time-outs, pads, chunking, arithmetic: as above. */
int tccl_double_tree_all_reduce_pipelined_rank(void *const *bufs, void *out, void *const *signal_pads,
                                               size_t pad_bytes, int world, int rank, size_t numel,
                                               int dtype, size_t chunk_elems,
                                               const tccl_pipeline_cfg *cfg, void *stream);
int tccl_signal_pad_timeouts(const void *pad0, size_t pad_bytes, unsigned *timeouts_out,
                             void *stream);

/* Two-shot all-reduce for all virtual ranks in ONE launch, in place: afterwards every
 * bufs[r] (and every outs[r], if given) holds sum_i bufs[i] -- each element the fp32 sum in
 * rank order rounded once, bit-identical to tccl_all_reduce_sum().  Shot 1: rank r's
 * workgroups reduce share r (numel / world elements) from all buffers into their own buffer;
 * then the reference's blockwise barrier (triton_barrier.py:39-142: workgroup g of every
 * rank signals workgroup g of every other rank through slot `g * world + sender` of the
 * receiver's pad and waits for the same from them); shot 2: every rank copies the other
 * shares from their owners' buffers.  This is the reduce-scatter + all-gather composition
 * the reference's slides name for large messages, as one kernel; it moves (3*world - 1)/world
 * buffers per rank instead of the (world + 1) of a one-shot all-reduce per rank.
 * 1 <= world <= TCCL_MAX_WORLD; numel % (world * 16 / esize) == 0 (whole vectors per share,
 * the reduce-scatter's precondition).  signal_pads / pad_bytes / time-outs / residency: as for
 * tccl_double_tree_all_reduce_pipelined; pad_bytes >= 4 * (world + TCCL_PAD_CONTROL_WORDS) is
 * enough, larger pads allow more workgroups per rank (cfg->lag and cfg->tile_kib are unused). */
int tccl_two_shot_all_reduce(void *const *bufs, void *const *outs, void *const *signal_pads,
                             size_t pad_bytes, int world, size_t numel, int dtype,
                             const tccl_pipeline_cfg *cfg, void *stream);
/* The same kernel as ONE RANK's launch, for ranks that are processes of their own on the same
 * GPU (see tccl_double_tree_all_reduce_pipelined_rank for the calling rules: same arguments in
 * every rank, the W launches running at the same time, tccl_blockwise_barrier() before and
 * after).  The barrier between the two shots is then exactly the reference's construct: a
 * blockwise barrier between kernels of different owners (triton_barrier.py:39-142), inside the
 * kernel.  `out` = this rank's output or NULL (the result is in bufs[rank] either way).
 * With TCCL_PIPE_OWN_BARRIERS in cfg->flags the kernel also begins and ends with that barrier, as
 * the reference's kernels begin with it (triton_one_shot_all_reduce_no_128.py:46), and no
 * tccl_blockwise_barrier() before or after is needed: one launch per rank per collective.  The pads
 * then hold three rows of slots per workgroup, pad_bytes >= 4 * (3 * world + TCCL_PAD_CONTROL_WORDS);
 * calls that follow each other without a host-side meeting of the ranks in between must be given
 * the same pad_bytes and world, which fix where a workgroup's rows lie, and pads of their own (not
 * those of the one-shot or double-tree entry points).
 * An empty input launches nothing and orders nothing. */
int tccl_two_shot_all_reduce_rank(void *const *bufs, void *out, void *const *signal_pads,
                                  size_t pad_bytes, int world, int rank, size_t numel, int dtype,
                                  const tccl_pipeline_cfg *cfg, void *stream);

/* The three one-shot collectives as ONE RANK's launch with the reference's barrier inside the
 * kernel, for ranks that are processes of their own on the same GPU: each replaces one of the
 * reference's per-rank launches together with the blockwise_barrier its kernel begins with --
 *   tccl_all_reduce_sum_rank      one_shot_all_reduce_kernel, triton_one_shot_all_reduce_no_128.py:35-64 (barrier :46)
 *   tccl_reduce_scatter_sum_rank  one_shot_reduce_scatter_kernel, triton_reduce_scatter.py:59-92 (barrier :70, commented out there)
 *   tccl_all_gather_rank          one_shot_all_gather_kernel, triton_all_gather.py:32-63 (barrier :43)
 * Workgroup g of this rank's launch meets workgroup g of every other rank's launch (every
 * rank's buffer is filled, and what was written to it is visible), pulls its tiles from all
 * `world` buffers (device-scope loads: a peer's producer kernel may end after this kernel
 * started), writes this rank's `out` -- the results of tccl_all_reduce_sum,
 * tccl_reduce_scatter_sum and tccl_all_gather, bit for bit -- and meets its peers again: when a
 * rank's kernel has ended, every rank has read that rank's buffer and it may be refilled (the
 * trailing barrier the reference lacks).  No barrier launch before or after is needed.
 * Calling rules: every rank makes the same call with its own `rank` and `out`; bufs and
 * signal_pads are the same tables in every rank's address space (HOST arrays of `world` device
 * pointers, peers' entries as opened with tccl_ipc_open); the W launches must be able to run at
 * the same time (each takes 1/world of the workgroups that fit the GPU, so ranks that share a
 * stream or a hardware queue can never meet) and must be given the same sizes and the same
 * cfg->workgroups (the total over all ranks, as always; 0 = chosen by the library, the same in
 * every rank).  Pads: zero-filled before the first use, left zero-filled by every completed
 * call, pad_bytes >= 4 * (2 * world + TCCL_PAD_CONTROL_WORDS) (two rows of slots per workgroup:
 * the leading and the trailing barrier alternate between them, so a flag is never raised over
 * one that has not been consumed); larger pads allow more workgroups per rank.  The same pads
 * may serve any sequence of these three calls, of any sizes, as long as every call is given the
 * same pad_bytes and world (they fix where a workgroup's two rows lie); they may not be shared
 * with the two-shot or double-tree entry points, which lay their rows out differently.  Waits are bounded (cfg->spin_limit, cfg->timeout_flag, the
 * time-out count in the last word of pad 0): a rank whose peers do not arrive gives up, leaves
 * `out` unwritten or partly written, and says so.  TCCL_PIPE_DRAW_PLACES does not apply
 * (TCCL_EINVAL); cfg->lag and cfg->tile_kib are unused.  Preconditions on the sizes as for the
 * entry points without _rank. */
int tccl_all_reduce_sum_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes,
                             int world, int rank, size_t numel, int dtype,
                             const tccl_pipeline_cfg *cfg, void *stream);
int tccl_reduce_scatter_sum_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes,
                                 int world, int rank, size_t numel_total, int dtype,
                                 const tccl_pipeline_cfg *cfg, void *stream);
int tccl_all_gather_rank(void *const *bufs, void *out, void *const *signal_pads, size_t pad_bytes,
                         int world, int rank, size_t bytes_per_rank,
                         const tccl_pipeline_cfg *cfg, void *stream);

/* tccl_two_shot_all_reduce() for callers that cannot allocate the signal pads it needs -- code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same operation, same results, same cfg; the signal pads live
 * in a static device array inside the library (TCCL_STATIC_SCRATCH_BYTES per GPU, held from
 * the moment the library is loaded until the process ends), and the call allocates nothing on
 * the device or the host: it enqueues one small kernel that clears the pads and then the
 * all-reduce itself.  (Set-up, once per device: the first call looks up the array's device
 * address, and the first signalling launch of the process outside graph capture creates the
 * one HIP event with which the library chains such launches.)  Limits: world <= TCCL_MAX_WORLD and at most TCCL_STATIC_MAX_WORKGROUPS
 * workgroups per rank; a cfg->workgroups beyond world * TCCL_STATIC_MAX_WORKGROUPS is refused
 * with TCCL_ESCRATCH (numel itself is not limited: the pads hold one flag per workgroup and
 * peer, whatever the size).  Every call on a GPU uses that GPU's one array: calls that overlap
 * in time on one GPU (two streams, two threads, two replaying graphs) race and must be kept
 * apart by the caller; calls of one process outside graph capture are chained by the library
 * like every signalling launch.  Time-outs are reported through cfg->timeout_flag only. */
#define TCCL_STATIC_MAX_WORKGROUPS 1024
#define TCCL_STATIC_SCRATCH_BYTES \
    ((TCCL_STATIC_MAX_WORKGROUPS * TCCL_MAX_WORLD + TCCL_PAD_CONTROL_WORDS) * 4 * TCCL_MAX_WORLD)
int tccl_two_shot_all_reduce_static(void *const *bufs, void *const *outs, int world, size_t numel, int dtype,
                                    const tccl_pipeline_cfg *cfg, void *stream);

/* A word for tccl_pipeline_cfg.timeout_flag: 32 bits of pinned, device-visible host memory,
 * zero to begin with.  The caller reads (and zeroes) it through the pointer.  Creating one
 * allocates host memory; no counterpart in the reference, whose waits spin for ever
 * (triton_barrier.py:108-118). */
int tccl_timeout_flag_create(uint32_t **flag_out);
int tccl_timeout_flag_destroy(uint32_t *flag);

/* Buffers that several processes on one GPU can map: what the reference gets from
 * _SymmetricMemory.empty_strided_p2p (triton_one_shot_all_reduce_no_128.py:116-122) and
 * rendezvous (:82).  tccl_symm_alloc returns a zero-filled device allocation of its own (below
 * 2 GiB; it waits for the null stream, so the zeros are in place before a peer can map it);
 * tccl_ipc_export writes its 64-byte handle, which the host side carries to the peers;
 * tccl_ipc_open maps a peer's allocation into this process and returns its address here, good for
 * every pointer table of this header; tccl_ipc_close unmaps it.  These four calls allocate, map or
 * synchronise: they belong to set-up, not to the hot path. */
#define TCCL_IPC_HANDLE_BYTES 64
int tccl_symm_alloc(size_t bytes, void **ptr_out);
int tccl_symm_free(void *ptr);
int tccl_ipc_export(void *ptr, unsigned char *handle_out /* TCCL_IPC_HANDLE_BYTES */);
int tccl_ipc_open(const unsigned char *handle /* TCCL_IPC_HANDLE_BYTES */, void **ptr_out);
int tccl_ipc_close(void *ptr);

/* The reference's blockwise_barrier (triton_barrier.py:39-142) as a launch of its own, one per
 * rank: rank `rank`'s kernel raises slot `block * world + rank` in every peer's pad and waits for
 * slot `block * world + peer` of its own pad, which it lowers again; `blocks` independent rows of
 * slots (the reference has one per workgroup of the collective's kernel).  Everything this rank
 * enqueued on `stream` before the call is complete and visible to the peers' work that follows
 * their call, and the other way round (the guarantee of triton_barrier.py:56-66); called again
 * after a collective it is the trailing barrier the reference lacks.  signal_pads: HOST array of
 * `world` device pointers, own pad at index `rank`, the peers' pads as opened with tccl_ipc_open;
 * each zero-filled before the first use, pad_bytes >= 4 * blocks * world, left zero-filled by every
 * completed barrier.  Waits are bounded: after spin_limit polls (0 = about a second) a lane sets
 * *timeout_flag (if given; pinned host memory, tccl_timeout_flag_create) and gives up. */
int tccl_blockwise_barrier(void *const *signal_pads, size_t pad_bytes, int world, int rank, int blocks,
                           unsigned spin_limit, uint32_t *timeout_flag, void *stream);

/* HIP-event helpers so a host language without HIP bindings can time launches on the very
 * stream they run on.  No counterpart in the reference (it times with torch.cuda.Event,
 * triton_reduce_scatter.py:216-226). */
int tccl_event_create(void **event_out);
int tccl_event_destroy(void *event);
int tccl_event_record(void *event, void *stream);
int tccl_event_synchronize(void *event);
int tccl_event_elapsed_ms(void *start, void *stop, float *ms_out);
int tccl_stream_synchronize(void *stream);

/* Device facts used for reporting: compute units, memory clock (kHz), bus width (bits),
 * L2 bytes.  Any pointer may be NULL. */
int tccl_device_info(int *compute_units, int *mem_clock_khz, int *mem_bus_bits, size_t *l2_bytes);

#ifdef __cplusplus
}
#endif
#endif /* TCCL_AMD_H */
