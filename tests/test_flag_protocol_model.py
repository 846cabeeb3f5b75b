"""A model of the flag protocol of the kernels that carry their barriers themselves (one launch per
rank, the reference's blockwise_barrier, triton_barrier.py:39-142, at the start of the kernel and
again at its end), run on the CPU under random and adversarial schedules.

What the model holds: W ranks, each a stream of calls; call k of a rank has G_k workgroups (the same
G_k in every rank), and workgroup g of a one-shot call passes two barriers with workgroup g of every
other rank -- leading on row g, trailing on row R + g -- a two-shot call three (row R + g, row g,
row 2 R + g).  A barrier is: store 1 into slot [row][own rank] of every peer's pad, then take
(1 -> 0) slot [row][peer] of the own pad for every peer.  A rank's call k + 1 starts when all its
workgroups of call k have ended.  Nothing else orders the ranks.

What must hold under every schedule: no flag is ever stored over a flag that has not been taken,
every workgroup ends (a lost flag shows as a workgroup that waits for ever), and the pads are all
zero afterwards.  With R fixed by the pad this holds for every sequence of workgroup counts; with
R = the call's own workgroup count -- a layout that looks equivalent -- it does not, and the model
must say so (a model that cannot tell the two apart pins nothing).

The pipelined double tree (triton_double_tree_allreduce.py:254-335 as designed: wait for the children's
chunk, reduce, signal the parent; wait for the parent's result, copy, signal the children) is modelled
the same way, chunk flags and barriers together: with its own leading and trailing barrier, or between
two barrier launches, every sequence of chunk counts, workgroup counts and lags ends with clean pads;
without a barrier after it a slow leaf loses a flag, and the model says so."""
import random

import pytest

ONE_SHOT, TWO_SHOT = "one_shot", "two_shot"
# the two-shot kernel without its own leading and trailing barrier (only the one between the shots, row g),
# and the barrier as a launch of its own on pads of its own, whose sender waits for its slot to be clear
TWO_SHOT_BARE, BARRIER_LAUNCH = "two_shot_bare", "barrier_launch"


def rows_of(kind, g, R):
    if kind == ONE_SHOT:
        return (g, R + g)
    if kind == TWO_SHOT:
        return (R + g, g, 2 * R + g)
    if kind == TWO_SHOT_BARE:
        return (g,)
    return (5000 + g,)


def barrier_steps(rank, world, row, sender_waits=False):
    """One blockwise barrier of a workgroup on `row`: raise the own slot in every peer's pad, take every
    peer's slot in the own pad."""
    steps = [("raise_when_clear" if sender_waits else "raise", peer, row, rank) for peer in range(world) if peer != rank]
    return steps + [("take", rank, row, peer) for peer in range(world) if peer != rank]


class Workgroup:
    """Workgroup g of one rank's launch: a list of micro-steps, each one memory operation
    (op, owner of the pad, slot key, sender)."""

    def __init__(self, steps):
        self.steps = steps
        self.at = 0

    @property
    def done(self):
        return self.at == len(self.steps)


def workgroups_of(kind, rank, world, G, R, rows):
    """The workgroups of one rank's launch of a call (kind, G)."""
    if isinstance(kind, tuple):                          # ("tree", chunks of tree a, chunks of tree b, lag, own barriers)
        return tree_workgroups(kind, rank, world, G)
    return [Workgroup([st for row in rows(kind, g, R) for st in barrier_steps(rank, world, row, kind == BARRIER_LAUNCH)])
            for g in range(G)]


def run(world, calls, fixed_rows, seed, stall=0.0, rows=rows_of):
    """calls: [(kind, G)], the same for every rank.  fixed_rows: R for every call, or None for R = G.
    stall: probability per scheduling decision that the slowest rank is passed over (an adversary that
    keeps one rank behind).  Returns (overwrites, stuck, pads_clean)."""
    rng = random.Random(seed)
    pads = [dict() for _ in range(world)]              # pads[owner][(row, sender)] = 0 / 1
    at_call = [0] * world
    live = [[] for _ in range(world)]

    def launch(rank):
        kind, G = calls[at_call[rank]]
        R = fixed_rows if fixed_rows is not None else G
        live[rank] = workgroups_of(kind, rank, world, G, R, rows)

    for r in range(world):
        launch(r)
    overwrites = 0
    slow = rng.randrange(world)
    while True:
        runnable = []
        for r in range(world):
            if at_call[r] == len(calls):
                continue
            for wg in live[r]:
                if wg.done:
                    continue
                op, owner, row, sender = wg.steps[wg.at]
                slot = pads[owner].get((row, sender), 0)
                if op == "raise" or slot == (1 if op == "take" else 0):
                    runnable.append((r, wg))
        if not runnable:
            break
        if stall and rng.random() < stall:
            others = [x for x in runnable if x[0] != slow]
            if others:
                runnable = others
        r, wg = rng.choice(runnable)
        op, owner, row, sender = wg.steps[wg.at]
        if op != "take":
            overwrites += pads[owner].get((row, sender), 0)
            pads[owner][(row, sender)] = 1
        else:
            pads[owner][(row, sender)] = 0
        wg.at += 1
        if all(w.done for w in live[r]):                  # the rank's kernel has ended: its next call starts
            at_call[r] += 1
            if at_call[r] < len(calls):
                launch(r)
    stuck = any(c < len(calls) for c in at_call)
    clean = all(v == 0 for pad in pads for v in pad.values())
    return overwrites, stuck, clean


def sequences(rng, kinds, length):
    return [(rng.choice(kinds), rng.choice((1, 2, 3, 5))) for _ in range(length)]


@pytest.mark.parametrize("kinds", [(ONE_SHOT,), (TWO_SHOT,)])
def test_rows_fixed_by_the_pad_are_safe_for_every_sequence_of_sizes(kinds):
    rng = random.Random(1)
    for trial in range(150):
        world = rng.choice((2, 3, 4))
        calls = sequences(rng, kinds, 6)
        for stall in (0.0, 0.9):
            overwrites, stuck, clean = run(world, calls, fixed_rows=5, seed=trial, stall=stall)
            assert (overwrites, stuck, clean) == (0, False, True), (world, calls, stall)


@pytest.mark.parametrize("kinds", [(ONE_SHOT,), (TWO_SHOT,)])
def test_the_model_catches_rows_that_move_with_the_workgroup_count(kinds):
    """R = G: a call with more workgroups than the one before it raises leading flags on rows where a
    slow peer still holds the last call's trailing flags."""
    rng = random.Random(2)
    failures = 0
    for trial in range(150):
        calls = sequences(rng, kinds, 6)
        overwrites, stuck, clean = run(3, calls, fixed_rows=None, seed=trial, stall=0.9)
        failures += bool(overwrites or stuck or not clean)
    assert failures > 10
    # ... and it is the growth that does it: with the same count in every call the moving layout is the fixed one
    for trial in range(50):
        calls = [(rng.choice(kinds), 3) for _ in range(6)]
        assert run(3, calls, fixed_rows=None, seed=trial, stall=0.9) == (0, False, True)


def rows_with_a_pad_per_family(kind, g, R):
    """The one-shot family's rows beyond every row of the two-shot family: another pad."""
    return tuple(1000 + row for row in rows_of(kind, g, R)) if kind == ONE_SHOT else rows_of(kind, g, R)


def test_families_need_pads_of_their_own():
    """One-shot and two-shot calls on the SAME pads, both with rows fixed by the pad: the two-shot call's
    leading barrier sits on the rows of the one-shot call's trailing barrier, and a flag is lost.  With a
    pad per family nothing is."""
    rng = random.Random(3)
    shared = separate = 0
    for trial in range(150):
        calls = sequences(rng, (ONE_SHOT, TWO_SHOT), 6)
        o, s, c = run(3, calls, fixed_rows=5, seed=trial, stall=0.9)
        shared += bool(o or s or not c)
        o, s, c = run(3, calls, fixed_rows=5, seed=trial, stall=0.9, rows=rows_with_a_pad_per_family)
        separate += bool(o or s or not c)
    assert shared > 10 and separate == 0


def test_barrier_launches_around_the_bare_kernel_mix_with_the_kernel_that_has_its_own():
    """The two-shot all-reduce as barrier launch + kernel + barrier launch and as one launch with the
    barriers inside, in any order on the same kernel pads (the barrier launches have pads of their own)."""
    rng = random.Random(4)
    for trial in range(150):
        calls = []
        for _ in range(5):
            G = rng.choice((1, 2, 3, 5))
            if rng.random() < 0.5:
                calls.append((TWO_SHOT, G))
            else:
                calls += [(BARRIER_LAUNCH, 4), (TWO_SHOT_BARE, G), (BARRIER_LAUNCH, 4)]
        for stall in (0.0, 0.9):
            assert run(3, calls, fixed_rows=5, seed=trial, stall=stall) == (0, False, True), calls
    # the barrier launch's own protocol, back to back: safe because its sender waits for a clear slot ...
    for trial in range(50):
        assert run(3, [(BARRIER_LAUNCH, 4)] * 8, fixed_rows=5, seed=trial, stall=0.9) == (0, False, True)
    # ... which a barrier on ONE row without that wait is not (the bare kernel's row, called back to back)
    bad = sum(run(3, [(TWO_SHOT_BARE, 3)] * 8, fixed_rows=5, seed=trial, stall=0.9) != (0, False, True) for trial in range(50))
    assert bad > 5


# ------------------------------------------------------------------ the pipelined double tree, one launch per rank
TREE_BARRIER_ROWS = 512                  # the barriers' second block of rows starts here, whatever G is


def tree_tables(world):
    """(parent, child0, child1) and height per tree and rank, as the kernel holds them; height 0 = leaf,
    the extra node on top (one child, tree.py:133-136) has the largest."""
    import tccl_amd
    nbr = [[None] * world for _ in range(2)]
    for r in range(world):
        six = tccl_amd.get_parents_and_children(world, r)
        nbr[0][r], nbr[1][r] = tuple(six[:3]), tuple(six[3:])
    height = [[0] * world for _ in range(2)]

    def h(t, r):
        kids = [c for c in nbr[t][r][1:] if c >= 0]
        return 0 if not kids else 1 + max(h(t, c) for c in kids)
    for t in range(2):
        for r in range(world):
            height[t][r] = h(t, r)
    return nbr, height


def tree_workgroups(kind, rank, world, G):
    """tree_pipelined_walk: workgroup g takes chunks g, g + G, ... of both trees; in round i the up-sweep
    step of its i-th chunk and the down-sweep step of its (i - lag)-th; with own barriers a blockwise
    barrier before and after (rows g and 512 + g of the barriers' block)."""
    _, nchunks_a, nchunks_b, lag, own_barriers = kind
    nchunks = (nchunks_a, nchunks_b)
    nbr, height = tree_tables(world)
    top = max(height[0])
    most = max(nchunks)
    out = []
    for g in range(min(G, most)):                       # workgroups beyond the last chunk leave at once
        steps = []
        if own_barriers:
            steps += barrier_steps(rank, world, ("bar", g))
        rounds = (most - g + G - 1) // G
        for i in range(rounds + lag):
            if i < rounds:
                c = g + i * G
                for t in range(2):
                    parent, c0, c1 = nbr[t][rank]
                    if c >= nchunks[t] or height[t][rank] == 0:
                        continue
                    steps += [("take", rank, ("chunk", t, c), kid) for kid in (c0, c1) if kid >= 0 and height[t][kid] > 0]
                    to = parent if height[t][rank] != top else c0
                    steps.append(("raise", to, ("chunk", t, c), rank))
            if i >= lag:
                c = g + (i - lag) * G
                for t in range(2):
                    parent, c0, c1 = nbr[t][rank]
                    if c >= nchunks[t] or height[t][rank] == top:
                        continue
                    steps.append(("take", rank, ("chunk", t, c), parent))
                    steps += [("raise", kid, ("chunk", t, c), rank) for kid in (c0, c1) if kid >= 0]
        if own_barriers:
            steps += barrier_steps(rank, world, ("bar", TREE_BARRIER_ROWS + g))
        out.append(Workgroup(steps))
    return out


@pytest.mark.parametrize("world", [2, 4, 8])
def test_double_tree_with_its_own_barriers_is_safe_for_every_sequence_of_sizes_and_grids(world):
    """Calls of different chunk counts, workgroup counts and lags back to back on the same pads: every
    workgroup ends (nothing waits in a circle), no flag is stored over one not yet taken, pads end clean."""
    rng = random.Random(5)
    for trial in range(40):
        calls = [(("tree", rng.choice((1, 2, 5, 9)), rng.choice((1, 3, 5, 8)), rng.choice((0, 1, 3)), True), rng.choice((1, 2, 3, 6)))
                 for _ in range(4)]
        for stall in (0.0, 0.9):
            assert run(world, calls, fixed_rows=5, seed=trial, stall=stall) == (0, False, True), calls


def test_double_tree_without_a_barrier_after_it_loses_a_leaf_s_flag():
    """What the trailing barrier is for: a parent does not wait for a leaf child before it sends the next
    call's result down, so without a barrier between two calls a slow leaf still holds the last call's flag
    in that slot.  A barrier launch either side of the bare kernel is the other safe form."""
    rng = random.Random(6)
    bare = ("tree", 3, 3, 1, False)
    bad = sum(run(4, [(bare, 2)] * 4, fixed_rows=5, seed=trial, stall=0.9) != (0, False, True) for trial in range(60))
    assert bad > 5
    for trial in range(40):
        calls = []
        for _ in range(3):
            calls += [(BARRIER_LAUNCH, 4), (("tree", rng.choice((1, 3, 6)), 3, 1, False), rng.choice((1, 2, 4))), (BARRIER_LAUNCH, 4)]
        assert run(4, calls, fixed_rows=5, seed=trial, stall=0.9) == (0, False, True), calls


# ------------------------------------------------------------------ one launch for all ranks: which workgroup takes which place
def run_one_launch(world, G, resident, lists, draw, seed):
    """All W ranks' workgroups in ONE launch of world * G workgroups of which at most `resident` run at a
    time, started in hardware order as slots come free (a workgroup holds its slot until it ends).  Place
    (rank, g) meets the places with the same g in a blockwise barrier (the two-shot kernel between its
    shots).  By hardware index workgroup b is place (b // G, b % G); drawn (take_place), a workgroup that
    starts on XCD x takes the next place of list x -- the places with g % lists == x in the order (g, rank) --
    or of the following lists when that one is used up.  Returns True when every workgroup has ended."""
    rng = random.Random(seed)
    total = world * G
    order = [[(g, r) for g in range(G) if g % lists == x for r in range(world)] for x in range(lists)]
    drawn = [0] * lists
    pads = [dict() for _ in range(world)]
    running, started, ended = [], 0, 0
    while ended < total:
        while started < total and len(running) < resident:
            if draw:
                x = rng.randrange(lists)                              # whichever XCD the hardware picked
                while drawn[x] == len(order[x]):
                    x = (x + 1) % lists
                g, rank = order[x][drawn[x]]
                drawn[x] += 1
            else:
                rank, g = started // G, started % G
            running.append(Workgroup(barrier_steps(rank, world, g)))
            started += 1
        runnable = []
        for wg in running:
            op, owner, row, sender = wg.steps[wg.at]
            if op == "raise" or pads[owner].get((row, sender), 0) == 1:
                runnable.append(wg)
        if not runnable:
            return False                                              # everything resident waits for a place not yet started
        wg = rng.choice(runnable)
        op, owner, row, sender = wg.steps[wg.at]
        pads[owner][(row, sender)] = 1 if op == "raise" else 0
        wg.at += 1
        if wg.done:
            running.remove(wg)
            ended += 1
    return True


def test_drawn_places_make_progress_whatever_is_resident():
    """With places drawn in the order in which workgroups really start, at most lists * (W - 1) workgroups can
    be waiting for a member of their group that has not started, so any residency above that drains any grid;
    with places bound to the hardware index the whole grid must be resident."""
    rng = random.Random(7)
    for trial in range(200):
        world, lists = rng.choice((2, 3, 4)), rng.choice((1, 2, 4))
        G = rng.choice((1, 3, 8, 17))
        resident = lists * (world - 1) + 1 + rng.choice((0, 1, 5))
        assert run_one_launch(world, G, resident, lists, True, trial), (world, G, resident, lists)
    # by index: fine when everything is resident, stuck as soon as a rank's workgroups fill the slots
    assert all(run_one_launch(3, 8, 24, 2, False, trial) for trial in range(20))
    assert not any(run_one_launch(3, 8, 8, 2, False, trial) for trial in range(20))
    # ... and the bound is tight: one slot fewer than lists * (W - 1) + 1 can be filled with waiting workgroups
    assert not all(run_one_launch(3, 8, 4, 2, True, trial) for trial in range(200))
