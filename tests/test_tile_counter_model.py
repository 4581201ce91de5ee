"""Model check of the grouped GEMM's tile counter protocol (moe_gemm.hip: tile_queue, queue_open, queue_draw and
the scheduler loop of grouped_gemm_kernel), on the CPU.

Every workgroup of a launch is a coroutine that yields before each access to the shared counter, so a scheduler
can interleave the workgroups of two launches that share a slot in any order.  Checked, over many random
interleavings:

  * a launch alone computes every tile, whatever the slot held before and however its workgroups interleave --
    exactly once when the stamp is there before the first draw (the usual case), at least once when a draw comes
    first (that workgroup takes the slot for lost and does its share in the fixed order);
  * a launch that starts after a later launch has stamped the slot never writes to the counter (so it cannot
    cost the later launch a ticket) and both compute all of their tiles;
  * a launch whose slot is taken over while it runs still computes all of its own tiles (some twice).

The model restates the device code's steps one for one; the constants are the kernel's."""
import random

import pytest

COUNT_BITS = 24
TAIL_SWEEPS = 2
NO_QUEUE = 1 << 30


class Counter:
    def __init__(self, value=0):
        self.value = value
        self.writes = {}   # launch name -> number of writes it made


def workgroup(name, b, nwg, total, stamp, ctr, done, queued=True):
    """One workgroup (index b of nwg) of a launch of `total` tiles; appends the tiles it computes to done."""
    sweep = nwg
    ok = False
    if queued:
        yield                                   # queue_open: the load ...
        now = ctr.value
        if b < 8:
            yield                               # ... and, for the first workgroups, the atomic max
            if ctr.value < stamp:
                ctr.value = stamp
            ctr.writes[name] = ctr.writes.get(name, 0) + 1
        ok = now < stamp + (1 << COUNT_BITS)
    fixed = max(1, total // sweep - TAIL_SWEEPS) if ok and total > sweep else NO_QUEUE
    sw = 0
    while True:
        tile = None
        if sw >= fixed:
            if fixed == NO_QUEUE:
                return
            yield                               # queue_draw: fetch-and-add on the low word
            raw = ctr.value & 0xffffffff
            ctr.value += 1
            ctr.writes[name] = ctr.writes.get(name, 0) + 1
            d = (raw - (stamp & 0xffffffff)) & 0xffffffff
            own = d if d < (1 << COUNT_BITS) else -1
            if own >= 0:
                tile = fixed * sweep + own
                if tile >= total:
                    return
            else:                               # slot lost: this workgroup's share of the tail in the fixed order
                sw = fixed
                fixed = NO_QUEUE
        if sw < fixed:
            last_partial = (sw + 1) * sweep > total
            tile = sw * sweep + b               # (the kernel permutes b within full sweeps; a bijection either way)
            _ = last_partial
            if tile >= total:
                return
        done.append(tile)
        sw += 1


def run(launches, rng, stamps_first=False):
    """launches: list of (name, nwg, total, stamp, start_when, counter) sharing one counter, start_when(done, counter)
    telling when the launch's workgroups appear (None: at once); stamps_first: a launch's first 8 workgroups get to
    the end of queue_open before anything else runs (what the kernel arranges: draws start one tile into the kernel);
    returns {name: tiles}, counter."""
    ctr = launches[0][5]
    done = {l[0]: [] for l in launches}
    live = []
    pending = list(launches)
    while pending or live:
        for l in list(pending):
            name, nwg, total, stamp, after, _ = l
            if after is None or after(done, ctr):
                pending.remove(l)
                gens = [(name, workgroup(name, b, nwg, total, stamp, ctr, done[name])) for b in range(nwg)]
                if stamps_first:   # up to the yield behind the atomic max (the third: start, load, max)
                    for _, g in gens[:8]:
                        for _ in range(3):
                            next(g, None)
                live += gens
        if not live:
            raise AssertionError("deadlock in the model's launch order")
        i = rng.randrange(len(live))
        name, g = live[i]
        if next(g, "end") == "end":
            live.pop(i)
    return done, ctr


def stamp_of(use):
    return (use + 1) << COUNT_BITS


@pytest.mark.parametrize("nwg,total", [(8, 5), (8, 8), (8, 9), (8, 24), (8, 61), (16, 100), (24, 200)])
def test_a_launch_alone_computes_every_tile(nwg, total):
    for seed in range(30):
        rng = random.Random(seed)
        leftover = rng.choice([0, stamp_of(0) + 17, stamp_of(3) + total + nwg])   # what an earlier use left behind
        done, _ = run([("a", nwg, total, stamp_of(5), None, Counter(leftover))], rng, stamps_first=True)
        assert sorted(done["a"]) == list(range(total)), (seed, leftover)
        done, _ = run([("a", nwg, total, stamp_of(5), None, Counter(leftover))], rng)
        assert set(done["a"]) == set(range(total)), (seed, leftover)


@pytest.mark.parametrize("nwg,total", [(8, 40), (16, 90)])
def test_a_launch_that_starts_late_never_touches_the_later_launchs_counter(nwg, total):
    for seed in range(30):
        rng = random.Random(seed)
        ctr = Counter(0)
        # b (later stamp) has stamped the slot and runs; then a (earlier stamp, same slot) starts beside it
        late = lambda done, c: c.value >= stamp_of(7) and len(done["b"]) >= total // 3
        done, ctr = run([("b", nwg, total, stamp_of(7), None, ctr), ("a", nwg, total, stamp_of(6), late, ctr)], rng, stamps_first=True)
        assert ctr.writes.get("a", 0) <= 8          # only the harmless atomic max of its first workgroups
        assert sorted(done["a"]) == list(range(total)), seed
        assert sorted(done["b"]) == list(range(total)), seed


@pytest.mark.parametrize("nwg,total", [(8, 40), (16, 90), (8, 200)])
def test_a_launch_whose_slot_is_taken_over_still_computes_all_of_its_tiles(nwg, total):
    for seed in range(40):
        rng = random.Random(seed)
        ctr = Counter(0)
        n = rng.randrange(1, total)
        done, _ = run([("a", nwg, total, stamp_of(6), None, ctr), ("b", nwg, total, stamp_of(7), lambda done, c: len(done["a"]) >= n, ctr)], rng)
        assert set(done["a"]) == set(range(total)), seed        # b's result is not defined in this arrangement


def test_a_launch_without_a_counter_walks_everything_in_the_fixed_order():
    rng = random.Random(0)
    ctr = Counter(123)
    done = {"a": []}
    gens = [workgroup("a", b, 8, 29, 0, ctr, done["a"], queued=False) for b in range(8)]
    for g in gens:
        for _ in g:
            pass
    assert sorted(done["a"]) == list(range(29)) and ctr.value == 123 and not ctr.writes
