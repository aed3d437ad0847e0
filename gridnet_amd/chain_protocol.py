"""Executable model of the hand-over protocol inside the one-launch chain backward
(``chain_bwd<ACT, true, ALL = true>`` in ``csrc/chain_bwd.hip``; the loop it takes backward is
gridnet/scripts/train_imagenet.py:76-86).

The kernel's workgroups stay resident for all outer steps and pass data to each other through
memory while they run.  This module restates WHO writes and reads WHAT in WHICH iteration --
the index arithmetic of the kernel, nothing of its numerics -- as small state machines that a
scheduler can interleave in any order, so that the protocol can be checked on the CPU:
no reader ever sees a value other than the one it is meant to see (nothing stale, nothing
overwritten early), nobody waits for ever, and when signalling is switched off every workgroup
still runs to its end and the status word says so.

Vocabulary (as in the kernel).  ``items = steps * B``; item ``n`` is element ``n % B`` of step
``steps - 1 - n // B`` (the walk is last step first).  The items of every step but the first hand
something on (``counted = (steps - 1) * B`` of them): item ``m`` produces what item ``m + B``
consumes.  In iteration ``n`` a workgroup

* looks after the item it is in charge of (``duty``: ``blk``, ``blk + W``, ...): if the counter it
  read an iteration ago says that all ``W`` workgroups have counted themselves in, it sums their
  shares, stores the LayerNorm sums for item ``duty + B`` and sets ``ready[duty]``;
* waits (bounded) for ``ready[n - B]`` if ``n >= B`` -- the word was requested an iteration ago;
  while it polls it keeps looking after its duty;
* reads what its neighbours left for item ``n`` (the halo buffer of the other parity) and the
  LayerNorm sums of item ``n``;
* requests ``ready[n + 1 - B]`` and its duty's counter for the next iteration;
* behind the barrier counts itself in for item ``n - 3``;
* stores the halo values of item ``n - 1`` (into its neighbours' records, buffer of that item's
  step parity) and its LayerNorm share of item ``n - 2``.

A store is visible to the counting-in that follows it by two iterations (halo) or one (share):
every wave waits for its stores to be acknowledged at the top of an iteration, and the barrier
gathers the waves before thread 0 adds to the counter.
"""

import random
from dataclasses import dataclass, field

MIN_BATCH = 6  # as kChainAllMinBatch in csrc/chain_bwd.hip


@dataclass
class Memory:
    W: int
    B: int
    steps: int
    publish: bool = True
    status: int = 0
    arrive: dict = field(default_factory=dict)   # item -> count
    ready: dict = field(default_factory=dict)    # item -> 1
    sums: dict = field(default_factory=dict)     # item -> item whose shares they were made of
    share: dict = field(default_factory=dict)    # (element, block) -> item
    halo: dict = field(default_factory=dict)     # (parity, element, receiver, sender) -> item


def step_of(n, B, steps):
    return steps - 1 - n // B


def neighbours(blk, W):
    """A ring stands in for the 26 blocks around a block."""
    return sorted({(blk - 1) % W, (blk + 1) % W} - {blk})


def workgroup(mem: Memory, blk: int, spin_limit: int, log: list):
    """Generator: yields at every point where another workgroup's memory operations may come in
    between.  Raises AssertionError when it reads something it must not see."""
    W, B, steps = mem.W, mem.B, mem.steps
    items, counted = steps * B, (steps - 1) * B
    duty, duty_count, ready_word = blk, 0, 1
    gave_up = False

    def finalize(m):
        for b in range(W):
            got = mem.share.get((m % B, b))
            # (once somebody has given up, workgroups run on without waiting and results are void)
            assert got == m or mem.status, f"workgroup {blk} finalizing item {m}: share of block {b} is of item {got}"
        mem.sums[m + B] = m
        if mem.publish:
            mem.ready[m] = 1

    def do_duty(count):
        nonlocal duty
        if duty < counted and count == W:
            finalize(duty)
            duty += W

    for n in range(items):
        yield  # top of the iteration: this workgroup's earlier stores have been acknowledged
        do_duty(duty_count)
        if n >= B:
            v, spins = ready_word, 0
            while v == 0 and not gave_up:
                yield  # one poll
                if duty < counted:
                    do_duty(mem.arrive.get(duty, 0))
                v = mem.ready.get(n - B, 0)
                spins += 1
                if v == 0 and (spins > spin_limit or mem.status):
                    gave_up = True
                    mem.status = 1
        if n >= B and not gave_up:
            j, s = step_of(n, B, steps), n % B
            for nb in neighbours(blk, W):
                got = mem.halo.get(((j + 1) & 1, s, blk, nb))
                assert got == n - B or mem.status, f"workgroup {blk} item {n}: halo values from {nb} are of item {got}"
            assert mem.sums.get(n) == n - B or mem.status, f"workgroup {blk} item {n}: sums are {mem.sums.get(n)}"
        # requests for the next iteration
        ready_word = mem.ready.get(n + 1 - B, 0) if B <= n + 1 < items else 1
        duty_count = mem.arrive.get(duty, 0) if duty < counted and duty + 3 <= n else 0
        yield  # the barrier
        if 3 <= n and n - 3 < counted:
            mem.arrive[n - 3] = mem.arrive.get(n - 3, 0) + 1
        if n >= 1:  # halo values of the item finished an iteration ago
            jd, sd = step_of(n - 1, B, steps), (n - 1) % B
            for nb in neighbours(blk, W):
                mem.halo[(jd & 1, sd, nb, blk)] = n - 1
        if n >= 2 and n - 2 < counted:
            mem.share[((n - 2) % B, blk)] = n - 2
        log.append((blk, n))
    return gave_up


def run(W: int, B: int, steps: int, seed: int, publish: bool = True, spin_limit: int = 10 ** 9,
        max_events: int = 10 ** 7, pick=None):
    """Interleave W workgroups at random (or by ``pick(rng, live)``) until all have ended.
    Returns (memory, order of completed iterations)."""
    assert B >= MIN_BATCH and steps >= 2
    rng = random.Random(seed)
    mem = Memory(W, B, steps, publish)
    log = []
    live = {b: workgroup(mem, b, spin_limit, log) for b in range(W)}
    events = 0
    while live:
        b = pick(rng, sorted(live)) if pick else rng.choice(sorted(live))
        try:
            next(live[b])
        except StopIteration:
            del live[b]
        events += 1
        assert events < max_events, "the workgroups do not finish: somebody waits for ever"
    return mem, log
