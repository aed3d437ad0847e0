"""The hand-over protocol of the one-launch chain backward (gridnet_hip_chain_backward_all),
replayed on the CPU: gridnet_amd/chain_protocol.py restates which workgroup writes and reads
what in which iteration of csrc/chain_bwd.hip's whole-chain kernel, and a scheduler interleaves
the workgroups in arbitrary orders.  Checked: every value read is the one meant (no stale value,
no buffer reused before its reader is done), nobody waits for ever, and with signalling switched
off every workgroup still ends and the status word is set."""

import pytest

from gridnet_amd import chain_protocol as cp


def sticky(stay):
    """A scheduler that keeps running the same workgroup with probability ``stay``: lets single
    workgroups run far ahead of (or fall far behind) the others."""
    state = {"last": None}

    def pick(rng, live):
        if state["last"] in live and rng.random() < stay:
            return state["last"]
        state["last"] = rng.choice(live)
        return state["last"]
    return pick


@pytest.mark.parametrize("W,B,steps", [(1, 6, 2), (2, 6, 3), (3, 7, 3), (5, 6, 4), (4, 9, 2), (8, 32, 3)])
@pytest.mark.parametrize("stay", [0.0, 0.9, 0.999])
def test_every_read_sees_its_value_and_all_end(W, B, steps, stay):
    for seed in range(6):
        mem, log = cp.run(W, B, steps, seed, pick=sticky(stay) if stay else None)
        assert mem.status == 0
        assert len(log) == W * steps * B
        counted = (steps - 1) * B
        assert all(mem.arrive.get(m) == W for m in range(counted))
        assert all(mem.ready.get(m) == 1 for m in range(counted))
        # the walk of every workgroup is in item order
        for b in range(W):
            assert [n for blk, n in log if blk == b] == list(range(steps * B))


def test_one_workgroup_held_back_holds_the_others_within_a_batch():
    """Nobody gets further ahead of the slowest workgroup than the dependency allows: an item
    needs its counterpart of the step after from everybody."""
    W, B, steps = 4, 8, 4
    slow = 2

    def pick(rng, live):  # workgroup `slow` gets one event in 50
        others = [b for b in live if b != slow]
        if slow in live and (not others or rng.random() < 0.02):
            return slow
        return rng.choice(others)

    mem, log = cp.run(W, B, steps, 1, pick=pick)
    assert mem.status == 0
    progress = {b: -1 for b in range(W)}
    for blk, n in log:
        progress[blk] = n
        # completing iteration n needed ready[n - B], hence everybody's count-in for item n - B,
        # which a workgroup makes in its iteration n - B + 3
        if n >= B:
            assert min(progress.values()) >= n - B + 3 - 1


@pytest.mark.parametrize("W,B,steps", [(1, 6, 2), (3, 6, 3), (6, 8, 3)])
def test_without_signalling_every_workgroup_gives_up_and_ends(W, B, steps):
    for seed in range(4):
        mem, log = cp.run(W, B, steps, seed, publish=False, spin_limit=5, pick=sticky(0.9))
        assert mem.status == 1
        assert len(log) == W * steps * B   # every iteration of every workgroup still ran


def test_a_batch_below_the_minimum_is_refused():
    with pytest.raises(AssertionError):
        cp.run(2, cp.MIN_BATCH - 1, 3, 0)
