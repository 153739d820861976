"""The stage hand-over of the fused kernel (csrc/fused_kernel.hpp, the ring of three stage buffers)
checked as a protocol, on the CPU: every interleaving of the waves of a workgroup is explored, and in
none of them may a wave read a stage that is not completely written, overwrite a stage that another
wave still has to read, or wait for ever.

What a wave does, as in the kernel:

    write its part of stage 0, count in for stage 0
    for i = 0, 1, ...:
        wait until all waves have counted in for stage i        (slot i % 3, uses i // 3 + 1)
        if stage i + 1 exists: write its part of stage i + 1 (slot (i + 1) % 3), count in for it
        read stage i (the multiply)

A count is the number of waves that have written their part, added up over the uses of a slot, as in
LDS.  The model also runs two variants that must fail, to show that the check can tell: a ring of
two slots, and the write placed before the wait.

The kernels of the default arithmetic write two stages ahead, at the end of an iteration, so that a
wave may run a whole iteration ahead of the slowest one of its workgroup (`late=True` below):

    write its part of stage 0, count step 0
    wait for step 0, write its part of stage 1, count step 1
    for i = 0, 1, ...:
        read stage i (the multiply, the candidates)
        wait until all waves have counted step i + 1            (all have finished iteration i - 1)
        write its part of stage i + 2 (slot (i + 2) % 3; past the last stage a write nobody reads)
        count step i + 2                                         (counter (i + 2) % 3)
"""
import pytest

SLOTS = 3


def late_program(stages, write_before_wait=False):
    """steps k = 0, 1, ...: step k writes stage k; ("wait", k) / ("count", k) name steps here"""
    program = [("write", 0), ("count", 0), ("wait", 0), ("write", 1), ("count", 1)]
    for i in range(stages):
        steps = [("wait", i + 1), ("write", i + 2), ("count", i + 2)]
        if write_before_wait:
            steps = [steps[1], steps[0], steps[2]]
        program += [("read", i)] + steps
    return program


def wave_program(stages, write_before_wait=False, late=False):
    if late:
        return late_program(stages, write_before_wait)
    program = [("write", 0), ("count", 0)]
    for i in range(stages):
        steps = [("wait", i)]
        if i + 1 < stages:
            steps += [("write", i + 1), ("count", i + 1)]
        if write_before_wait:
            steps = steps[1:] + steps[:1]
        program += steps + [("read", i)]
    return program


def explore(waves, stages, slots=SLOTS, write_before_wait=False, late=False):
    """Breadth-first search over all interleavings.  A wave's program is a list of steps; the state
    is the tuple of program counters (everything else follows from them).  Returns the set of
    reachable states, or raises AssertionError with the offending state."""
    program = wave_program(stages, write_before_wait, late)
    length = len(program)
    # (the late protocol also writes the two stages past the last one, which nobody reads)
    counts = stages + 2 if late else stages

    def counted(pcs, stage):
        """waves that have counted in for `stage`"""
        at = program.index(("count", stage))
        return sum(1 for pc in pcs if pc > at)

    def done_reading(pcs, stage):
        at = program.index(("read", stage))
        return all(pc > at for pc in pcs)

    def written(pcs, stage):
        at = program.index(("write", stage))
        return all(pc > at for pc in pcs)

    start = (0,) * waves
    seen = {start}
    frontier = [start]
    while frontier:
        upcoming = []
        for pcs in frontier:
            moved = False
            for w, pc in enumerate(pcs):
                if pc == length:
                    continue
                kind, stage = program[pc]
                if kind == "wait":
                    # the counter of the slot holds the counts of all its uses so far
                    slot = stage % slots
                    total = sum(counted(pcs, s) for s in range(counts) if s % slots == slot)
                    if total < waves * (stage // slots + 1):
                        continue  # this wave cannot move now
                elif kind == "write":
                    # the slot still holds stage - slots: every wave must be done reading it
                    old = stage - slots
                    assert old < 0 or done_reading(pcs, old), ("overwrites a stage being read", pcs, w, stage)
                elif kind == "read":
                    assert written(pcs, stage), ("reads an incomplete stage", pcs, w, stage)
                    # and no wave has started to overwrite it
                    later = stage + slots
                    if later < counts:
                        at = program.index(("write", later))
                        assert all(p <= at for p in pcs), ("reads a stage being overwritten", pcs, w, stage)
                moved = True
                nxt = pcs[:w] + (pc + 1,) + pcs[w + 1:]
                if nxt not in seen:
                    seen.add(nxt)
                    upcoming.append(nxt)
            assert moved or all(pc == length for pc in pcs), ("no wave can move", pcs)
        frontier = upcoming
    return seen


@pytest.mark.parametrize("waves,stages", [(2, 9), (3, 7), (4, 5)])
def test_every_interleaving_is_safe_and_finishes(waves, stages):
    assert len(explore(waves, stages)) > stages


@pytest.mark.parametrize("stages", [1, 2, 3, 4])
def test_short_runs(stages):
    assert len(explore(4, stages)) > 0


def test_a_wave_may_run_a_stage_ahead():
    # some interleaving has one wave reading stage i + 1 while another has not yet read stage i:
    # that slack is what the ring is for (a barrier per stage would not have it); two stages ahead
    # is never reached
    stages = 6
    program = wave_program(stages)
    read_at = {s: program.index(("read", s)) for s in range(stages)}
    states = explore(2, stages)
    assert any(a == read_at[3] and b <= read_at[2] for a, b in states)
    assert not any(a >= read_at[4] and b <= read_at[2] for a, b in states)


def test_the_check_catches_a_ring_that_is_too_short():
    with pytest.raises(AssertionError, match="being read|being overwritten"):
        explore(3, 6, slots=2)


def test_the_check_catches_a_write_before_the_wait():
    with pytest.raises(AssertionError, match="being read|being overwritten"):
        explore(3, 6, write_before_wait=True)


# ---- the protocol of the default arithmetic: two stages ahead, written at the end of an iteration

@pytest.mark.parametrize("waves,stages", [(2, 9), (3, 6), (4, 4)])
def test_late_writes_every_interleaving_is_safe_and_finishes(waves, stages):
    assert len(explore(waves, stages, late=True)) > stages


@pytest.mark.parametrize("stages", [1, 2, 3])
def test_late_writes_short_runs(stages):
    assert len(explore(4, stages, late=True)) > 0


def test_late_writes_let_a_wave_run_an_iteration_ahead():
    # one wave may have read stage i + 1 completely and be at the end of that iteration while another
    # has only just started to read stage i; it never starts to read stage i + 2 before the other is
    # done with stage i
    stages = 6
    program = wave_program(stages, late=True)
    read_at = {s: program.index(("read", s)) for s in range(stages)}
    states = explore(2, stages, late=True)
    assert any(a > read_at[3] and b <= read_at[2] for a, b in states)
    assert not any(a > read_at[4] and b <= read_at[2] for a, b in states)


def test_late_writes_the_check_catches_a_ring_that_is_too_short():
    with pytest.raises(AssertionError, match="being read|being overwritten"):
        explore(3, 6, slots=2, late=True)


def test_late_writes_the_check_catches_a_write_before_the_wait():
    with pytest.raises(AssertionError, match="being read|being overwritten"):
        explore(3, 6, write_before_wait=True, late=True)
