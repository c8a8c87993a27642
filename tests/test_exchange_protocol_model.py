"""CPU model of the exchange between the workgroups ("slices") that share one GroupNorm unit
(csrc/groupnorm.hip: gn_exchange), run over randomised interleavings.

What the kernel does per slice, and what the model replays one memory operation at a time:

  1. read the unit's launch count `epoch` (once, at kernel start); tag = epoch + 1
  2. publish (tag, mean) and (tag, M2) of its own part as two separate 64-bit words
  3. lane l polls slice l's two words until both carry the tag, at most `spin_limit` times -
     without limit for the slice's OWN words, which arrive without anybody's help; a sibling
     that has not published by then is computed from the sibling's part of the INPUT (two
     passes, all of whose loads have returned before the next step), after which its words are
     read once more and win if they have arrived
  4. merge all slices (Chan), then fetch_add(done) (its old value is used in step 6)
  5. only now store the output over its own part (the call may be in place)
  6. the slice whose fetch_add returned split - 1 stores done = 0, epoch = tag

All of it is relaxed atomics: stores become visible to the other slices after arbitrary delays
and in any order across addresses.  One thing the protocol leans on is modelled as a fact of
the machine: a kernel's stores are all visible when the next launch on the stream starts.  That
a slice's output never becomes visible before its own two words is not assumed: the slice
issues its output stores only after it has read both words back.

Checked over many random schedules, several consecutive launches per unit and changing split
factors: a word of an earlier launch is never accepted, every slice ends up with the statistics
of exactly this launch's data whichever way it obtained them, an overwritten input is never
used, and the counters return to their rest state.  The reference has no counterpart (it runs
three ordered kernels, M/nn/GroupNorm.cpp:105-145).
"""
import random

import pytest

MAX_SPLIT = 64


class Unit:
    """Device memory of one unit as the other slices see it."""

    def __init__(self):
        self.slot_mean = [(0, None)] * MAX_SPLIT  # (tag, value)
        self.slot_m2 = [(0, None)] * MAX_SPLIT
        self.epoch = 0
        self.done = 0
        self.fallbacks = 0


class Launch:
    def __init__(self, unit, split, launch_id, rng, spin_limit):
        self.unit, self.split, self.rng, self.spin_limit = unit, split, rng, spin_limit
        # this launch's data: the true (mean, M2) of every slice, unlike any other launch's
        self.truth = [(launch_id * 1000 + s + 0.25, launch_id * 1000 + s + 0.75) for s in range(split)]
        self.overwritten = [False] * split      # slice s has stored output over its input
        self.pending = []                       # [(slice, address kind, index, value)] not yet visible
        self.accepted = [dict() for _ in range(split)]
        self.finished = [False] * split

    # -- relaxed stores: visible later, in any order across addresses, in order per address
    def store(self, s, kind, index, value):
        self.pending.append((s, kind, index, value))

    def commit_one(self, i):
        s, kind, index, value = self.pending.pop(i)
        u = self.unit
        if kind == "mean":
            u.slot_mean[index] = value
        elif kind == "m2":
            u.slot_m2[index] = value
        elif kind == "done":
            u.done = value
        elif kind == "epoch":
            u.epoch = value
        elif kind == "output":
            self.overwritten[index] = True

    def committable(self):
        """Indices of pending stores that may become visible now: the oldest one per address."""
        seen, ok = set(), []
        for i, (s, kind, index, value) in enumerate(self.pending):
            key = (kind, index)
            if key in seen:
                continue
            seen.add(key)
            ok.append(i)
        return ok

    def slice_program(self, s):
        """Generator: one yield per memory operation of slice s."""
        u = self.unit
        epoch = u.epoch                       # 1. (all stores of earlier launches are visible)
        yield
        tag = epoch + 1
        mean, m2 = self.truth[s]
        self.store(s, "mean", s, (tag, mean))  # 2.
        yield
        self.store(s, "m2", s, (tag, m2))
        yield
        got = {}
        waiting = list(range(self.split))
        polls = {l: 0 for l in waiting}
        while waiting:                        # 3. the lanes poll side by side
            l = self.rng.choice(waiting)
            wm, wq = u.slot_mean[l], u.slot_m2[l]
            yield
            if wm[0] == tag and wq[0] == tag:
                got[l] = (wm[1], wq[1], "published")
                waiting.remove(l)
                continue
            polls[l] += 1
            if l != s and polls[l] >= self.spin_limit:   # give up on sibling l: compute it from its input
                clean = not self.overwritten[l]
                yield                         # (the two passes over the sibling's input)
                clean = clean and not self.overwritten[l]
                wm, wq = u.slot_mean[l], u.slot_m2[l]   # read its words once more: they win
                yield
                if wm[0] == tag and wq[0] == tag:
                    got[l] = (wm[1], wq[1], "published late")
                else:
                    assert clean, "slice %d used input of slice %d that was already overwritten" % (s, l)
                    got[l] = (self.truth[l][0], self.truth[l][1], "recomputed")
                    u.fallbacks += 1
                waiting.remove(l)
        self.accepted[s] = got
        old = u.done                          # 4. fetch_add is atomic at memory: immediate
        u.done = old + 1
        yield
        self.store(s, "output", s, True)      # 5.
        yield
        if old == self.split - 1:             # 6.
            self.store(s, "done", 0, 0)
            yield
            self.store(s, "epoch", 0, tag)
            yield
        self.finished[s] = True

    def run(self, starve=None):
        """Random schedule.  `starve`: a slice that is not dispatched until all others are stuck
        waiting or finished (what another stream filling the GPU can do)."""
        programs = {s: self.slice_program(s) for s in range(self.split)}
        steps = 0
        while programs or self.pending:
            steps += 1
            assert steps < 200000, "schedule does not terminate"
            runnable = [s for s in programs if s != starve]
            if starve in programs and (not runnable or self.rng.random() < 0.002):
                runnable.append(starve)  # dispatched at last (or by chance)
            can_commit = self.committable()
            if can_commit and (not runnable or self.rng.random() < 0.4):
                self.commit_one(self.rng.choice(can_commit))
                continue
            s = self.rng.choice(runnable)
            try:
                next(programs[s])
            except StopIteration:
                del programs[s]
        # every slice holds this launch's statistics of every sibling
        for s in range(self.split):
            assert set(self.accepted[s]) == set(range(self.split))
            for l, (mean, m2, how) in self.accepted[s].items():
                assert (mean, m2) == self.truth[l], "slice %d took %r for slice %d (%s)" % (s, (mean, m2), l, how)
        assert all(self.finished) and all(self.overwritten)


@pytest.mark.parametrize("seed", range(40))
def test_random_interleavings_never_accept_a_stale_word(seed):
    rng = random.Random(seed)
    unit = Unit()
    launch_id = 0
    expected_epoch = 0
    for _ in range(12):  # consecutive launches on the same unit (same stream: ordered)
        split = rng.choice([1, 2, 2, 4, 4, 8, 16, 64])
        launch_id += 1
        if split == 1:
            continue  # a whole unit in one workgroup does not touch the exchange area at all
        spin_limit = rng.choice([1, 1, 2, 5, 50, 10 ** 9])
        starve = rng.randrange(split) if rng.random() < 0.5 and spin_limit < 10 ** 9 else None
        Launch(unit, split, launch_id, rng, spin_limit).run(starve)
        expected_epoch += 1
        # rest state: nothing left to reset before the next launch (a replayed graph relies on it)
        assert unit.done == 0
        assert unit.epoch == expected_epoch
    assert unit.epoch == expected_epoch


def test_patient_slices_never_fall_back_and_impatient_ones_do():
    rng = random.Random(7)
    unit = Unit()
    for launch_id in range(1, 6):
        Launch(unit, 4, launch_id, rng, 10 ** 9).run()
    assert unit.fallbacks == 0
    for launch_id in range(6, 30):
        Launch(unit, 8, launch_id, rng, 1).run(starve=launch_id % 8)
    assert unit.fallbacks > 0


def test_a_different_split_on_the_same_unit_sees_only_its_own_tags():
    # launch A with 8 slices leaves tag e+1 in slots 0..7; launch B with 2 slices must not take
    # slot 1's old word, and a later launch with 8 slices must not take B's or A's
    rng = random.Random(3)
    unit = Unit()
    Launch(unit, 8, 1, rng, 10 ** 9).run()
    assert [t for t, _ in unit.slot_mean[:8]] == [1] * 8
    Launch(unit, 2, 2, rng, 3).run()
    assert [t for t, _ in unit.slot_mean[:8]] == [2, 2, 1, 1, 1, 1, 1, 1]
    Launch(unit, 8, 3, rng, 2).run(starve=5)
    assert unit.epoch == 3 and unit.done == 0
