"""A CPU model of the scan-over-workgroups protocol of the preprocess launch (the control word, the
two generations of count / offset words, the scanner, bounded waits, the sticky "aborted" bit and
the host-side reset), run under random schedules with limited residency.

The model follows flashgs_amd/csrc/preprocess.hip step by step - every read or write of a shared
word is one scheduling point - so that the properties the kernel relies on can be checked on
interleavings no GPU run can be steered into:

* without a give-up every workgroup gets the number of keys in front of it, the pair counter ends at
  start + total, the control word is flipped exactly once and the generation the next launch will
  use is all zeros;
* a scanner that gives up while workgroups are still to be dispatched leaves the generation alone and
  the words marked: the late workgroups of that launch and every workgroup of later launches touch
  nothing and the pair counter stays negative, until the words are cleared;
* after the clear the next launches are correct again, whatever ran before.
"""
import random

import pytest

INT_MIN = -(1 << 31)
COUNT, OFFSET, POISON = 1, 2, 3
GENERATION, ABORTED = 1, 2


class Words:
    """The scan words of one stream: control word, two generations of (counts, offsets)."""

    def __init__(self, capacity):
        self.capacity = capacity
        self.clear()

    def clear(self):                      # fgs_reset_scan
        self.control = 0
        self.counts = [[0] * self.capacity for _ in range(2)]
        self.offsets = [[0] * self.capacity for _ in range(2)]


def workgroup(words, out, ticket, num_blocks, key_count, spin_limit, grid_threads):
    """One workgroup of the launch as a generator: yields at every access to a shared word."""
    control = words.control
    yield
    if control & ABORTED:
        out["curr"] = min(out["curr"], INT_MIN)
        out["touched"].discard(ticket)
        return
    which = control & GENERATION
    other = which ^ 1
    # strided share of the clear of the other generation
    for w in range(ticket + 1, 2 * words.capacity, grid_threads):
        (words.counts[other] if w < words.capacity else words.offsets[other])[w % words.capacity] = 0
        yield
    if ticket < 0:                                   # the scanner (workgroup 0 of the grid)
        start = out["curr"]
        yield
        running, base, spins, gave_up = start, 0, 0, False
        while base < num_blocks:
            word = words.counts[which][base]
            yield
            if word:
                words.offsets[which][base] = (OFFSET, running)
                running += word[1]
                base += 1
                spins = 0
                yield
            else:
                spins += 1
                if spins > spin_limit:
                    gave_up = True
                    break
        if gave_up:
            for j in range(base, num_blocks):
                words.offsets[which][j] = (POISON, 0)
                yield
            out["curr"] = min(out["curr"], INT_MIN)
            words.control = which | ABORTED
        else:
            if out["curr"] == start:                 # compare-and-swap against the starting value
                out["curr"] = running
            words.control = other
        return
    words.counts[which][ticket] = (COUNT, key_count)
    yield
    spins = 0
    while True:
        word = words.offsets[which][ticket]
        yield
        if word and word[0] == OFFSET:
            out["slots"][ticket] = word[1]
            return
        spins += 1
        if (word and word[0] == POISON) or spins > spin_limit:
            out["curr"] = min(out["curr"], INT_MIN)
            out["slots"][ticket] = None
            return


def launch(words, key_counts, residency, spin_limit, rng, start=0, slow_first=0):
    """Dispatches the scanner and the workgroups in index order, at most `residency` at a time, and
    advances a randomly chosen resident one per step.  `slow_first` steps are burnt before any
    workgroup but the scanner may move (a scanner that polls while nobody has published)."""
    num_blocks = len(key_counts)
    out = dict(curr=start, slots={}, touched=set(range(num_blocks)))
    todo = [workgroup(words, out, t, num_blocks, key_counts[t] if t >= 0 else 0, spin_limit, num_blocks + 1)
            for t in range(-1, num_blocks)]
    resident, nxt, burnt = [], 0, 0
    while resident or nxt < len(todo):
        while nxt < len(todo) and len(resident) < residency:
            resident.append(todo[nxt])
            nxt += 1
        pick = 0 if burnt < slow_first and resident[0] is todo[0] else rng.randrange(len(resident))
        burnt += 1
        try:
            next(resident[pick])
        except StopIteration:
            resident.pop(pick)
    return out


def check_good(words, out, key_counts, start, control_before):
    prefix = start
    for t, k in enumerate(key_counts):
        assert out["slots"][t] == prefix, (t, out["slots"][t], prefix)
        prefix += k
    assert out["curr"] == prefix
    assert words.control == (control_before & GENERATION) ^ 1
    nxt = words.control & GENERATION                 # what the next launch starts from: all zeros
    assert not any(words.counts[nxt][: len(key_counts)]) and not any(words.offsets[nxt][: len(key_counts)])


@pytest.mark.parametrize("seed", range(12))
def test_launches_without_a_give_up(seed):
    rng = random.Random(seed)
    words = Words(64)
    for _ in range(6):                               # launches of different sizes on the same words
        n = rng.randrange(1, 60)
        keys = [rng.randrange(0, 50) for _ in range(n)]
        start = rng.choice([0, 0, 1000])
        before = words.control
        out = launch(words, keys, residency=rng.choice([2, 3, 8, 100]), spin_limit=10 ** 9, rng=rng, start=start)
        check_good(words, out, keys, start, before)


@pytest.mark.parametrize("seed", range(12))
def test_a_scanner_that_gives_up_marks_the_words_until_they_are_cleared(seed):
    rng = random.Random(100 + seed)
    words = Words(64)
    keys = [rng.randrange(1, 50) for _ in range(40)]
    out = launch(words, keys, residency=100, spin_limit=10 ** 9, rng=rng)
    check_good(words, out, keys, 0, 0)
    before = words.control
    # a grid larger than the residency and a scanner that runs out of polls before anybody
    # has published: workgroups are dispatched after the give-up
    out = launch(words, keys, residency=4, spin_limit=3, rng=rng, slow_first=50)
    assert out["curr"] < 0
    assert words.control == (before & GENERATION) | ABORTED          # generation unchanged, marked
    assert len(out["touched"]) < len(keys)                           # late workgroups did nothing at all
    # later launches - other sizes, ample polls - are refused at once and write nothing
    snapshot = ([list(a) for a in words.counts], [list(a) for a in words.offsets])
    for n in (7, 55):
        other = [rng.randrange(0, 9) for _ in range(n)]
        out = launch(words, other, residency=rng.choice([3, 100]), spin_limit=10 ** 9, rng=rng)
        assert out["curr"] < 0 and not out["slots"] and not out["touched"]
        assert ([list(a) for a in words.counts], [list(a) for a in words.offsets]) == snapshot
    words.clear()
    for n in (55, 7, 40):                            # stale words of the aborted launch cannot match: all gone
        other = [rng.randrange(0, 9) for _ in range(n)]
        before = words.control
        out = launch(words, other, residency=rng.choice([3, 100]), spin_limit=10 ** 9, rng=rng)
        check_good(words, out, other, 0, before)


def test_a_workgroup_that_gives_up_alone_only_spoils_its_own_launch():
    """A workgroup whose own wait runs out (the scanner is fine) lowers the pair counter; the scanner
    still reads every count and flips the generation, so the next launch is clean."""
    rng = random.Random(5)
    words = Words(32)
    keys = [3] * 20
    before = words.control

    # residency 2 and one poll: a workgroup polls once right after publishing, before the scanner
    # (which gets its turn only half of the time) has written its offset
    out = launch(words, keys, residency=2, spin_limit=10 ** 9, rng=rng)
    check_good(words, out, keys, 0, before)
    before = words.control
    tries = 0
    while True:
        tries += 1
        w2 = Words(32)
        w2.control = before
        out = launch(w2, keys, residency=3, spin_limit=1, rng=random.Random(tries))
        if w2.control & ABORTED:
            continue                                 # this schedule made the scanner give up: not the case meant here
        if out["curr"] < 0:
            break
        assert tries < 200
    assert w2.control == (before & GENERATION) ^ 1
    out = launch(w2, keys, residency=3, spin_limit=10 ** 9, rng=rng)
    check_good(w2, out, keys, 0, w2.control ^ 1)
