"""The packing of a step's entries into the arrays that kernels read (`engine/batch.py`, laid out by the native
runtime core): against the layout written out here, for steps drawn at random, and what is refused."""
import random

import pytest

from arle_amd.engine.batch import StepEntry, build_step_batch


def _layout(entries, slot_of, length_of):
    tokens = [t for e in entries for t in e.tokens]
    positions = [length_of[e.request] + k for e in entries for k in range(len(e.tokens))]
    slots = [slot_of[e.request] for e in entries for _ in e.tokens]
    row0 = [0]
    for e in entries:
        row0.append(row0[-1] + len(e.tokens))
    wanted = [row0[i] + w for i, e in enumerate(entries) for w in e.want]
    return tokens, positions, slots, row0, wanted


@pytest.mark.parametrize("seed", range(40))
def test_random_steps_are_laid_out_as_written_out(seed):
    rng = random.Random(seed)
    vocab = rng.choice([5, 100, 151936])
    n = rng.randint(1, 9)
    entries = []
    for i in range(n):
        m = rng.choice([1, 1, 1, 2, 5, 40])
        want = [rng.randrange(m) for _ in range(rng.randint(0, 4))]      # any order, repeats allowed
        entries.append(StepEntry(f"r{i}", [rng.randrange(vocab) for _ in range(m)], want))
    slot_of = dict(zip((e.request for e in entries), rng.sample(range(64), n)))
    length_of = {e.request: rng.randint(0, 5000) for e in entries}
    b = build_step_batch(entries, slot_of.__getitem__, length_of.__getitem__, vocab, "cpu")
    tokens, positions, slots, row0, wanted = _layout(entries, slot_of, length_of)
    assert b.token_ids.tolist() == tokens and b.positions.tolist() == positions and b.slot_of_token.tolist() == slots
    assert b.seg_row0.tolist() == row0 and b.want_rows.tolist() == wanted
    assert b.seg_slot.tolist() == [slot_of[e.request] for e in entries]
    assert b.seg_start.tolist() == [length_of[e.request] for e in entries]
    assert (b.num_tokens, b.max_position) == (len(tokens), max(positions))
    assert (b.max_qlen, b.min_qlen) == (max(len(e.tokens) for e in entries), min(len(e.tokens) for e in entries))
    assert b.single_segments == sum(len(e.tokens) == 1 for e in entries)
    assert b.max_portion_kv == max((length_of[e.request] + len(e.tokens) for e in entries if len(e.tokens) > 1), default=0)


@pytest.mark.parametrize("entries,what", [
    ([], "at least one entry"),
    ([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])], "twice"),
    ([StepEntry("a", [], [])], "no tokens"),
    ([StepEntry("a", [1, 100], [0])], "outside the vocabulary"),
    ([StepEntry("a", [-1], [0])], "outside the vocabulary"),
    ([StepEntry("a", [2 ** 40], [0])], "outside the vocabulary"),
    ([StepEntry("a", [1, 2], [2])], "wanted place"),
    ([StepEntry("a", [1, 2], [-1])], "wanted place"),
    ([StepEntry("a", [1.5, 2], [0])], "integers"),         # not cut to 1 without a word
    ([StepEntry("a", ["7"], [0])], "integers"),
    ([StepEntry("a", [None], [0])], "integers"),
    ([StepEntry("a", [2 ** 70], [0])], "integers"),
])
def test_what_a_step_may_not_hold_is_refused(entries, what):
    with pytest.raises(ValueError, match=what):
        build_step_batch(entries, lambda r: 0, lambda r: 0, 100, "cpu")
