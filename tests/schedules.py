"""Ways of cutting the same requests into steps; shared by the CPU-logic and the GPU tests.

Every function drives `Engine.step` and returns, per request, the float32 logits of every
position [len(tokens), vocab] as NumPy arrays, so that any two cuts and the plain
implementation can be compared position by position.
"""

from __future__ import annotations

import numpy as np

from beholdd.engine import StepEntry


def _rows(logits):
    return logits.float().cpu().numpy()


def whole(engine, requests):
    """Each request alone, all its tokens in one step."""
    out = []
    for tokens in requests:
        slot = engine.alloc_slot()
        out.append(_rows(engine.step([StepEntry(slot, list(tokens), list(range(len(tokens))))])))
        engine.free_slot(slot)
    return out


def tail_one_by_one(engine, requests, tail=32):
    """Each request alone: the first n - tail tokens in one step, the last `tail` one by one."""
    out = []
    for tokens in requests:
        tokens = list(tokens)
        cut = max(1, len(tokens) - tail)
        slot = engine.alloc_slot()
        rows = [_rows(engine.step([StepEntry(slot, tokens[:cut], list(range(cut)))]))]
        for token in tokens[cut:]:
            rows.append(_rows(engine.step([StepEntry(slot, [token], [0])])))
        engine.free_slot(slot)
        out.append(np.concatenate(rows, axis=0))
    return out


def batches(engine, requests, batch_size, prompt_fraction=0.6):
    """Batches of unequal lengths, one after another so that slots and pages are used again:
    each request's first part (a fraction of its length) goes in with the others' in one
    step, the rest one token per step; shorter requests end earlier and free their slots."""
    out = [None] * len(requests)
    for start in range(0, len(requests), batch_size):
        group = list(range(start, min(start + batch_size, len(requests))))
        slots = {i: engine.alloc_slot() for i in group}
        cuts = {i: max(1, int(len(requests[i]) * prompt_fraction)) for i in group}
        rows = {i: [] for i in group}
        logits = _rows(engine.step([StepEntry(slots[i], list(requests[i][:cuts[i]]), list(range(cuts[i])))
                                    for i in group]))
        at = 0
        for i in group:
            rows[i].append(logits[at:at + cuts[i]])
            at += cuts[i]
        done = {i: cuts[i] for i in group}
        live = [i for i in group if done[i] < len(requests[i])]
        for i in group:
            if i not in live:
                engine.free_slot(slots.pop(i))
        while live:
            logits = _rows(engine.step([StepEntry(slots[i], [requests[i][done[i]]], [0]) for i in live]))
            for row, i in enumerate(live):
                rows[i].append(logits[row:row + 1])
                done[i] += 1
            still = []
            for i in live:
                if done[i] < len(requests[i]):
                    still.append(i)
                else:
                    engine.free_slot(slots.pop(i))      # a shorter request ends earlier
            live = still
        for i in group:
            out[i] = np.concatenate(rows[i], axis=0)
    return out


def portions(engine, requests, sizes=(2, 62, 1, 64, 2, 63, 1, 1, 65, 3, 61), rest_every=4):
    """All requests together, every one fed in portions of unequal sizes: steps of several tokens onto a cache
    that already holds some (also ending exactly at a page's end, one before and one after), portions of one
    token beside portions of many in the same step, and now and then a request that rests for a step while its
    batch-mates advance.  A request ends when its tokens are used up; the others go on."""
    slots = [engine.alloc_slot() for _ in requests]
    done = [0] * len(requests)
    rows = [[] for _ in requests]
    live = list(range(len(requests)))
    step = 0
    while live:
        resting = [i for i in live if (step + i) % rest_every == rest_every - 1]
        moving = [i for i in live if i not in resting] or live
        counts = {i: min(sizes[(step + 3 * i) % len(sizes)], len(requests[i]) - done[i]) for i in moving}
        logits = _rows(engine.step([StepEntry(slots[i], list(requests[i][done[i]:done[i] + counts[i]]),
                                              list(range(counts[i]))) for i in moving]))
        at = 0
        for i in moving:
            rows[i].append(logits[at:at + counts[i]])
            at += counts[i]
            done[i] += counts[i]
            if done[i] == len(requests[i]):
                engine.free_slot(slots[i])
                live.remove(i)
        step += 1
    return [np.concatenate(r, axis=0) for r in rows]


class TraceRecorder:
    """Stands where an engine stands in the functions above and writes down what they do, as the steps of a
    trace for bin/trace_run: requests are named r0, r1, ... in the order in which they get their slots."""

    def __init__(self):
        self.steps, self.name_of, self.started = [], {}, 0

    def alloc_slot(self):
        slot = self.started
        self.name_of[slot] = f"r{self.started}"
        self.started += 1
        return slot

    def free_slot(self, slot):
        self.steps[-1]["end"].append(self.name_of.pop(slot))

    def step(self, entries):
        import torch
        self.steps.append({"step": len(self.steps), "end": [],
                           "entries": [{"id": self.name_of[e.slot], "tokens": [int(t) for t in e.tokens],
                                        "want": [int(w) for w in e.want]} for e in entries]})
        return torch.zeros(sum(len(e.want) for e in entries), 1)


def trace_of(schedule, requests, **options):
    """The steps that `schedule(engine, requests, **options)` would run, as trace records."""
    recorder = TraceRecorder()
    schedule(recorder, requests, **options)
    return recorder.steps


def relative_error(got, want):
    """max |got - want| / max |want|: the measure the acceptance tolerance is stated in."""
    return float(np.abs(got.astype(np.float64) - want.astype(np.float64)).max() / np.abs(want).max())


def random_requests(vocab, lengths, seed):
    rng = np.random.default_rng(seed)
    return [[int(t) for t in rng.integers(0, vocab, size=n)] for n in lengths]
