"""The generation loop's decisions, with a stepper that needs no model: which tokens are
emitted, when a sequence ends, when its slot is freed, how requests are split into batches."""

import pytest
import torch

from beholdd.engine import (FINISH_LENGTH, FINISH_STOP, GenerationError, generate, plan_batches, positions_needed)
from beholdd.sampling import SamplingParams, uniform


class ScriptedStepper:
    """A sequence's next token is a function of its length and its first token; logits carry it."""

    page_size = 64

    def __init__(self, capacity_pages=64, max_slots=8, max_position=4096, vocab=50):
        self.capacity_pages, self.max_slots, self.max_position, self.vocab = capacity_pages, max_slots, max_position, vocab
        self.free = list(range(max_slots))
        self.state = {}           # slot -> (first token, length)
        self.steps = []           # (kind, [slots])
        self.peak_slots = 0
        self.log = []

    def alloc_slot(self):
        slot = self.free.pop(0)
        self.state[slot] = None
        self.peak_slots = max(self.peak_slots, len(self.state))
        self.log.append(("alloc", slot))
        return slot

    def free_slot(self, slot):
        assert slot in self.state, "freed twice"
        del self.state[slot]
        self.free.insert(0, slot)
        self.log.append(("free", slot))

    def next_token(self, first, length):
        return (first * 7 + length * 3) % self.vocab

    def step(self, entries):
        kinds = {len(e.tokens) == 1 and self.state[e.slot] is not None for e in entries}
        assert len(kinds) == 1, "a step either starts all its sequences or continues all of them"
        rows = []
        for e in entries:
            if self.state[e.slot] is None:
                self.state[e.slot] = (e.tokens[0], len(e.tokens))
            else:
                first, length = self.state[e.slot]
                assert e.tokens == [self.next_token(first, length)], "the token fed back is the one that was chosen"
                self.state[e.slot] = (first, length + 1)
            first, length = self.state[e.slot]
            assert e.want == [len(e.tokens) - 1]
            row = torch.zeros(self.vocab)
            row[self.next_token(first, length)] = 5.0
            rows.append(row)
        self.steps.append(("prefill" if kinds == {False} else "decode", [e.slot for e in entries]))
        return torch.stack(rows)

    def select(self, logits, params, requests, steps):
        assert len(params) == len(requests) == len(steps) == logits.shape[0]
        return [int(torch.argmax(row)) for row in logits]


def expected_tokens(stepper, prompt, n):
    return [stepper.next_token(prompt[0], len(prompt) + i) for i in range(n)]


def test_unequal_prompts_one_step_then_one_token_each():
    s = ScriptedStepper()
    prompts = [[1, 2, 3, 4, 5], [9] * 11, [4] * 17]
    results = generate(s, prompts, 8)
    for prompt, result in zip(prompts, results):
        assert result.token_ids == expected_tokens(s, prompt, 8)
        assert result.finish_reason == FINISH_LENGTH and result.stop_token is None
        assert result.prompt_tokens == len(prompt) and result.completion_tokens == 8
    assert s.steps[0] == ("prefill", [0, 1, 2]) and all(kind == "decode" for kind, _ in s.steps[1:])
    assert len(s.steps) == 8                   # prefill + 7 decode steps: the last token is never evaluated
    assert s.state == {}


def test_stop_token_is_not_emitted_and_others_go_on():
    s = ScriptedStepper()
    prompts = [[1, 2, 3], [2, 2], [5]]
    free_run = [expected_tokens(s, p, 6) for p in prompts]
    stop = free_run[1][2]
    seen = []
    results = generate(s, prompts, 6, stop_token_ids=[stop], on_token=lambda i, t: seen.append((i, t)))
    for i, (result, tokens) in enumerate(zip(results, free_run)):
        if stop in tokens:
            cut = tokens.index(stop)
            assert result.token_ids == tokens[:cut] and result.finish_reason == FINISH_STOP and result.stop_token == stop
        else:
            assert result.token_ids == tokens and result.finish_reason == FINISH_LENGTH
        assert [t for j, t in seen if j == i] == result.token_ids       # the callback sees exactly what is emitted
    assert results[1].finish_reason == FINISH_STOP
    later = [slots for kind, slots in s.steps if kind == "decode"][-1]
    assert 1 not in later                                                # the stopped sequence left the batch
    assert s.state == {}


def test_sequences_that_end_earlier_free_their_slots_at_once():
    s = ScriptedStepper()
    generate(s, [[1], [2], [3]], [2, 5, 3])
    order = [entry for entry in s.log if entry[0] == "free"]
    assert order == [("free", 0), ("free", 2), ("free", 1)]
    sizes = [len(slots) for _, slots in s.steps]
    assert sizes == [3, 3, 2, 1, 1]


def test_zero_new_tokens_touches_nothing():
    s = ScriptedStepper()
    results = generate(s, [[1, 2], [3]], [0, 2])
    assert results[0].token_ids == [] and results[0].finish_reason == FINISH_LENGTH
    assert results[1].completion_tokens == 2
    assert s.steps[0] == ("prefill", [0])                # only the second request ever ran
    assert generate(ScriptedStepper(), [[1]], 0)[0].token_ids == []


def test_context_boundary():
    # crates/beholdd-model/src/qwen3moe/forward.rs:3053-3065: a prompt of the whole context may select one token
    s = ScriptedStepper(max_position=10)
    assert positions_needed(10, 1) == 10 and positions_needed(10, 0) == 10 and positions_needed(3, 8) == 10
    assert generate(s, [[1] * 10], 1)[0].completion_tokens == 1
    assert generate(ScriptedStepper(max_position=10), [[1] * 3], 8)[0].completion_tokens == 8
    with pytest.raises(GenerationError, match="needs 11 evaluated positions"):
        generate(ScriptedStepper(max_position=10), [[1] * 3], 9)
    with pytest.raises(GenerationError, match="at least one prompt token"):
        generate(ScriptedStepper(), [[]], 1)
    with pytest.raises(GenerationError, match="negative"):
        generate(ScriptedStepper(), [[1]], -1)


def test_requests_run_as_one_batch_after_another():
    s = ScriptedStepper(max_slots=3)
    prompts = [[i + 1] * (i + 1) for i in range(8)]
    results = generate(s, prompts, 4)
    assert [r.token_ids for r in results] == [expected_tokens(s, p, 4) for p in prompts]
    prefills = [slots for kind, slots in s.steps if kind == "prefill"]
    assert [len(p) for p in prefills] == [3, 3, 2] and s.peak_slots == 3
    assert sorted(prefills[1]) == sorted(prefills[0])    # the second batch runs in the slots the first gave back
    assert [len(b) for b in plan_batches([5] * 8, [4] * 8, 64, 64, 8, 2)] == [2, 2, 2, 2]
    # the cache's pages bound a batch too: each request needs 2 pages of 64, the cache has 5
    assert [len(b) for b in plan_batches([100] * 5, [20] * 5, 64, 5, 8, None)] == [2, 2, 1]
    with pytest.raises(GenerationError, match="cache pages"):
        plan_batches([1000], [10], 64, 5, 8, None)


def test_callback_error_aborts_and_frees_everything():
    s = ScriptedStepper()

    def on_token(index, token):
        if index == 1:
            raise RuntimeError("consumer went away")

    with pytest.raises(RuntimeError, match="went away"):
        generate(s, [[1], [2], [3]], 4, on_token=on_token)
    assert s.state == {}
    calls = {"n": 0}

    def control():
        calls["n"] += 1
        if calls["n"] == 3:
            raise KeyboardInterrupt

    s = ScriptedStepper()
    with pytest.raises(KeyboardInterrupt):
        generate(s, [[1], [2]], 10, control=control)
    assert s.state == {} and len(s.steps) == 2           # the prefill and one decode step ran before the third poll


def test_per_request_limits_and_parameters():
    s = ScriptedStepper()
    results = generate(s, [[1], [2]], [1, 3], [SamplingParams(), SamplingParams(temperature=0.5, seed=3)])
    assert [r.completion_tokens for r in results] == [1, 3]
    with pytest.raises(GenerationError, match="one max_new_tokens"):
        generate(s, [[1], [2]], [1])


def test_uniform_numbers_are_a_pure_function_of_seed_request_step():
    values = {uniform(s, r, t) for s in range(3) for r in range(5) for t in range(20)}
    assert len(values) == 300 and all(0.0 <= v < 1.0 for v in values)
    assert uniform(1, 2, 3) == uniform(1, 2, 3)
    mean = sum(uniform(0, 0, t) for t in range(4000)) / 4000
    assert abs(mean - 0.5) < 0.03
    for bad in (dict(temperature=-1.0), dict(top_k=-1), dict(top_p=0.0), dict(top_p=1.5),
                dict(temperature=float("nan")), dict(temperature=float("inf")), dict(temperature="0.8"),
                dict(temperature=[0.8]), dict(top_k=1.5), dict(top_k=None), dict(top_k=1 << 40), dict(top_k=True),
                dict(top_p=None), dict(top_p=[0.5]), dict(top_p=float("nan")), dict(seed=None), dict(seed=0.5)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    import numpy as np
    assert SamplingParams(temperature=np.float32(0.5), top_k=np.int64(3), seed=np.int32(2)).top_k == 3


def test_arguments_of_the_wrong_type_are_refused_with_a_reason():
    s = ScriptedStepper()
    for prompts, wrong in ((7, "prompts are a list"), ([[1], 5], "request 1: a prompt is a list"),
                           ([[1], "ab"], "request 1: a prompt is a list")):
        with pytest.raises(GenerationError, match=wrong):
            generate(s, prompts, 1)
    for n_new in ("3", 1.5, None, True):
        with pytest.raises(GenerationError, match="max_new_tokens is an integer"):
            generate(s, [[1]], n_new)
    for stops in (3, None, [0.5], ["a"], 2.0):
        with pytest.raises(GenerationError, match="stop_token_ids are a list"):
            generate(s, [[1]], 1, stop_token_ids=stops)
    for size in ("2", 1.5, (1, 2)):
        with pytest.raises(GenerationError, match="batch_size is an integer"):
            generate(s, [[1]], 1, batch_size=size)
    assert s.state == {} and s.steps == []
    import numpy as np
    listed = generate(ScriptedStepper(), [[1, 2, 3], [4]], 3)
    arrays = generate(ScriptedStepper(), [np.array([1, 2, 3]), np.array([4], dtype=np.int32)], np.int64(3))
    assert [r.token_ids for r in arrays] == [r.token_ids for r in listed]      # arrays of token ids are as good as lists


# ---- the loop that runs one step ahead of the host ------------------------------------------------

class AheadStepper(ScriptedStepper):
    """The scripted stepper with selections that the next step can read "on the device": an entry with
    `fed_row` takes its token from that row of the last selection's buffer."""

    class Selection:
        def __init__(self, owner, buffer, device_rows, error=None):
            self.owner, self.buffer, self.device_rows, self.error = owner, buffer, list(device_rows), error

        def take(self, positions):
            return AheadStepper.Selection(self.owner, self.buffer, [self.device_rows[i] for i in positions], self.error)

        def result(self):
            self.owner.results_read += 1
            if self.error is not None:
                raise self.error
            return [self.buffer[row] for row in self.device_rows]

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.buffer, self.results_read, self.wasted = [], 0, 0

    def step(self, entries):
        resolved = []
        for e in entries:
            if e.fed_row is not None:
                assert e.tokens == [0] and e.want == [0]
                e = type(e)(e.slot, [self.buffer[e.fed_row]], e.want)
            resolved.append(e)
        return super().step(resolved)

    def select_async(self, logits, params, requests, steps):
        self.buffer = self.select(logits, params, requests, steps)       # a new selection overwrites the buffer
        return AheadStepper.Selection(self, self.buffer, range(len(self.buffer)))


def both_loops(**kwargs):
    return [ScriptedStepper(**kwargs), AheadStepper(**kwargs)]


def test_the_loop_ahead_gives_the_same_tokens_reasons_and_callbacks():
    prompts = [[1, 2, 3], [2, 2], [5], [7, 1]]
    free_run = [expected_tokens(ScriptedStepper(), p, 9) for p in prompts]
    for stop in (free_run[1][2], free_run[0][0], free_run[3][8], 49):
        outcomes = []
        for s in both_loops():
            seen = []
            results = generate(s, prompts, [9, 9, 4, 9], stop_token_ids=[stop], on_token=lambda i, t: seen.append((i, t)))
            outcomes.append(([(r.token_ids, r.finish_reason, r.stop_token) for r in results], seen))
            assert s.state == {} and sorted(s.free) == list(range(s.max_slots))       # every slot came back, once
        assert outcomes[0] == outcomes[1]


def test_the_loop_ahead_steps_a_stopped_sequence_once_in_vain_and_no_more():
    prompts = [[1, 2, 3], [2, 2], [5]]
    plain, ahead = both_loops()
    free_run = [expected_tokens(plain, p, 6) for p in prompts]
    stop = free_run[1][2]
    generate(plain, prompts, 6, stop_token_ids=[stop])
    generate(ahead, prompts, 6, stop_token_ids=[stop])
    rows = lambda s: sum(len(slots) for _, slots in s.steps)
    stopped = sum(1 for tokens in free_run if stop in tokens[:5])     # a stop at the last token costs no extra step
    assert rows(ahead) == rows(plain) + stopped
    # ends by length are known beforehand: nothing is stepped in vain
    plain, ahead = both_loops()
    generate(plain, [[1], [2], [3]], [2, 5, 3])
    generate(ahead, [[1], [2], [3]], [2, 5, 3])
    assert [len(slots) for _, slots in ahead.steps] == [len(slots) for _, slots in plain.steps] == [3, 3, 2, 1, 1]
    assert [e for e in ahead.log if e[0] == "free"] == [("free", 0), ("free", 2), ("free", 1)]


def test_the_loop_ahead_batches_errors_and_limits():
    s = AheadStepper(max_slots=3)
    prompts = [[i + 1] * (i + 1) for i in range(8)]
    results = generate(s, prompts, 4)
    assert [r.token_ids for r in results] == [expected_tokens(s, p, 4) for p in prompts]
    assert s.peak_slots == 3 and s.state == {}
    assert generate(AheadStepper(), [[1, 2], [3]], [0, 1])[1].completion_tokens == 1
    assert generate(AheadStepper(max_position=10), [[1] * 10], 1)[0].completion_tokens == 1

    def on_token(index, token):
        if index == 1:
            raise RuntimeError("consumer went away")

    s = AheadStepper()
    with pytest.raises(RuntimeError, match="went away"):
        generate(s, [[1], [2], [3]], 4, on_token=on_token)
    assert s.state == {}
    # with a callback for logits the plain loop runs (the rows must still be there when the callback looks)
    s = AheadStepper()
    looked = []
    generate(s, [[1], [2]], 3, on_logits=lambda i, step, row: looked.append((i, step)))
    assert s.results_read == 0 and looked == [(0, 0), (1, 0), (0, 1), (1, 1), (0, 2), (1, 2)]


def test_prompts_beyond_a_step_are_fed_in_portions():
    from beholdd.engine.generation import prefill_portions
    assert prefill_portions([5, 11, 17], None) == [[(0, 0, 5), (1, 0, 11), (2, 0, 17)]]
    assert prefill_portions([5, 11, 17], 33) == [[(0, 0, 5), (1, 0, 11), (2, 0, 17)]]
    plan = prefill_portions([5, 11, 17], 8)
    assert plan == [[(0, 0, 5), (1, 0, 3)], [(1, 3, 8)], [(2, 0, 8)], [(2, 8, 8)], [(2, 16, 1)]]
    for lens, cap in (([1, 1, 1], 1), ([40, 3, 29, 64], 16), ([7], 3)):
        plan = prefill_portions(lens, cap)
        assert all(0 < sum(count for _, _, count in step) <= cap for step in plan)
        for index, n in enumerate(lens):       # every prompt whole, in order, each token once
            pieces = [(first, count) for step in plan for i, first, count in step if i == index]
            assert pieces[0][0] == 0 and sum(count for _, count in pieces) == n
            assert all(a[0] + a[1] == b[0] for a, b in zip(pieces, pieces[1:]))


class PortionStepper(ScriptedStepper):
    """The scripted stepper with a limit on a step's tokens: prompts arrive in portions, and a sequence's next
    token is asked for only with the portion that ends its prompt."""

    def __init__(self, max_rows_per_step, **kw):
        super().__init__(**kw)
        self.max_rows_per_step = max_rows_per_step
        self.fed = {}

    def step(self, entries):
        assert sum(len(e.tokens) for e in entries) <= self.max_rows_per_step
        rows = []
        for e in entries:
            started = self.state[e.slot]
            if started is None or started[2]:       # still in its prompt
                first = e.tokens[0] if started is None else started[0]
                length = len(e.tokens) + (0 if started is None else started[1])
                self.state[e.slot] = (first, length, not e.want)
            else:
                first, length, _ = started
                assert e.tokens == [self.next_token(first, length)] and e.want == [0]
                self.state[e.slot] = (first, length + 1, False)
            if e.want:
                assert e.want == [len(e.tokens) - 1]
                first, length, _ = self.state[e.slot]
                row = torch.zeros(self.vocab)
                row[self.next_token(first, length)] = 5.0
                rows.append(row)
        self.steps.append([(e.slot, len(e.tokens)) for e in entries])
        return torch.stack(rows) if rows else None


def test_generation_with_a_limit_on_a_steps_tokens():
    prompts = [[3] * 5, [9] * 11, [4] * 17, [6]]
    s = PortionStepper(8)
    results = generate(s, prompts, [4, 2, 3, 5])
    for prompt, result, n in zip(prompts, results, [4, 2, 3, 5]):
        assert result.token_ids == expected_tokens(s, prompt, n)
    assert s.steps[:6] == [[(0, 5), (1, 3)], [(1, 8)], [(2, 8)], [(2, 8)], [(2, 1), (3, 1)], [(0, 1), (1, 1), (2, 1), (3, 1)]]
    assert s.state == {}
