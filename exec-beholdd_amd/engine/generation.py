"""The generation loop above the step function.

For one sequence this is the reference's loop (crates/beholdd-model/src/qwen3moe/forward.rs:597-686):
the whole prompt in one step, then one token per step; a selected stop token is reported but
neither emitted, appended nor evaluated (:655-661); the last emitted token is never evaluated
(:664), so a request needs prompt + max_new - 1 positions (:612-625); max_new = 0 returns at
once without touching the model (:628-634).  Here a batch of sequences with unequal prompts
runs together: all prompts in one step, then one token each; a sequence that ends leaves the
batch and gives its slot back while the others go on; and requests beyond one batch run as
one batch after another.

The loop decides on the host and talks to the model only through a *stepper*:
    stepper.page_size, stepper.capacity_pages, stepper.max_slots, stepper.max_position
    stepper.alloc_slot() -> slot;  stepper.free_slot(slot)
    stepper.step(entries: list[StepEntry]) -> logits (one row per entry that wants one)
    stepper.select(logits, params, request_indices, steps) -> list[int]
A stepper may say `stepper.max_rows_per_step`: the most tokens one step takes.  Prompts that together bring more
are fed in portions, step after step, before the first token is chosen (`prefill`); the step function gives the
same logits however the tokens are cut.
A stepper may also offer
    stepper.select_async(logits, params, request_indices, steps) -> selection with `result() -> list[int]`,
        `device_rows` and `take(positions)`
    and take `StepEntry(slot, [0], [0], fed_row=r)`: the token at row r of the last selection, read on
    the device.
Then the loop runs one step ahead of what it knows: it starts the next step for every sequence that has
tokens left to generate before it looks at the tokens just chosen, so the device never waits for the host.
A sequence that turns out to have chosen a stop token has then been stepped once in vain; its slot is
freed as always and what that step computed for it is dropped.  The tokens, their order and the finish
reasons are those of the plain loop.
"""

from __future__ import annotations

import numbers
from dataclasses import dataclass, field

from ..sampling import SamplingParams
from .step import StepEntry

FINISH_LENGTH = "length"     # the reference's MaxNewTokens -> Length (crates/beholdd-runtime/src/native.rs:662-665)
FINISH_STOP = "stop"         # StopToken -> Stop


class GenerationError(ValueError):
    pass


@dataclass
class GenerationResult:
    token_ids: list = field(default_factory=list)
    finish_reason: str = FINISH_LENGTH
    stop_token: int | None = None
    prompt_tokens: int = 0

    @property
    def completion_tokens(self) -> int:
        return len(self.token_ids)


def positions_needed(prompt_len: int, max_new: int) -> int:
    """Positions a request evaluates: the last selected token is never fed back."""
    return prompt_len + max_new - (1 if max_new > 0 else 0)


def plan_batches(prompt_lens: list, max_new: list, page_size: int, capacity_pages: int, max_slots: int,
                 batch_size: int | None) -> list:
    """Split requests, in order, into batches that fit the cache: lists of request indices."""
    limit = min(max_slots, batch_size) if batch_size else max_slots
    batches, current, pages = [], [], 0
    for index, (n_prompt, n_new) in enumerate(zip(prompt_lens, max_new)):
        if n_new == 0:
            continue
        need = -(-positions_needed(n_prompt, n_new) // page_size)
        if need > capacity_pages:
            raise GenerationError(
                f"request {index} needs {need} cache pages of {page_size} tokens, the cache has {capacity_pages}")
        if current and (len(current) >= limit or pages + need > capacity_pages):
            batches.append(current)
            current, pages = [], 0
        current.append(index)
        pages += need
    if current:
        batches.append(current)
    return batches


def _whole_number(value) -> bool:
    return isinstance(value, numbers.Integral) and not isinstance(value, bool)


def _token_sequence(value) -> bool:
    """A list, a tuple, an array: something with a length that can be gone through, and no text."""
    return hasattr(value, "__len__") and hasattr(value, "__iter__") and not isinstance(value, (str, bytes, dict))


def generate(stepper, prompts: list, max_new_tokens, sampling=None, stop_token_ids=(), on_token=None,
             batch_size: int | None = None, control=None, on_logits=None) -> list:
    """Generate for every prompt (a list of token ids each).

    `max_new_tokens` and `sampling` are one value for all requests or a list with one per
    request.  `on_token(request_index, token)` is called for every emitted token in order;
    `control()` is polled before every step and may raise to cancel;
    `on_logits(request_index, step, logits_row)` sees the device row each token is chosen from.
    """
    if not _token_sequence(prompts):
        raise GenerationError(f"prompts are a list of lists of token ids, got {prompts!r}")
    n = len(prompts)
    max_new = list(max_new_tokens) if isinstance(max_new_tokens, (list, tuple)) else [max_new_tokens] * n
    if sampling is None:
        sampling = SamplingParams()
    params = list(sampling) if isinstance(sampling, (list, tuple)) else [sampling] * n
    if len(max_new) != n or len(params) != n:
        raise GenerationError("one max_new_tokens and one sampling parameter set per prompt")
    if not _token_sequence(stop_token_ids) or not all(_whole_number(t) for t in stop_token_ids):
        raise GenerationError(f"stop_token_ids are a list of token ids, got {stop_token_ids!r}")
    stops = frozenset(int(t) for t in stop_token_ids)
    if batch_size is not None and not _whole_number(batch_size):
        raise GenerationError(f"batch_size is an integer or None, got {batch_size!r}")
    for index, (prompt, n_new) in enumerate(zip(prompts, max_new)):
        if not _token_sequence(prompt):
            raise GenerationError(f"request {index}: a prompt is a list of token ids, got {prompt!r}")
        if len(prompt) == 0:
            raise GenerationError(f"request {index}: generation requires at least one prompt token")
        if not _whole_number(n_new):
            raise GenerationError(f"request {index}: max_new_tokens is an integer, got {n_new!r}")
        if n_new < 0:
            raise GenerationError(f"request {index}: max_new_tokens must not be negative")
        needed = positions_needed(len(prompt), n_new)
        if needed > stepper.max_position:
            raise GenerationError(
                f"request {index}: prompt plus {n_new} generated tokens needs {needed} evaluated positions, "
                f"exceeding the context of {stepper.max_position}")
    results = [GenerationResult(prompt_tokens=len(p)) for p in prompts]
    batches = plan_batches([len(p) for p in prompts], max_new, stepper.page_size, stepper.capacity_pages,
                           stepper.max_slots, batch_size)
    for batch in batches:
        _run_batch(stepper, batch, prompts, max_new, params, stops, on_token, control, results, on_logits)
    return results


def prefill_portions(prompt_lens: list, max_rows: int | None) -> list:
    """How the prompts of a batch go through steps of at most `max_rows` tokens: a list of steps, each a list of
    (index into the batch, first token, tokens).  Prompts are taken in order; a step is filled before the next
    one starts, so a prompt may be cut where a step is full."""
    if not max_rows or sum(prompt_lens) <= max_rows:
        return [[(index, 0, n) for index, n in enumerate(prompt_lens)]]
    steps, current, room = [], [], max_rows
    for index, n in enumerate(prompt_lens):
        fed = 0
        while fed < n:
            take = min(n - fed, room)
            current.append((index, fed, take))
            fed += take
            room -= take
            if room == 0:
                steps.append(current)
                current, room = [], max_rows
    if current:
        steps.append(current)
    return steps


def prefill(stepper, slots: list, prompts: list, control=None):
    """Feed every prompt whole, in as many steps as `stepper.max_rows_per_step` asks for; returns the logits of
    each prompt's last token, one row per prompt in order."""
    plan = prefill_portions([len(p) for p in prompts], getattr(stepper, "max_rows_per_step", None))
    if len(plan) == 1:
        return stepper.step([StepEntry(slot, list(prompt), [len(prompt) - 1]) for slot, prompt in zip(slots, prompts)])
    import torch
    rows = [None] * len(prompts)
    for number, portion in enumerate(plan):
        if number and control is not None:
            control()
        entries, ending = [], []
        for index, first, count in portion:
            last = first + count == len(prompts[index])
            entries.append(StepEntry(slots[index], list(prompts[index][first:first + count]), [count - 1] if last else []))
            if last:
                ending.append(index)
        logits = stepper.step(entries)
        for row, index in enumerate(ending):
            rows[index] = logits[row]
    return torch.stack(rows)


def _run_batch(stepper, batch, prompts, max_new, params, stops, on_token, control, results, on_logits):
    if on_logits is None and hasattr(stepper, "select_async"):
        return _run_batch_ahead(stepper, batch, prompts, max_new, params, stops, on_token, control, results)
    slots = {}
    try:
        for index in batch:
            slots[index] = stepper.alloc_slot()
        if control is not None:
            control()
        live = list(batch)
        logits = prefill(stepper, [slots[i] for i in live], [prompts[i] for i in live], control)
        step = 0
        while live:
            tokens = stepper.select(logits, [params[i] for i in live], live, [step] * len(live))
            if on_logits is not None:
                for row, index in enumerate(live):
                    on_logits(index, step, logits[row])
            going = []
            for index, token in zip(live, tokens):
                result = results[index]
                if token in stops:
                    result.finish_reason, result.stop_token = FINISH_STOP, token
                else:
                    if on_token is not None:
                        on_token(index, token)
                    result.token_ids.append(token)
                    if len(result.token_ids) < max_new[index]:
                        going.append((index, token))
                        continue
                    result.finish_reason = FINISH_LENGTH
                stepper.free_slot(slots.pop(index))    # the sequence has ended; its slot is free at once
            live = [index for index, _ in going]
            if not live:
                break
            if control is not None:
                control()
            logits = stepper.step([StepEntry(slots[index], [token], [0]) for index, token in going])
            step += 1
    finally:
        for slot in slots.values():
            stepper.free_slot(slot)


def decode_ahead(stepper, slots: list, chosen, params: list, requests: list, steps: list):
    """One decode step of the sequences in `slots`, started before the host knows their tokens: `chosen` is the
    selection (not waited for) that holds them, one element per slot, and the step reads them on the device.
    Returns the selection of this step's tokens, not waited for either."""
    logits = stepper.step([StepEntry(slot, [0], [0], fed_row=row) for slot, row in zip(slots, chosen.device_rows)])
    return stepper.select_async(logits, params, requests, steps)


def _run_batch_ahead(stepper, batch, prompts, max_new, params, stops, on_token, control, results):
    """`_run_batch` one step ahead of the host (see the module's text)."""
    slots = {}
    try:
        for index in batch:
            slots[index] = stepper.alloc_slot()
        if control is not None:
            control()
        live = list(batch)
        logits = prefill(stepper, [slots[i] for i in live], [prompts[i] for i in live], control)
        step = 0
        chosen = stepper.select_async(logits, [params[i] for i in live], live, [step] * len(live))
        while live:
            # those that go on unless the token being chosen for them is a stop token: step them already
            ahead = [at for at, index in enumerate(live) if len(results[index].token_ids) + 1 < max_new[index]]
            chosen_ahead = None
            if ahead:
                if control is not None:
                    control()
                chosen_ahead = decode_ahead(stepper, [slots[live[at]] for at in ahead], chosen.take(ahead),
                                            [params[live[at]] for at in ahead], [live[at] for at in ahead],
                                            [step + 1] * len(ahead))
            tokens = chosen.result()
            going = set()
            for index, token in zip(live, tokens):
                result = results[index]
                if token in stops:
                    result.finish_reason, result.stop_token = FINISH_STOP, token
                else:
                    if on_token is not None:
                        on_token(index, token)
                    result.token_ids.append(token)
                    if len(result.token_ids) < max_new[index]:
                        going.add(index)
                        continue
                    result.finish_reason = FINISH_LENGTH
                stepper.free_slot(slots.pop(index))    # the sequence has ended; its slot is free at once
            if chosen_ahead is None:
                break
            kept = [position for position, at in enumerate(ahead) if live[at] in going]
            live = [live[ahead[position]] for position in kept]
            chosen = chosen_ahead.take(kept)
            step += 1
    finally:
        for slot in slots.values():
            stepper.free_slot(slot)
