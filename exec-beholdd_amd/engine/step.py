"""One step over a batch of sequences with unequal lengths.

The reference's step is `forward_cached_chunk(tokens, cache)`: one sequence, a chunk of any
length starting where the cache ends, logits of the last position
(crates/beholdd-model/src/qwen3moe/forward.rs:811-915).  Here a step takes several sequences
at once, each with its own next tokens, flattened row after row; every row carries its
absolute position and its sequence, so nothing is padded and a row's result does not depend
on what else is in the batch.  Checks come before any arithmetic (:821-848), and lengths
change only after the whole step succeeded (:902-914).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from ..parts.base import StepContext


class StepError(ValueError):
    """A step's entries are malformed."""


@dataclass
class StepEntry:
    slot: int
    tokens: list
    want: list = field(default_factory=list)   # indices into `tokens` whose logits are returned
    fed_row: int | None = None                 # the entry's one token is not `tokens[0]` (ignored then) but stands
                                               # at this row of the sampler's device buffer, not yet seen by the host


def check_entries(entries: list, cache, vocab: int) -> None:
    """Refuse malformed entries before anything is changed or computed."""
    if not entries:
        raise StepError("a step needs at least one entry")
    for index, entry in enumerate(entries):
        n_new = len(entry.tokens)
        if n_new == 0:
            raise StepError(f"entry {index} (slot {entry.slot}) brings no tokens")
        cache.length(entry.slot)       # raises for a slot that is not in use
        if entry.fed_row is not None:
            if n_new != 1 or not isinstance(entry.fed_row, (int, np.integer)) or entry.fed_row < 0:
                raise StepError(f"entry {index} (slot {entry.slot}): a token fed on the device is one token from a "
                                f"row >= 0, got {n_new} tokens and row {entry.fed_row!r}")
        for token in (entry.tokens if entry.fed_row is None else ()):
            if not isinstance(token, (int, np.integer)) or isinstance(token, bool) or not 0 <= token < vocab:
                raise StepError(f"entry {index} (slot {entry.slot}): token {token!r} is outside the vocabulary "
                                f"of {vocab}")
        for place in entry.want:
            if not isinstance(place, (int, np.integer)) or isinstance(place, bool) or not 0 <= place < n_new:
                raise StepError(f"entry {index} (slot {entry.slot}): wanted place {place!r} is outside its "
                                f"{n_new} tokens")


def build_step(kernels, act_dtype, device, cache, entries: list, vocab: int):
    """Check the entries and lay the step out.  Returns (context, want_rows tensor, requests)."""
    check_entries(entries, cache, vocab)
    tokens, positions, row_seq, seq_start, seq_slot, seq_past, want_rows = [], [], [], [0], [], [], []
    requests = []
    for index, entry in enumerate(entries):
        n_new = len(entry.tokens)
        past = cache.length(entry.slot)
        for place in entry.want:
            want_rows.append(len(tokens) + int(place))
        tokens.extend(int(t) for t in entry.tokens)
        positions.extend(range(past, past + n_new))
        row_seq.extend([index] * n_new)
        seq_start.append(len(tokens))
        seq_slot.append(entry.slot)
        seq_past.append(past)
        requests.append((entry.slot, n_new))

    n_rows, n_seqs = len(tokens), len(entries)
    pieces = [tokens, positions, row_seq, seq_start, seq_slot, seq_past, want_rows]
    packed = torch.from_numpy(np.concatenate([np.asarray(p, dtype=np.int32) for p in pieces]))
    packed = packed.to(device)
    views, at = [], 0
    for piece in pieces:
        views.append(packed[at:at + len(piece)])
        at += len(piece)
    ctx = StepContext(
        kernels=kernels, act_dtype=act_dtype, device=torch.device(device), n_rows=n_rows, n_seqs=n_seqs,
        tokens=views[0], positions=views[1], row_seq=views[2], seq_start=views[3], seq_slot=views[4],
        seq_past=views[5], host_seq_start=seq_start, host_seq_slot=seq_slot, host_seq_past=seq_past,
        is_decode=(n_rows == n_seqs), max_position=max(positions),
        max_rows_per_seq=max(n for _, n in requests))
    return ctx, views[6], requests
