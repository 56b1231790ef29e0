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


def _sequence(value) -> bool:
    """A list, a tuple or a one-dimensional array: something with a length that can be gone through, and no text."""
    return (hasattr(value, "__len__") and hasattr(value, "__iter__") and not isinstance(value, (str, bytes, dict))
            and getattr(value, "ndim", 1) == 1)


def check_entries(entries: list, cache, vocab: int) -> None:
    """Refuse malformed entries before anything is changed or computed."""
    if not entries:
        raise StepError("a step needs at least one entry")
    for index, entry in enumerate(entries):
        if not isinstance(entry.slot, (int, np.integer)) or isinstance(entry.slot, bool):
            raise StepError(f"entry {index}: the slot is an integer, got {entry.slot!r}")
        if not _sequence(entry.tokens) or not _sequence(entry.want):
            raise StepError(f"entry {index} (slot {entry.slot}): tokens and wanted places are lists")
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


# ---- how a step's numbers lie in one buffer ----------------------------------------------------------------

class StepLayout:
    """The pieces of a step's integer data, their order and their places in ONE int32 buffer, followed by a
    page table [n_seqs, table_width] for every key/value group of the cache.  The step function fills a fresh
    buffer with it and copies it to the device once; a captured decode step keeps a buffer of this layout for
    good and refreshes it before every replay.  A new piece is added here and nowhere else."""

    PIECES = ("tokens", "positions", "row_seq", "seq_start", "seq_slot", "seq_past", "want_rows", "token_src")

    def __init__(self, n_rows: int, n_seqs: int, n_want: int, kv_groups, table_width: int):
        self.n_rows, self.n_seqs, self.n_want = int(n_rows), int(n_seqs), int(n_want)
        self.kv_groups, self.table_width = list(kv_groups), int(table_width)
        sizes = {"tokens": n_rows, "positions": n_rows, "row_seq": n_rows, "seq_start": n_seqs + 1,
                 "seq_slot": n_seqs, "seq_past": n_seqs, "want_rows": n_want, "token_src": n_rows}
        self.place, at = {}, 0
        for name in self.PIECES:
            self.place[name] = (at, at + sizes[name])
            at += sizes[name]
        self.table_place = {}
        for group in self.kv_groups:
            self.table_place[group] = (at, at + n_seqs * self.table_width)
            at += n_seqs * self.table_width
        self.total = at

    def views(self, buffer):
        """Name -> view of `buffer` (a NumPy array or a tensor of `total` int32); "tables" -> {group: [n_seqs, width]}."""
        out = {name: buffer[lo:hi] for name, (lo, hi) in self.place.items()}
        out["tables"] = {group: buffer[lo:hi].reshape(self.n_seqs, self.table_width)
                         for group, (lo, hi) in self.table_place.items()}
        return out

    def fill(self, host, entries: list, pasts: list) -> None:
        """Write everything but the page tables into the host views `host` (from `views`)."""
        if self.n_rows == self.n_seqs:       # one token each: whole pieces at once
            count = np.arange(self.n_seqs + 1, dtype=np.int32)
            host["tokens"][:] = [0 if e.fed_row is not None else e.tokens[0] for e in entries]
            host["token_src"][:] = [-1 if e.fed_row is None else e.fed_row for e in entries]
            host["positions"][:] = pasts
            host["row_seq"][:] = count[:-1]
            host["seq_start"][:] = count
            host["seq_slot"][:] = [e.slot for e in entries]
            host["seq_past"][:] = pasts
            host["want_rows"][:] = [row for row, e in enumerate(entries) for _ in e.want]
            return
        at = want_at = 0
        host["seq_start"][0] = 0
        for index, (entry, past) in enumerate(zip(entries, pasts)):
            n_new = len(entry.tokens)
            fed = entry.fed_row is not None
            host["tokens"][at:at + n_new] = 0 if fed else entry.tokens
            host["token_src"][at:at + n_new] = entry.fed_row if fed else -1
            host["positions"][at:at + n_new] = np.arange(past, past + n_new)
            host["row_seq"][at:at + n_new] = index
            for place in entry.want:
                host["want_rows"][want_at] = at + int(place)
                want_at += 1
            at += n_new
            host["seq_start"][index + 1] = at
            host["seq_slot"][index] = entry.slot
            host["seq_past"][index] = past

    def context(self, device_views, kernels, act_dtype, device, *, max_position: int, max_rows_per_seq: int,
                host=None, fed_tokens=None) -> StepContext:
        """The step as parts see it, over views of the device buffer.  `host` (views of the host copy) gives
        the host-side lists; a captured step has none.  `fed_tokens` switches on tokens read on the device."""
        lists = {name: ([int(v) for v in host[name]] if host is not None else None)
                 for name in ("seq_start", "seq_slot", "seq_past")}
        return StepContext(
            kernels=kernels, act_dtype=act_dtype, device=torch.device(device), n_rows=self.n_rows, n_seqs=self.n_seqs,
            tokens=device_views["tokens"], positions=device_views["positions"], row_seq=device_views["row_seq"],
            seq_start=device_views["seq_start"], seq_slot=device_views["seq_slot"], seq_past=device_views["seq_past"],
            host_seq_start=lists["seq_start"], host_seq_slot=lists["seq_slot"], host_seq_past=lists["seq_past"],
            is_decode=(self.n_rows == self.n_seqs), max_position=int(max_position),
            max_rows_per_seq=int(max_rows_per_seq),
            token_src=device_views["token_src"] if fed_tokens is not None else None, fed_tokens=fed_tokens)


def cache_for_runs(model, cache, tables: dict):
    """`cache_for_run(i)` for a model's forward: the LayerCache of the i-th scheduled run, or None for a
    run whose layer keeps nothing.  `tables`: key/value group index -> page table of this step's sequences."""
    runs, writes, needs = model.schedule, model.run_writes, model.entry_needs

    def cache_for_run(run):
        layer, entry = runs[run]
        if entry not in needs or model.blocks[layer].cache_need() is None:
            return None
        return cache.layer_cache(entry, writes[run], tables)

    return cache_for_run


class StepStaging:
    """Pinned host memory for the numbers of eager steps, a few buffers in turn: the copy to the device does not make
    the host wait for what the stream still has to run (a copy from ordinary memory does), so that the host lays
    out and launches a prompt's next portion while the device works on the one before."""

    RING = 4

    def __init__(self):
        self._buffers = [None] * self.RING
        self._sent = [None] * self.RING
        self._turn = 0

    def send(self, host_buffer: np.ndarray, device) -> torch.Tensor:
        turn = self._turn
        self._turn = (turn + 1) % self.RING
        if self._sent[turn] is not None:
            self._sent[turn].synchronize()      # its last copy, RING steps ago
        pinned = self._buffers[turn]
        if pinned is None or pinned.numel() < host_buffer.size:
            pinned = self._buffers[turn] = torch.empty(max(4096, 2 * host_buffer.size), dtype=torch.int32, pin_memory=True)
        staged = pinned[:host_buffer.size]
        staged.copy_(torch.from_numpy(host_buffer))
        on_device = torch.empty(host_buffer.size, dtype=torch.int32, device=device)
        on_device.copy_(staged, non_blocking=True)
        self._sent[turn] = torch.cuda.Event()
        self._sent[turn].record()
        return on_device


def build_step(kernels, act_dtype, device, cache, entries: list, staging: StepStaging | None = None):
    """Lay out a step whose entries were checked and whose room was reserved: one buffer, one copy to the
    device (through `staging`, if given and the device is a GPU, without a wait).  Returns (context, want_rows
    tensor, page tables by key/value group)."""
    pasts = [cache.length(entry.slot) for entry in entries]
    slots = [entry.slot for entry in entries]
    n_rows = sum(len(entry.tokens) for entry in entries)
    kv_groups = cache.kv_group_indices()
    width = max([1] + [cache.pages_held(group, slot) for group in kv_groups for slot in slots])
    layout = StepLayout(n_rows, len(entries), sum(len(entry.want) for entry in entries), kv_groups, width)
    host_buffer = np.zeros(layout.total, dtype=np.int32)
    host = layout.views(host_buffer)
    layout.fill(host, entries, pasts)
    for group in kv_groups:
        cache.write_page_table(group, slots, host["tables"][group])
    if staging is not None and torch.device(device).type == "cuda":
        views = layout.views(staging.send(host_buffer, device))
    else:
        views = layout.views(torch.from_numpy(host_buffer).to(device))
    ctx = layout.context(views, kernels, act_dtype, device, host=host,
                         max_position=max(past + len(entry.tokens) for entry, past in zip(entries, pasts)) - 1,
                         max_rows_per_seq=max(len(entry.tokens) for entry in entries))
    return ctx, views["want_rows"], views["tables"]
