"""The cache: a slot for each live sequence, paged keys and values, fixed-size state.

Layout.  A *slot* is one sequence's handle: its length, its pages and its row in every state
region.  Layers are sorted into *groups* by what they need (`CacheNeed`): every group has
storage of its own.  A key/value group holds, for each of its cache entries (one per
scheduled layer run that writes a cache), keys [pages, kv_heads, page_size, head_dim] and values
[pages, kv_heads, head_dim, page_size] (the order of one head's elements inside a page is the
kernel library's: the kernel that writes them and the attention kernels agree on it, and the
cache itself never looks inside); a sequence's position p lives in page `table[p // page_size]`
at token `p % page_size`, and a
group with a window gives pages back once every position in them has left the window.  A
state group holds [entries, max_slots, *shape] and a slot's rows are zero when it starts.

Rules kept from the reference's single-sequence caches: a step first *reserves* room for all
its new tokens or changes nothing (append refuses without mutating,
crates/beholdd-model/src/qwen3moe/forward.rs:201-226); lengths are *committed* once, after the
whole step (:902-914, crates/beholdd-model/src/recorded_model.rs:498-510); a slot that is given
back is used again without clearing, because every row is written before it can be read
(crates/beholdd-model/src/recorded_attention.rs:704-712); and the bytes are accounted for
before anything is allocated (recorded_attention.rs:244-299).
"""

from __future__ import annotations

import heapq
import numbers
from dataclasses import dataclass, field

import torch

from ..parts.base import CacheNeed, LayerCache


class CacheError(RuntimeError):
    """A slot or page was used against the rules (double free, unknown slot...)."""


class CacheFull(CacheError):
    """Not enough free pages or slots; nothing was changed."""


def _element_size(dtype: torch.dtype) -> int:
    return torch.empty((), dtype=dtype).element_size()


@dataclass
class GroupPlan:
    need: CacheNeed
    entries: list
    kv_bytes: int
    state_bytes: int


@dataclass
class CachePlan:
    """Byte accounting, computed from sizes alone."""
    page_size: int
    n_pages: int
    max_slots: int
    groups: list = field(default_factory=list)

    @property
    def total_bytes(self) -> int:
        return sum(g.kv_bytes + g.state_bytes for g in self.groups)

    def describe(self) -> str:
        lines = [f"cache: {self.n_pages} pages of {self.page_size} tokens, up to {self.max_slots} sequences, "
                 f"{self.total_bytes} bytes"]
        for g in self.groups:
            if g.need.kind == "kv":
                window = f", window {g.need.window}" if g.need.window else ""
                lines.append(f"  keys/values of {len(g.entries)} layers ({g.need.kv_heads} heads x "
                             f"{g.need.head_dim}{window}): {g.kv_bytes} bytes")
            else:
                lines.append(f"  state {tuple(g.need.state_shape)} of {len(g.entries)} layers: {g.state_bytes} bytes")
        return "\n".join(lines)


class _Group:
    def __init__(self, need: CacheNeed, entries: list):
        self.need = need
        self.entries = list(entries)
        self.index_of = {entry: i for i, entry in enumerate(self.entries)}
        self.k = self.v = self.state = None
        self.free_pages: list = []
        self.pages_of: dict = {}     # slot -> list of page ids (or -1 once released), position order


_MOST_SLOTS = 1 << 20     # every slot has a place in the free list and a row in each table


class SequenceCache:
    def __init__(self, entry_needs: dict, max_tokens: int, dtype: torch.dtype, device, page_size: int,
                 max_slots: int | None = None, max_position: int | None = None):
        for name, value, optional in (("max_tokens", max_tokens, False), ("max_slots", max_slots, True),
                                      ("max_position", max_position, True)):
            if value is None and optional:
                continue
            if isinstance(value, bool) or not isinstance(value, numbers.Integral) or not 0 <= value < 1 << 40:
                raise ValueError(f"{name} is a count of tokens or sequences (an integer below 2^40), got {value!r}")
        if max_tokens <= 0:
            raise ValueError("the cache must hold at least one token")
        if max_slots is not None and max_slots > _MOST_SLOTS:
            raise ValueError(f"max_slots is at most {_MOST_SLOTS}, got {max_slots}")
        self.page_size = int(page_size)
        self.n_pages = -(-int(max_tokens) // self.page_size)
        self.max_slots = int(max_slots) if max_slots else min(self.n_pages, 1024)
        self.max_position = int(max_position) if max_position else self.n_pages * self.page_size
        self.dtype, self.device = dtype, torch.device(device)
        by_need: dict = {}
        for entry in sorted(entry_needs):
            by_need.setdefault(entry_needs[entry], []).append(entry)
        self.groups = [_Group(need, entries) for need, entries in by_need.items()]
        self.group_of_entry = {entry: g for g in self.groups for entry in g.entries}
        self._free_slots = list(range(self.max_slots))
        heapq.heapify(self._free_slots)
        self._length: dict = {}      # live slot -> committed length
        self._allocated = False
        self._state_before: list = []    # (group, slot indices, their state rows) as they were before the running step

    # ---- accounting and allocation ----
    def plan(self) -> CachePlan:
        plan = CachePlan(self.page_size, self.n_pages, self.max_slots)
        for g in self.groups:
            kv = state = 0
            if g.need.kind == "kv":
                kv = (len(g.entries) * 2 * self.n_pages * g.need.kv_heads * self.page_size * g.need.head_dim
                      * _element_size(self.dtype))
            else:
                count = 1
                for axis in g.need.state_shape:
                    count *= axis
                state = len(g.entries) * self.max_slots * count * _element_size(g.need.state_dtype)
            plan.groups.append(GroupPlan(g.need, g.entries, kv, state))
        return plan

    def allocate(self, limit_bytes: int | None = None) -> CachePlan:
        plan = self.plan()
        if limit_bytes is not None and plan.total_bytes > limit_bytes:
            raise CacheFull(f"the cache needs {plan.total_bytes} bytes, the limit is {limit_bytes}")
        for g in self.groups:
            if g.need.kind == "kv":
                head = (len(g.entries), self.n_pages, g.need.kv_heads)
                # zeros, not empty: rows of a page that no token has written yet must hold finite numbers
                g.k = torch.zeros((*head, self.page_size, g.need.head_dim), dtype=self.dtype, device=self.device)
                g.v = torch.zeros((*head, g.need.head_dim, self.page_size), dtype=self.dtype, device=self.device)
                g.free_pages = list(range(self.n_pages - 1, -1, -1))   # pop() hands out page 0 first
            else:
                g.state = torch.zeros((len(g.entries), self.max_slots, *g.need.state_shape),
                                      dtype=g.need.state_dtype, device=self.device)
        self._allocated = True
        return plan

    def allocated_bytes(self) -> int:
        total = 0
        for g in self.groups:
            for tensor in (g.k, g.v, g.state):
                if tensor is not None:
                    total += tensor.numel() * tensor.element_size()
        return total

    # ---- slots ----
    def alloc_slot(self) -> int:
        if not self._free_slots:
            raise CacheFull(f"all {self.max_slots} sequence slots are in use")
        slot = heapq.heappop(self._free_slots)
        self._length[slot] = 0
        for g in self.groups:
            if g.need.kind == "kv":
                g.pages_of[slot] = []
            elif g.state is not None:
                g.state[:, slot].zero_()
        return slot

    def free_slot(self, slot: int) -> None:
        if slot not in self._length:
            raise CacheError(f"slot {slot} is not in use (freed twice, or never given out)")
        del self._length[slot]
        for g in self.groups:
            if g.need.kind == "kv":
                for page in g.pages_of.pop(slot):
                    if page >= 0:
                        g.free_pages.append(page)
        heapq.heappush(self._free_slots, slot)

    def live_slots(self) -> list:
        return sorted(self._length)

    def length(self, slot: int) -> int:
        try:
            return self._length[slot]
        except KeyError:
            raise CacheError(f"slot {slot} is not in use") from None

    def free_page_count(self) -> int:
        kv = [len(g.free_pages) for g in self.groups if g.need.kind == "kv"]
        return min(kv) if kv else self.n_pages

    # ---- a step: reserve, run, commit ----
    def reserve(self, requests: list) -> None:
        """Make room for `n_new` more tokens of each (slot, n_new), or change nothing."""
        seen = set()
        for slot, n_new in requests:
            if slot in seen:
                raise CacheError(f"slot {slot} occurs twice in one step")
            seen.add(slot)
            if n_new <= 0:
                raise CacheError(f"slot {slot}: a step brings at least one token")
            end = self.length(slot) + n_new
            if end > self.max_position:
                raise CacheFull(f"slot {slot}: {end} positions exceed the limit of {self.max_position}")
        for g in self.groups:
            if g.need.kind != "kv":
                continue
            wanted = 0
            for slot, n_new in requests:
                have = len(g.pages_of[slot])
                wanted += max(0, -(-(self._length[slot] + n_new) // self.page_size) - have)
            if wanted > len(g.free_pages):
                raise CacheFull(f"the step needs {wanted} more cache pages of {self.page_size} tokens, "
                                f"{len(g.free_pages)} are free")
        for g in self.groups:
            if g.need.kind != "kv":
                continue
            for slot, n_new in requests:
                pages = g.pages_of[slot]
                while len(pages) * self.page_size < self._length[slot] + n_new:
                    pages.append(g.free_pages.pop())
        # State regions are updated in place while the step runs; keep what the step's slots held, so that a
        # failed step can put it back (the key/value pages need no such copy: rows beyond a sequence's length are
        # never read).
        self._state_before = []
        for g in self.groups:
            if g.need.kind == "state" and g.state is not None:
                index = torch.tensor([slot for slot, _ in requests], dtype=torch.long, device=self.device)
                self._state_before.append((g, index, g.state.index_select(1, index)))

    def commit(self, requests: list) -> None:
        """The step succeeded: the new tokens become part of their sequences."""
        self._state_before = []
        for slot, n_new in requests:
            self._length[slot] += n_new
        for g in self.groups:
            if g.need.kind != "kv" or not g.need.window:
                continue
            for slot, _ in requests:
                # the next query stands at position length; it sees positions > length - window
                dead_before = self._length[slot] - g.need.window + 1
                pages = g.pages_of[slot]
                for index in range(min(len(pages), max(0, dead_before) // self.page_size)):
                    if pages[index] >= 0:
                        g.free_pages.append(pages[index])
                        pages[index] = -1

    def rollback(self, requests: list) -> None:
        """The step failed: give back pages that `reserve` took beyond the committed lengths, and put back
        the state that the step's sequences held before it."""
        for g, index, before in self._state_before:
            g.state.index_copy_(1, index, before)
        self._state_before = []
        for g in self.groups:
            if g.need.kind != "kv":
                continue
            for slot, _ in requests:
                if slot not in self._length:
                    continue
                pages = g.pages_of[slot]
                keep = -(-self._length[slot] // self.page_size)
                while len(pages) > keep:
                    page = pages.pop()
                    if page >= 0:
                        g.free_pages.append(page)
                g.pages_of[slot] = list(pages)   # a new list: whoever remembers the old one sees that entries went away

    # ---- what kernels and mixers get ----
    def kv_group_indices(self) -> list:
        """The indices (into `groups`) of the groups that hold keys and values."""
        return [index for index, g in enumerate(self.groups) if g.need.kind == "kv"]

    def pages_held(self, group: int, slot: int) -> int:
        return len(self.groups[group].pages_of[slot])

    def write_page_table(self, group: int, slots: list, out) -> None:
        """Write the page ids of `slots` into `out` [len(slots), width] (a host array): a row per sequence in
        position order, 0 where a page was given back or none is held yet."""
        g = self.groups[group]
        for row, slot in enumerate(slots):
            pages = g.pages_of[slot]
            out[row, :] = 0
            out[row, :len(pages)] = [max(page, 0) for page in pages]

    def page_tables(self, slots: list, min_width: int = 1) -> dict:
        """For each key/value group, an int32 device tensor [len(slots), width] of page ids."""
        import numpy as np

        tables = {}
        for index in self.kv_group_indices():
            width = max(min_width, max(self.pages_held(index, slot) for slot in slots))
            host = np.zeros((len(slots), width), dtype=np.int32)
            self.write_page_table(index, slots, host)
            tables[index] = torch.from_numpy(host).to(self.device, non_blocking=False)
        return tables

    def layer_cache(self, entry: int, writes: bool, tables: dict) -> LayerCache:
        g = self.group_of_entry[entry]
        at = g.index_of[entry]
        if g.need.kind == "kv":
            return LayerCache(g.need, writes, k_pages=g.k[at], v_pages=g.v[at],
                              page_table=tables[self.groups.index(g)])
        return LayerCache(g.need, writes, state=g.state[at])

    # ---- self-check, for tests ----
    def check_invariants(self) -> None:
        live, free = set(self._length), set(self._free_slots)
        if live & free:
            raise CacheError(f"slots {sorted(live & free)} are both free and in use")
        if len(self._free_slots) != len(free):
            raise CacheError("a slot is on the free list twice")
        if live | free != set(range(self.max_slots)):
            raise CacheError(f"slots {sorted(set(range(self.max_slots)) - live - free)} are lost")
        for g in self.groups:
            if g.need.kind != "kv" or not self._allocated:
                continue
            held = [p for pages in g.pages_of.values() for p in pages if p >= 0]
            if len(held) != len(set(held)):
                raise CacheError("a cache page is held twice")
            if len(g.free_pages) != len(set(g.free_pages)):
                raise CacheError("a cache page is on the free list twice")
            if set(held) & set(g.free_pages):
                raise CacheError("a cache page is both held and free")
            if len(held) + len(g.free_pages) != self.n_pages:
                raise CacheError(f"{self.n_pages - len(held) - len(g.free_pages)} cache pages are lost")
            if set(g.pages_of) != live:
                raise CacheError("page lists and live slots disagree")
            for slot, pages in g.pages_of.items():
                if len(pages) * self.page_size < self._length[slot]:
                    raise CacheError(f"slot {slot} holds fewer pages than its length needs")
