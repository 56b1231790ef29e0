"""Decode steps as HIP graphs.

A decode step launches a few hundred small kernels; replaying them as one captured graph takes
the host out of the loop.  A graph is captured for a given number of sequences and a given
page-table width (the longest sequence's pages, rounded up to a bucket) and replayed for every
later step of that shape: the step's numbers (tokens, positions, slots, page tables) live in one
static device buffer that is refreshed with a single copy before each replay.

Only kernels go into a graph: no memset nodes, no library calls (torch only hands out the
temporaries, from the graph's private pool).  Parts whose `forward` reads the step's host-side
lists would bake one step's values into the graph, so a model is captured only if every part
declares `graph_safe = True`.
"""

from __future__ import annotations

import gc
import weakref

import numpy as np
import torch

from ..parts.base import LayerCache, StepContext

def _weakly(engine):
    return engine if isinstance(engine, weakref.ProxyTypes) else weakref.proxy(engine)


PAGE_BUCKET = 16      # page-table widths are rounded up to a multiple of this many pages


class DecodeGraph:
    def __init__(self, engine, n_seqs: int, table_width: int):
        # the engine owns its graphs; they point back weakly, so that an engine nobody holds any more is
        # freed at once and not by a later garbage collection
        self.engine, self.n_seqs, self.table_width = _weakly(engine), n_seqs, table_width
        cache = engine.cache
        self.kv_groups = [index for index, g in enumerate(cache.groups) if g.need.kind == "kv"]
        b = n_seqs
        self.n_meta = 8 * b + 1
        total = self.n_meta + len(self.kv_groups) * b * table_width
        self.host = torch.zeros(total, dtype=torch.int32).pin_memory()
        self.device = torch.zeros(total, dtype=torch.int32, device=engine.device)
        view, at = [], 0
        for size in (b, b, b, b + 1, b, b, b, b):
            view.append(self.device[at:at + size])
            at += size
        self.tables = {}
        for index in self.kv_groups:
            self.tables[index] = self.device[at:at + b * table_width].view(b, table_width)
            at += b * table_width
        page = cache.page_size
        self.ctx = StepContext(
            kernels=engine.kernels, act_dtype=engine.dtype, device=engine.device, n_rows=b, n_seqs=b,
            tokens=view[0], positions=view[1], row_seq=view[2], seq_start=view[3], seq_slot=view[4],
            seq_past=view[5], host_seq_start=None, host_seq_slot=None, host_seq_past=None, is_decode=True,
            max_position=min(table_width * page, cache.max_position) - 1, max_rows_per_seq=1,
            token_src=view[7], fed_tokens=engine.sampler.device_tokens)
        self.want_rows = view[6]
        self.fed_buffer = engine.sampler.out       # the capture holds its address
        self.graph = None
        self.logits = None
        self.copied = None        # event: the last host-to-device copy of the step's numbers is done
        self.known = {}           # kv group -> per row (the page list the host table row was written from, how far)

    def fill(self, entries, pasts):
        """Write this step's numbers into the static buffer (one host-to-device copy)."""
        b, cache = self.n_seqs, self.engine.cache
        if self.copied is not None:
            self.copied.synchronize()     # the pinned buffer may not change under a copy in flight
        host = self.host.numpy()
        slots = [e.slot for e in entries]
        host[0:b] = [e.tokens[0] if e.fed_row is None else 0 for e in entries]
        host[7 * b + 1:8 * b + 1] = [-1 if e.fed_row is None else e.fed_row for e in entries]
        host[b:2 * b] = pasts
        host[2 * b:3 * b] = np.arange(b)
        host[3 * b:4 * b + 1] = np.arange(b + 1)
        host[4 * b + 1:5 * b + 1] = slots
        host[5 * b + 1:6 * b + 1] = pasts
        host[6 * b + 1:7 * b + 1] = np.arange(b)
        at = self.n_meta
        for index in self.kv_groups:
            table = host[at:at + b * self.table_width].reshape(b, self.table_width)
            group = cache.groups[index]
            known = self.known.setdefault(index, [(None, 0)] * b)
            for row, slot in enumerate(slots):
                pages = group.pages_of[slot]
                before, count = known[row]
                # a sequence's page list only grows while it lives (a window apart), so a row that was
                # written for this very list needs its new pages only
                if before is pages and count <= len(pages) and not group.need.window:
                    for j in range(count, len(pages)):
                        table[row, j] = pages[j]
                else:
                    table[row, :] = 0
                    table[row, :len(pages)] = [max(page, 0) for page in pages]
                known[row] = (pages, len(pages))
            at += b * self.table_width
        self.device.copy_(self.host, non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()

    def _forward(self):
        engine = self.engine
        model, cache = engine.model, engine.cache
        runs, writes = model.schedule, model.run_writes

        def cache_for_run(run):
            entry = runs[run][1]
            if entry not in model.entry_needs or model.blocks[runs[run][0]].cache_need() is None:
                return None
            return cache.layer_cache(entry, writes[run], self.tables)

        return model.forward(self.ctx, cache_for_run, self.want_rows)

    def run(self):
        """Replay (capturing first if need be); the logits tensor is reused by the next run."""
        if self.graph is None:
            self._forward()                      # once eagerly: loads every kernel before the capture
            torch.cuda.synchronize(self.engine.device)
            graph = torch.cuda.CUDAGraph()
            # No garbage collection while the stream is capturing: it could free another engine's graphs or
            # memory there, and the runtime refuses such calls during a capture (the process aborts).
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph):
                    self.logits = self._forward()
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
        self.graph.replay()
        return self.logits


class DecodeGraphs:
    """The graphs of one engine, by (sequences, page-table width)."""

    def __init__(self, engine, limit: int = 48):
        self.engine, self.limit = _weakly(engine), limit
        self.graphs: dict = {}

    def usable(self, ctx_entries) -> bool:
        model = self.engine.model
        return (getattr(model, "graph_safe", False) and self.engine.device.type == "cuda"
                and all(len(e.tokens) == 1 for e in ctx_entries))

    def step(self, entries, pasts):
        cache = self.engine.cache
        pages = max(-(-(past + 1) // cache.page_size) for past in pasts)
        width = -(-pages // PAGE_BUCKET) * PAGE_BUCKET
        key = (len(entries), width)
        graph = self.graphs.pop(key, None)
        if graph is not None and graph.fed_buffer is not self.engine.sampler.out:
            graph = None                 # the sampler has a new buffer: what was captured reads the old one
        if graph is None:
            if len(self.graphs) >= self.limit:
                self.graphs.pop(next(iter(self.graphs)))        # the least recently used
            graph = DecodeGraph(self.engine, *key)
        self.graphs[key] = graph
        graph.fill(entries, pasts)
        return graph.run()
