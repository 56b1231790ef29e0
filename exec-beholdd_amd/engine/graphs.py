"""Decode steps as HIP graphs.

A decode step launches a few hundred small kernels; replaying them as one captured graph takes
the host out of the loop.  A graph is captured for a given number of sequences, a given number of
tokens that each of them brings (one, unless `DecodeGraphs.rows_per_sequence` allows short steps
of several) and a given page-table width (the longest sequence's pages, rounded up to a bucket)
and replayed for every later step of that shape: the step's numbers (tokens, positions, slots,
page tables) live in one static device buffer that is refreshed with a single copy before each replay.

Only kernels go into a graph: no memset nodes, no library calls (torch only hands out the
temporaries, from the graph's private pool).  Parts whose `forward` reads the step's host-side
lists would bake one step's values into the graph, so a model is captured only if every part
declares `graph_safe = True`.
"""

from __future__ import annotations

import gc
import weakref

import torch

from .step import StepLayout, cache_for_runs


def _weakly(engine):
    return engine if isinstance(engine, weakref.ProxyTypes) else weakref.proxy(engine)


PAGE_BUCKET = 16      # page-table widths are rounded up to a multiple of this many pages


class DecodeGraph:
    def __init__(self, engine, n_seqs: int, table_width: int, rows: int = 1, pool=None):
        self.pool, self.rows = pool, rows
        # the engine owns its graphs; they point back weakly, so that an engine nobody holds any more is
        # freed at once and not by a later garbage collection
        self.engine, self.n_seqs, self.table_width = _weakly(engine), n_seqs, table_width
        cache = engine.cache
        self.layout = StepLayout(n_seqs * rows, n_seqs, n_seqs * rows, cache.kv_group_indices(), table_width)
        self.host = torch.zeros(self.layout.total, dtype=torch.int32).pin_memory()
        self.device = torch.zeros(self.layout.total, dtype=torch.int32, device=engine.device)
        self.host_views = self.layout.views(self.host.numpy())
        views = self.layout.views(self.device)
        self.tables = views["tables"]
        self.ctx = self.layout.context(
            views, engine.kernels, engine.dtype, engine.device, max_rows_per_seq=rows,
            max_position=min(table_width * cache.page_size, cache.max_position) - 1,
            fed_tokens=engine.sampler.device_tokens)
        self.want_rows = views["want_rows"]
        self.fed_buffer = engine.sampler.out       # the capture holds its address
        self.graph = None
        self.logits = None
        self.copied = None        # event: the last host-to-device copy of the step's numbers is done
        self.known = {}           # kv group -> per row (the page list the host table row was written from, how far)

    def fill(self, entries, pasts):
        """Write this step's numbers into the static buffer (one host-to-device copy)."""
        cache = self.engine.cache
        if self.copied is not None:
            self.copied.synchronize()     # the pinned buffer may not change under a copy in flight
        host = self.host_views
        self.layout.fill(host, [_every_row_wanted(e) for e in entries], pasts)
        slots = [e.slot for e in entries]
        for index in self.layout.kv_groups:
            table = host["tables"][index]
            group = cache.groups[index]
            known = self.known.setdefault(index, [(None, 0)] * self.n_seqs)
            for row, slot in enumerate(slots):
                pages = group.pages_of[slot]
                before, count = known[row]
                # a sequence's page list only grows while it lives (a window apart), so a row that was
                # written for this very list needs its new pages only
                if before is pages and count <= len(pages) and not group.need.window:
                    for j in range(count, len(pages)):
                        table[row, j] = pages[j]
                else:
                    cache.write_page_table(index, [slot], table[row:row + 1])
                known[row] = (pages, len(pages))
        self.device.copy_(self.host, non_blocking=True)
        self.copied = torch.cuda.Event()
        self.copied.record()

    def _forward(self):
        engine = self.engine
        return engine.model.forward(self.ctx, cache_for_runs(engine.model, engine.cache, self.tables), self.want_rows)

    def run(self):
        """This step's logits.  The first step of a shape runs kernel by kernel (which also loads every kernel
        before the capture) and is then captured without being run again: a part that keeps state advances it
        once per step, whether the step was launched or replayed.  Later steps replay the capture; their logits
        tensor is reused by the next replay."""
        if self.graph is None:
            logits = self._forward()
            torch.cuda.synchronize(self.engine.device)
            graph = torch.cuda.CUDAGraph()
            # No garbage collection while the stream is capturing: it could free another engine's graphs or
            # memory there, and the runtime refuses such calls during a capture (the process aborts).
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph, pool=self.pool):
                    self.logits = self._forward()
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
            return logits
        self.graph.replay()
        return self.logits


class _every_row_wanted:
    """An entry of a captured step as the layout sees it: the capture computes every row's logits, and the
    engine picks the wanted ones afterwards."""

    def __init__(self, entry):
        self.slot, self.tokens, self.fed_row, self.want = entry.slot, entry.tokens, entry.fed_row, tuple(range(len(entry.tokens)))


class DecodeGraphs:
    """The graphs of one engine, by (sequences, page-table width, tokens per sequence)."""

    def __init__(self, engine, limit: int = 48, rows_per_sequence: int = 1):
        self.engine, self.limit = _weakly(engine), max(int(limit), 1)
        # The most tokens per sequence of a step that is captured (every sequence of the step bringing as many).  The
        # generation loop decodes one token per sequence; a caller whose steps bring a few each may raise this.
        self.rows_per_sequence = max(int(rows_per_sequence), 1)
        self.graphs: dict = {}
        # One pool of device memory for all captures of the engine: only one of them runs at a time, on one
        # stream, so the temporaries of one step may stand where another's stood; what a capture returns (its
        # logits) stays its own for as long as the capture lives.
        self.pool = torch.cuda.graph_pool_handle()

    def usable(self, ctx_entries) -> bool:
        model = self.engine.model
        rows = len(ctx_entries[0].tokens)
        return (getattr(model, "graph_safe", False) and self.engine.device.type == "cuda"
                and 1 <= rows <= self.rows_per_sequence and (rows == 1 or rows <= getattr(model, "graph_safe_rows", 1))
                and all(len(e.tokens) == rows for e in ctx_entries)
                and (rows == 1 or all(e.fed_row is None for e in ctx_entries)))

    def step(self, entries, pasts, extras=None):
        cache = self.engine.cache
        rows = len(entries[0].tokens)
        pages = max(-(-(past + rows) // cache.page_size) for past in pasts)
        width = -(-pages // PAGE_BUCKET) * PAGE_BUCKET
        key = (len(entries), width, rows)
        graph = self.graphs.pop(key, None)
        if graph is not None and graph.fed_buffer is not self.engine.sampler.out:
            graph = None                 # the sampler has a new buffer: what was captured reads the old one
        if graph is None:
            if len(self.graphs) >= self.limit:
                self.graphs.pop(next(iter(self.graphs)))        # the least recently used
            graph = DecodeGraph(self.engine, *key, pool=self.pool)
        self.graphs[key] = graph
        graph.fill(entries, pasts)
        logits = graph.run()
        if extras is not None:
            extras.update(graph.ctx.extras)      # what the parts left when the step was launched and captured: every replay writes it again
        return logits
