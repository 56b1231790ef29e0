"""The engine: a loaded model, its cache, the step function and generation above it.

Construction follows the reference's load (crates/beholdd-runtime/src/native.rs:181-337):
architecture tag -> model class, typed configuration, every tensor bound by name with its
shape checked, byte accounting before allocation.  The Python entry point mirrors the
reference's embedded API (crates/beholdd-embed/src/lib.rs:51-105): construct once,
`generate(...)`, with token ids in place of text.
"""

from __future__ import annotations

import numbers

import torch

from ..cache import SequenceCache
from ..config.base import read_config_json
from ..registry import resolve_architecture
from ..sampling import Sampler, SamplingParams
from ..weights.binder import bind
from ..weights.random_init import random_tensor_on_device
from . import generation
from .graphs import DecodeGraphs
from .memory import plan_memory
from .step import StepEntry, StepError, StepStaging, build_step, cache_for_runs, check_entries

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError(f"engine dtype must be bfloat16 or float32, got {name}")
        return name
    try:
        return _DTYPES[str(name).lower()]
    except KeyError:
        raise ValueError(f"engine dtype must be bfloat16 or float32, got {name!r}") from None


class MemoryBudgetError(RuntimeError):
    """Weights and cache together would take more device memory than the caller allows; nothing was loaded."""


GRAPH_LIMIT = 48      # captured decode steps an engine keeps (least recently used goes first)


class Engine:
    """`Engine(model_dir, dtype, max_tokens)`; then `step(...)` or `generate(...)`.

    `max_rows_per_step` bounds the tokens one step may bring (default: as many as the cache holds); the
    generation loop feeds prompts beyond it in portions, and `step` refuses more.  It sizes the step's working
    memory in the byte plan (`plan`, `memory_plan()`): weights as kept, the transient while they are loaded,
    the cache, the largest step's temporaries and logits, the sampler and the captured decode steps.
    `memory_limit_bytes` bounds that plan's total and is checked from the checkpoint's header and the sizes
    alone, before a tensor is read or the cache allocated (the reference enforces its limits before any I/O,
    crates/beholdd-model/src/qwen3moe/recorded_attention.rs:344-365)."""

    def __init__(self, model_dir: str | None = None, dtype="bfloat16", max_tokens: int = 4096,
                 max_slots: int | None = None, device="cuda:0", kernels=None, model=None,
                 memory_limit_bytes: int | None = None, use_graphs: bool = True,
                 max_rows_per_step: int | None = None, graph_limit: int = GRAPH_LIMIT, graph_rows_per_sequence: int = 1):
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        if kernels is None:
            from ..kernels import HipKernels   # fails loudly without a GPU or the library
            kernels = HipKernels(self.device)
        self.kernels = kernels
        for name, value, least, optional in (("max_rows_per_step", max_rows_per_step, 1, True), ("graph_limit", graph_limit, 0, False),
                                             ("graph_rows_per_sequence", graph_rows_per_sequence, 1, False),
                                             ("memory_limit_bytes", memory_limit_bytes, 0, True)):
            if value is None and optional:
                continue
            if isinstance(value, bool) or not isinstance(value, numbers.Integral) or value < least:
                raise ValueError(f"{name} is an integer of at least {least}{' or None' if optional else ''}, got {value!r}")
        with_graphs = bool(use_graphs and self.device.type == "cuda")

        def make_cache(built):
            return SequenceCache(built.entry_needs, max_tokens, self.dtype, self.device, kernels.page_size,
                                 max_slots=max_slots, max_position=built.max_position)

        def within_budget(weight_bytes, cache):
            capacity = cache.n_pages * cache.page_size
            # never below one token for every sequence, so that a decode step of a full batch fits
            self.max_rows_per_step = min(max(int(max_rows_per_step), cache.max_slots), capacity) if max_rows_per_step else capacity
            self.plan = plan_memory(model, weight_bytes, cache.plan(), 2 if self.dtype == torch.bfloat16 else 4,
                                    kernels if hasattr(kernels, "gemm_working_bytes") else None, self.max_rows_per_step,
                                    cache.max_slots, cache.max_position, cache.page_size, graph_limit, with_graphs,
                                    max(int(graph_rows_per_sequence), 1))
            if memory_limit_bytes is not None and self.plan.total_bytes > memory_limit_bytes:
                raise MemoryBudgetError(f"the engine needs {self.plan.total_bytes} bytes, the limit is "
                                        f"{memory_limit_bytes}:\n{self.plan.describe()}")

        if model is None:
            if model_dir is None:
                raise ValueError("give a model folder or a built model")
            model, weights = open_model(model_dir, self.dtype, self.device)
            try:
                self.weight_bytes = weights.planned_bytes(model.tensor_specs())
                self.cache = make_cache(model)
                within_budget(self.weight_bytes, self.cache)
                model.load(weights, self.device)
            finally:
                weights.reader.close()
        else:
            self.weight_bytes = sum(t.numel() * t.element_size() for t in _model_tensors(model))
            self.cache = make_cache(model)
            within_budget(self.weight_bytes, self.cache)
        self.model = model
        self.config = model.config
        if hasattr(model, "prepare"):
            model.prepare(kernels)
        self.cache_plan = self.cache.allocate()
        self.sampler = Sampler(kernels, self.device, capacity=self.cache.max_slots)
        self._last_selection = None
        self._staging = StepStaging() if self.device.type == "cuda" else None
        self.graphs = DecodeGraphs(self, graph_limit, graph_rows_per_sequence) if with_graphs else None

    # ---- what the generation loop needs of a stepper ----
    @property
    def page_size(self) -> int:
        return self.cache.page_size

    @property
    def capacity_pages(self) -> int:
        return self.cache.n_pages

    @property
    def max_slots(self) -> int:
        return self.cache.max_slots

    @property
    def max_position(self) -> int:
        return self.cache.max_position

    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def select(self, logits, params, requests, steps):
        return self.select_async(logits, params, requests, steps).result()

    def select_async(self, logits, params, requests, steps):
        """Start the selection and return at once: a `Selection` whose `result()` waits.  The step after
        it may take its tokens on the device (`StepEntry.fed_row`) while the host has not read them."""
        self._last_selection = self.sampler.select_async(logits, params, requests, steps)
        return self._last_selection

    # ---- the step function ----
    def step(self, entries: list, extras: dict | None = None):
        """Run the given tokens of each entry's sequence from the cache; return float32 logits
        [wanted, vocab] in the order of the entries and of their `want` lists (None if nothing is
        wanted).  `extras`, a dictionary of the caller's, receives what parts left in the step's
        `StepContext.extras` (one row per token of the step, in the order of the entries).
        On an error no sequence's length changes.  The logits of a decode step stand in memory
        that a later decode step may write again: copy what has to outlive the next step."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        if self.graphs is not None and entries and self.graphs.usable(entries):
            return self._graph_step(entries, extras)
        if any(e.fed_row is not None for e in entries):
            # only the captured decode step reads tokens on the device; here the host waits for them
            if self._last_selection is None:
                raise ValueError("an entry takes its token from a selection, but nothing was selected yet")
            entries = [e if e.fed_row is None
                       else StepEntry(e.slot, [self._last_selection.token_at(e.fed_row)], e.want) for e in entries]
        check_entries(entries, self.cache, self.model.vocab)
        requests = [(e.slot, len(e.tokens)) for e in entries]
        n_rows = sum(n for _, n in requests)
        if n_rows > self.max_rows_per_step:
            raise StepError(f"the step brings {n_rows} tokens, this engine takes {self.max_rows_per_step} a step "
                            "(max_rows_per_step): feed the prompts in portions")
        self.cache.reserve(requests)
        try:
            ctx, want_rows, tables = build_step(self.kernels, self.dtype, self.device, self.cache, entries, self._staging)
            logits = self.model.forward(ctx, cache_for_runs(self.model, self.cache, tables), want_rows)
        except BaseException:
            self.cache.rollback(requests)
            raise
        self.cache.commit(requests)
        if extras is not None:
            extras.update(ctx.extras)
        return logits

    def _graph_step(self, entries: list, extras: dict | None = None):
        """A decode step (every sequence bringing the same few tokens, as a rule one) replayed from a captured HIP graph."""
        check_entries(entries, self.cache, self.model.vocab)
        rows = len(entries[0].tokens)
        requests = [(e.slot, rows) for e in entries]
        self.cache.reserve(requests)
        try:
            pasts = [self.cache.length(e.slot) for e in entries]
            logits = self.graphs.step(entries, pasts, extras)
        except BaseException:
            self.cache.rollback(requests)
            raise
        self.cache.commit(requests)
        wanted = [index * rows + place for index, e in enumerate(entries) for place in e.want]
        if not wanted:
            return None
        if wanted == list(range(len(entries) * rows)):
            return logits
        return logits[torch.tensor(wanted, device=self.device)]

    # ---- generation ----
    def generate(self, prompts: list, max_new_tokens=16, temperature: float = 0.0, top_k: int = 0,
                 top_p: float = 1.0, seed: int = 0, stop_token_ids=(), on_token=None, batch_size=None,
                 control=None, on_logits=None) -> list:
        sampling = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, seed=seed)
        return generation.generate(self, prompts, max_new_tokens, sampling, stop_token_ids, on_token,
                                   batch_size, control, on_logits)

    def memory_plan(self) -> str:
        return f"{self.plan.describe()}\n{self.cache_plan.describe()}"


def _model_tensors(model):
    seen, out = set(), []

    def visit(obj, depth=0):
        if isinstance(obj, torch.Tensor):
            if obj.data_ptr() not in seen:
                seen.add(obj.data_ptr())
                out.append(obj)
        elif isinstance(obj, (list, tuple)):
            for item in obj:
                visit(item, depth + 1)
        elif hasattr(obj, "__dict__") and depth < 6 and not isinstance(obj, type):
            for value in vars(obj).values():
                visit(value, depth + 1)

    for part in model.parts():
        visit(part)
    return out


def open_model(model_dir: str, dtype, device):
    """config.json -> architecture -> model (no tensors yet), and the checkpoint's tensors bound to it by name
    with nothing read yet.  The caller loads (`model.load(weights, device)`) and closes `weights.reader`."""
    dtype = parse_dtype(dtype)
    data, path = read_config_json(model_dir)
    entry = resolve_architecture(data, path)
    config = entry.config_class.from_dict(data, path)
    model = entry.build(config)
    return model, bind(model.tensor_specs(), model_dir, dtype, device)


def load_model(model_dir: str, dtype, device):
    """config.json -> architecture -> model; model.safetensors -> its tensors, bound by name."""
    model, weights = open_model(model_dir, dtype, device)
    try:
        model.load(weights, device)
    finally:
        weights.reader.close()
    return model


def random_model_on_device(config_dict: dict, seed: int, dtype, device):
    """A model with seeded random weights drawn on the device (nothing is written to disk)."""
    dtype = parse_dtype(dtype)
    entry = resolve_architecture(config_dict)
    config = entry.config_class.from_dict(config_dict)
    model = entry.build(config)
    specs = {spec.name: spec for spec in model.tensor_specs()}
    model.load(lambda name: random_tensor_on_device(specs[name], seed, device, dtype), device)
    return model
