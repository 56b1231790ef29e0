"""The byte plan of an engine: everything it will hold on the device, itemised before anything is allocated.

The reference itemises its decode buffers and the largest staging buffer and enforces its limits before any
I/O (crates/beholdd-model/src/qwen3moe.rs:661-758 `greedy_decode_buffer_bytes`,
crates/beholdd-model/src/qwen3moe/recorded_attention.rs:244-299 `largest_staging_bytes`, :344-365).  Here the
items are: the weights as they are kept (rows padded to the kernels' blocks), the largest transient while they
are loaded and regrouped, tables the parts build (rotation), the cache, the working memory of the largest
step the engine will run (`max_rows_per_step` rows; the parts say what they allocate, `StepSize`), the logits
and the step's numbers, the sampler's buffers and the captured decode steps (one pool that all captures of an
engine share, and each capture's logits and numbers).
"""

from __future__ import annotations

from dataclasses import dataclass, field

from ..parts.base import StepSize

UNIT = 512      # torch's allocator hands out device memory in multiples of this many bytes


def _rounded(n_bytes: int) -> int:
    return -(-int(n_bytes) // UNIT) * UNIT


@dataclass
class MemoryPlan:
    items: list = field(default_factory=list)        # (label, bytes)
    unaccounted: list = field(default_factory=list)  # names of parts that do not say what they allocate

    def add(self, label: str, n_bytes: int) -> None:
        self.items.append((label, int(n_bytes)))

    @property
    def total_bytes(self) -> int:
        return sum(n_bytes for _, n_bytes in self.items)

    def bytes_of(self, label: str) -> int:
        return sum(n_bytes for name, n_bytes in self.items if name == label)

    def describe(self) -> str:
        lines = [f"{label}: {n_bytes} bytes" for label, n_bytes in self.items]
        if self.unaccounted:
            lines.append(f"not counted (parts that do not say what a step of theirs allocates): {', '.join(self.unaccounted)}")
        lines.append(f"total: {self.total_bytes} bytes")
        return "\n".join(lines)


def step_size(model, rows: int, seqs: int, act_size: int, max_position: int, sizes, max_rows_per_seq=None) -> StepSize:
    seqs = max(1, min(int(seqs), int(rows)))
    longest = int(max_rows_per_seq) if max_rows_per_seq else min(int(rows), int(max_position))
    return StepSize(rows=int(rows), seqs=seqs, wanted=seqs, act_size=act_size, max_position=max(int(max_position) - 1, 0),
                    max_rows_per_seq=max(longest, 1), sizes=sizes)


def step_numbers_bytes(rows: int, seqs: int, kv_groups: int, table_width: int) -> int:
    """The step's integers on the device (`StepLayout.total` int32)."""
    return _rounded(4 * (4 * rows + 3 * seqs + 1 + seqs + kv_groups * seqs * table_width))


def weights_as_kept(model, act_size: int, sizes) -> tuple:
    """(bytes of the weights as the engine keeps them, bytes of the largest transient while loading): a matrix
    that the kernel library regroups has its rows padded to whole blocks, and while it is stacked from its
    checkpoint tensors or regrouped a second copy of it exists."""
    kept = transient = 0
    linears = [linear for part in model.parts() for linear in _linears(part)]
    in_linears = set()
    for linear in linears:
        if getattr(linear, "shared", False):
            continue
        rows, cols = linear.out_features, linear.in_features
        packs = bool(getattr(linear, "packs", lambda size: False)(act_size))
        size = sizes.packed_bytes(rows, cols, act_size) if (packs and sizes is not None) else _rounded(rows * cols * act_size)
        kept += size
        transient = max(transient, size if (packs or len(linear.names) > 1) else 0)
        in_linears.update(linear.names)
    for spec in model.tensor_specs():
        if spec.name not in in_linears:
            count = 1
            for axis in spec.shape:
                count *= int(axis)
            kept += _rounded(count * (4 if spec.kind == "norm" and act_size == 4 else act_size))
    return kept, transient


def _linears(part, depth: int = 0) -> list:
    from ..parts.linear import Linear
    if isinstance(part, Linear):
        return [part]
    found = []
    if depth < 4 and hasattr(part, "__dict__"):
        for value in vars(part).values():
            if isinstance(value, (list, tuple)):
                for item in value:
                    found += _linears(item, depth + 1)
            elif hasattr(value, "__dict__") and not isinstance(value, type):
                found += _linears(value, depth + 1)
    return found


def tables_bytes(model) -> int:
    """Rotation tables and their like: what shared parts build once per model."""
    total = 0
    for part in getattr(model, "shared_parts", ()):
        half = getattr(part, "rotary_dim", 0) // 2
        total += 2 * _rounded(getattr(part, "max_position", 0) * half * 4)
    return total


def plan_memory(model, weight_bytes: int, cache_plan, act_size: int, sizes, max_rows_per_step: int, max_slots: int,
                max_position: int, page_size: int, graph_limit: int, graphs: bool = True, graph_rows: int = 1) -> MemoryPlan:
    plan = MemoryPlan()
    kept, transient = weights_as_kept(model, act_size, sizes)
    plan.add("weights", int(weight_bytes))
    plan.add("weights' padding to the kernels' blocks and the allocator's units", max(kept - int(weight_bytes), 0))
    plan.add("largest transient while the weights are loaded and regrouped", transient)
    plan.add("tables the parts build", tables_bytes(model))
    plan.add("cache", cache_plan.total_bytes)
    kv_groups = sum(1 for g in cache_plan.groups if g.need.kind == "kv")
    state_bytes = sum(g.state_bytes for g in cache_plan.groups)
    plan.add("state rows kept during a step, to put back if it fails", state_bytes)
    if hasattr(model, "working_bytes"):
        rows = int(max_rows_per_step)
        width = -(-max_position // page_size)
        big = step_size(model, rows, min(max_slots, rows), act_size, max_position, sizes)
        plan.add(f"working memory of a step of {rows} rows", model.working_bytes(big)
                 + step_numbers_bytes(rows, big.seqs, kv_groups, width))
        plan.unaccounted = model.unaccounted_parts() if hasattr(model, "unaccounted_parts") else []
        if graphs and getattr(model, "graph_safe", False):
            most = max_slots * graph_rows       # every sequence of a captured step brings the same one to graph_rows tokens
            small = step_size(model, most, max_slots, act_size, max_position, sizes, max_rows_per_seq=graph_rows)
            pool = model.working_bytes(small)
            each = _rounded(most * model.vocab * 4) + step_numbers_bytes(most, max_slots, kv_groups, width + 16)
            plan.add(f"captured decode steps (one pool; up to {graph_limit} captures' logits and numbers)",
                     pool + graph_limit * each)
    else:
        plan.unaccounted = [type(model).__name__]
    vocab = getattr(model, "vocab", 0)
    sample = sizes.sample_working_bytes(max_slots, vocab) if sizes is not None else 0
    plan.add("sampler", 2 * _rounded(2 * max_slots * 4) + sample + 8 * UNIT)
    return plan
