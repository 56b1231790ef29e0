"""What a part is, what it sees of a step, and the registries that configurations choose from.

A model is put together from parts: a *mixer* (attention here), a *feed-forward*, a *norm*,
a *position encoding*, arranged by a *block*.  Each part takes its sizes and constants as
constructor parameters and does not know which model it is in.  A configuration names, layer
by layer, which registered part to build; the builder functions registered here turn the
configuration into constructor parameters.

Interfaces
----------
Every part:
    tensor_specs() -> list[TensorSpec]     the checkpoint tensors it needs, by full name
    load(get)                              take them: get(name) -> device tensor
Norm:
    forward(ctx, hidden_f32, rows=None) -> activations [n, width] in ctx.act_dtype
Position encoding:
    tables() -> (cos, sin) float32 [positions, rotary/2], or (None, None)
Mixer:
    cache_need() -> CacheNeed | None       what it keeps per sequence between steps
    forward(ctx, x, hidden, cache)         adds its output into `hidden` (float32, the residual)
Feed-forward:
    forward(ctx, x, hidden)                adds its output into `hidden`
Block:
    mixer, feed_forward attributes; forward(ctx, hidden, cache)
A norm may ride on the products around it (optional, one flag per role):
    norm.request() -> NormRequest          what the product that completes the norm's input needs
    producer (mixer or feed-forward) with `prepares_next_norm = True`:
        forward(..., then_norm=NormRequest) returns what its last product prepared (whatever
        `kernels.gemm(..., then_norm=)` returned: the next part's input in the kernel library's own
        form, or None when the product could not carry the norm)
    consumer (mixer or feed-forward) with `takes_prepared_input = True`: its `x` may be that
        prepared form; it hands `x` to the kernel library's products untouched.
The block joins a producer and a consumer this way only when all three offer it, and runs the norm
as a step of its own otherwise.
A matrix that one product alone reads may be kept the way that product reads it fastest (optional):
    consumer with `input_reader` (a ProductReader: the product its `x` goes to, and nowhere else): its `x` may
        then be in the kernel library's own form for that product; it hands `x` to that product untouched.
    norm with `serves_reader = True`: forward(..., reader=) and request(reader) take that ProductReader.
    Inside a part, `ctx.new_activations(rows, width, reader=linear.reader())` asks for such a matrix between two
    of its own kernel calls.  Parts that say nothing get and give plain matrices.
A mixer with a "state" cache need updates its rows of `cache.state` in place while it runs.  The cache keeps
what the step's sequences held before the step and puts it back if the step fails, so a mixer needs no
second bank; and the engine runs a part's forward exactly once per step, whether the step is launched kernel
by kernel or replayed from a capture, so a state advances once per token.
Every part may say what its forward allocates: working_bytes(step: StepSize) -> int, from sizes alone; the
engine's byte plan adds them up before anything is allocated and names the parts that do not say.
A part may declare `graph_safe = True`: its forward uses only the device tensors of the step
context (never the host_* lists, never a host-side decision that changes from step to step).
Decode steps of a model whose parts all say so are captured and replayed as HIP graphs.  That speaks of steps
of one token per sequence; a part whose forward keeps to the device tensors for steps of several tokens per sequence too
says `graph_safe_rows = n` (up to n tokens) or `None` (any number), and an engine that is told to capture such steps
captures them only for models whose parts all allow it (`graph_rows_allowed`).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import torch


def graph_rows_allowed(parts) -> int:
    """Up to how many tokens per sequence a captured step of these parts may bring (0: none may be captured)."""
    most = 1 << 30
    for part in parts:
        if not getattr(part, "graph_safe", False):
            return 0
        rows = getattr(part, "graph_safe_rows", 1)
        if rows is not None:
            most = min(most, int(rows))
    return most


# ---- what a mixer keeps between steps ------------------------------------------------------

@dataclass(frozen=True)
class CacheNeed:
    """Storage one layer needs for each sequence.

    kind "kv":    keys and values of `kv_heads` heads of `head_dim` for every position, or for
                  the last `window` positions only (window 0 = all); paged.
    kind "state": one tensor of `state_shape` and `state_dtype` per sequence, of fixed size,
                  zero when a sequence starts.
    Layers whose needs are equal share one storage group.
    """
    kind: str
    kv_heads: int = 0
    head_dim: int = 0
    window: int = 0
    state_shape: tuple = ()
    state_dtype: torch.dtype = torch.float32

    def __post_init__(self):
        if self.kind not in ("kv", "state"):
            raise ValueError(f"cache need kind must be 'kv' or 'state', got {self.kind!r}")
        if self.kind == "kv" and (self.kv_heads <= 0 or self.head_dim <= 0 or self.window < 0):
            raise ValueError("a kv cache need has positive head count and head size and a window >= 0")
        if self.kind == "state" and not self.state_shape:
            raise ValueError("a state cache need has a shape")


# ---- what a part sees of one step ------------------------------------------------------------

@dataclass
class StepContext:
    """One step: `n_rows` tokens of `n_seqs` sequences, flattened sequence after sequence.

    Device tensors (int32): tokens [T], positions [T] (absolute position of each row),
    row_seq [T] (index of the row's sequence in this batch), seq_start [B+1] (first row of each
    sequence), seq_slot [B] (cache slot of each sequence), seq_past [B] (tokens the cache held
    before this step).  The `host_*` lists carry the same numbers for parts that decide on the
    host.  `is_decode` says that every sequence brings exactly one token.
    `extras` is the step's second way out, beside the logits: a part may leave there what a caller wants to
    inspect (a routed feed-forward its routing, a mixer its state's norm), under a key of its own; the step
    function hands the dictionary to a caller who asks for it (`Engine.step(entries, extras={})`).  In a
    captured step the tensors left there are written again by every replay.
    """
    kernels: object
    act_dtype: torch.dtype
    device: torch.device
    n_rows: int
    n_seqs: int
    tokens: torch.Tensor
    positions: torch.Tensor
    row_seq: torch.Tensor
    seq_start: torch.Tensor
    seq_slot: torch.Tensor
    seq_past: torch.Tensor
    host_seq_start: list
    host_seq_slot: list
    host_seq_past: list
    is_decode: bool
    max_position: int                      # largest absolute position in this step
    max_rows_per_seq: int = 1              # most tokens any one sequence brings
    token_src: torch.Tensor | None = None  # int32 [T]: >= 0 where a row's token is fed_tokens[token_src[row]]
    fed_tokens: torch.Tensor | None = None # int32: tokens chosen on the device that the host has not read yet
    extras: dict = field(default_factory=dict)

    def new_activations(self, *shape, reader=None):
        """An empty matrix of the activation type.  `reader` (a ProductReader) names the product that reads it
        next and nothing else does: the kernel library may then hand out the matrix in the form that product
        reads fastest, which only its own kernels fill and read."""
        if reader is not None and len(shape) == 2 and hasattr(self.kernels, "new_rows"):
            return self.kernels.new_rows(shape[0], shape[1], self.act_dtype, reader.outputs, reader.swiglu,
                                         getattr(reader, "packed", True))
        return torch.empty(shape, dtype=self.act_dtype, device=self.device)

    def new_f32(self, *shape) -> torch.Tensor:
        return torch.empty(shape, dtype=torch.float32, device=self.device)


@dataclass
class StepSize:
    """The sizes of a step, for the byte plan: a part's optional `working_bytes(step)` answers from them how many
    bytes its `forward` allocates in such a step (its output included), before anything is allocated.  `sizes`
    is the kernel library's own account of what its calls allocate (`kernels.KernelSizes`), or None for a
    stepper without one."""
    rows: int
    seqs: int
    wanted: int
    act_size: int
    max_position: int
    max_rows_per_seq: int
    sizes: object | None = None

    def matrix(self, rows: int, width: int, element_size: int | None = None, reader=None) -> int:
        """Bytes of a matrix as `StepContext.new_activations` / `new_f32` hand it out."""
        size = self.act_size if element_size is None else element_size
        if reader is not None and self.sizes is not None and size == self.act_size:
            return self.sizes.rows_bytes(rows, width, size, reader.outputs, reader.swiglu, getattr(reader, "packed", True))
        return -(-int(rows) * int(width) * size // 512) * 512

    def product(self, rows: int, outputs: int, inputs: int, packed: bool = True, swiglu: bool = False,
                then_norm: bool = False) -> int:
        """Bytes that a matrix product of the kernel library allocates beside its output."""
        if self.sizes is None:
            return 0
        return self.sizes.gemm_working_bytes(rows, outputs, inputs, self.act_size, packed, swiglu, then_norm)


@dataclass
class ProductReader:
    """The matrix product that reads an activation matrix next: `outputs` columns of result, through the
    gated activation or not (then its weight has twice as many rows); `packed`: its weight is in the kernel
    library's own form (`Linear.prepare`), not a plain matrix."""
    outputs: int
    swiglu: bool = False
    packed: bool = True


@dataclass
class NormRequest:
    """An RMSNorm (weight [width], eps) offered to the product that completes its input; `reader`: the
    product that reads the norm's output, if it is the only one that does."""
    weight: torch.Tensor
    eps: float
    reader: ProductReader | None = None


@dataclass
class LayerCache:
    """The storage of one cache entry as handed to a mixer for one step.

    kv need:    k_pages [pages, kv_heads, page_size, head_dim], v_pages [pages, kv_heads, head_dim,
                page_size], to be written and read through the kernel library only (it orders the
                elements of a head inside a page as its attention kernels want them); page_table
                int32 [n_seqs, width] for the sequences of this step, in batch order.
    state need: state [max_slots, *state_shape]; index it with ctx.seq_slot.
    `writes` is False when the schedule lets this layer read another layer's entry.
    """
    need: CacheNeed
    writes: bool = True
    k_pages: torch.Tensor | None = None
    v_pages: torch.Tensor | None = None
    page_table: torch.Tensor | None = None
    state: torch.Tensor | None = None


# ---- registries ---------------------------------------------------------------------------------

class Registry:
    """Name -> builder.  A builder is `build(config, layer_index, prefix, shared) -> part`."""

    def __init__(self, what: str):
        self.what = what
        self._items: dict = {}

    def register(self, name: str, builder=None):
        if builder is None:                 # decorator form
            return lambda fn: self.register(name, fn)
        if name in self._items:
            raise ValueError(f"{self.what} {name!r} is already registered")
        self._items[name] = builder
        return builder

    def unregister(self, name: str):
        self._items.pop(name, None)

    def get(self, name: str):
        try:
            return self._items[name]
        except KeyError:
            raise KeyError(f"no {self.what} named {name!r}; registered: {sorted(self._items)}") from None

    def names(self) -> list[str]:
        return sorted(self._items)

    def __contains__(self, name):
        return name in self._items


MIXERS = Registry("mixer")
FEED_FORWARDS = Registry("feed-forward")
NORMS = Registry("norm")
POSITION_ENCODINGS = Registry("position encoding")
BLOCKS = Registry("block")
