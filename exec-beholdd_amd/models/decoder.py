"""A decoder as data: embedding, a list of blocks, the order in which they run, final norm, head.

The configuration supplies, layer by layer, the names of the parts (`layer_kinds()`) and the
order of execution (`schedule()`): a list of (layer index, cache entry index).  A layer may be
named twice (its weights run twice, each run with a cache entry of its own), and an entry may
be shared: the first run that names an entry writes it, later runs read it.
The whole-model order follows the reference: embed, every layer, then final norm and head on
the rows that are asked for (crates/beholdd-model/src/qwen3moe/forward.rs:811-915, :1416-1455).
"""

from __future__ import annotations

from ..parts.base import BLOCKS, NORMS, POSITION_ENCODINGS, graph_rows_allowed
from ..parts.embedding import Embedding, LMHead


class DecoderModel:
    def __init__(self, config, embedding, blocks, schedule, final_norm, head, shared_parts=()):
        self.config = config
        self.embedding, self.blocks, self.final_norm, self.head = embedding, list(blocks), final_norm, head
        self.shared_parts = list(shared_parts)
        self.schedule = [(int(layer), int(entry)) for layer, entry in schedule]
        for layer, entry in self.schedule:
            if not 0 <= layer < len(self.blocks):
                raise ValueError(f"the schedule names layer {layer}, the model has {len(self.blocks)}")
            if entry < 0:
                raise ValueError("cache entry indices are not negative")
        # entry -> need, and which scheduled run owns (writes) each entry
        self.entry_needs: dict = {}
        self.run_writes: list = []
        for layer, entry in self.schedule:
            need = self.blocks[layer].cache_need()
            if need is None:
                self.run_writes.append(False)
                continue
            if entry in self.entry_needs:
                if self.entry_needs[entry] != need:
                    raise ValueError(f"cache entry {entry} is shared by layers with different needs")
                self.run_writes.append(False)
            else:
                self.entry_needs[entry] = need
                self.run_writes.append(True)

    @property
    def vocab(self) -> int:
        return self.embedding.vocab

    @property
    def max_position(self) -> int:
        return self.config.max_position

    def parts(self):
        return [self.embedding, *self.shared_parts, *self.blocks, self.final_norm, self.head]

    @property
    def graph_safe(self):
        """True when a decode step of this model may be captured as a HIP graph: every part's
        forward depends on the step's device tensors only."""
        return all(getattr(part, "graph_safe", False)
                   for part in (self.embedding, *self.blocks, self.final_norm, self.head))

    @property
    def graph_safe_rows(self) -> int:
        """Up to how many tokens per sequence a captured step may bring (every sequence the same number)."""
        return graph_rows_allowed((self.embedding, *self.blocks, self.final_norm, self.head))

    def tensor_specs(self):
        return [spec for part in self.parts() for spec in part.tensor_specs()]

    def load(self, get, device):
        for part in self.parts():
            part.load(get)
        for part in self.shared_parts:
            if hasattr(part, "build_tables"):
                part.build_tables(device)

    def prepare(self, kernels):
        """After loading: parts may have the kernel library regroup their weights."""
        for part in self.parts():
            if hasattr(part, "prepare"):
                part.prepare(kernels)

    def working_bytes(self, step) -> int:
        """Bytes a step of these sizes allocates at its peak: the residual, the widest layer (a layer's
        temporaries are freed before the next one runs; what a block prepares for the next is counted with
        the block that made it), the final norm on the wanted rows and the logits."""
        total = self.embedding.working_bytes(step) if hasattr(self.embedding, "working_bytes") else 0
        widest = max([block.working_bytes(step) for block in self.blocks if hasattr(block, "working_bytes")], default=0)
        last = 0
        if hasattr(self.final_norm, "working_bytes"):
            last += self.final_norm.working_bytes(step, rows=step.wanted)
        if hasattr(self.head, "working_bytes"):
            last += self.head.working_bytes(step)
        return total + widest + last

    def unaccounted_parts(self) -> list:
        """Names of parts that do not say what their forward allocates (the byte plan lists them)."""
        names = [type(part).__name__ for part in (self.embedding, self.final_norm, self.head) if not hasattr(part, "working_bytes")]
        for block in self.blocks:
            names += block.unaccounted_parts() if hasattr(block, "unaccounted_parts") else [type(block).__name__]
        return sorted(set(names))

    def forward(self, ctx, cache_for_run, want_rows):
        """Run one step.  `cache_for_run(i)` gives the LayerCache of the i-th scheduled run (or
        None); `want_rows` (int32 device tensor, may be empty) lists the rows whose logits are
        returned as float32 [len(want_rows), vocab]."""
        hidden = self.embedding.forward(ctx)
        prepared = None      # the next block's first norm, when the block before could prepare it
        for run, (layer, _entry) in enumerate(self.schedule):
            following = self.blocks[self.schedule[run + 1][0]] if run + 1 < len(self.schedule) else None
            prepared = self.blocks[layer].forward(ctx, hidden, cache_for_run(run), prepared, following)
        if want_rows is None or want_rows.numel() == 0:
            return None
        reader = getattr(self.head, "input_reader", None) if getattr(self.final_norm, "serves_reader", False) else None
        normed = (self.final_norm.forward(ctx, hidden, rows=want_rows, reader=reader) if reader is not None
                  else self.final_norm.forward(ctx, hidden, rows=want_rows))
        return self.head.forward(ctx, normed)


def build_decoder(config, position_encoding="rope", layer_prefix: str = "model.layers.{}.",
                  embedding_name: str = "model.embed_tokens.weight", final_norm_name: str = "model.norm.weight",
                  head_name: str = "lm_head.weight", final_norm_kind: str = "rmsnorm",
                  make_embedding=None, make_head=None) -> DecoderModel:
    """Put a decoder together from the registered parts that `config` names.

    `position_encoding` is the registered name of the one encoding that all layers share, or a dictionary
    label -> registered name when layers differ: part builders find them in `shared["position_encodings"][label]`
    (and the one labelled "default", or the first, in `shared["position_encoding"]`).  `make_embedding(config)` and
    `make_head(config, embedding)` replace the plain embedding and head (a scaled embedding, a head that caps
    its logits); each returns a part with the interface of `parts.embedding`'s."""
    shared = {}
    labelled = position_encoding if isinstance(position_encoding, dict) else {"default": position_encoding}
    encodings = {label: POSITION_ENCODINGS.get(name)(config, shared) for label, name in labelled.items()}
    shared["position_encodings"] = encodings
    shared["position_encoding"] = encodings.get("default", next(iter(encodings.values())))
    embedding = make_embedding(config) if make_embedding else Embedding(config.vocab, config.hidden, embedding_name)
    blocks = []
    for index, kinds in enumerate(config.layer_kinds()):
        blocks.append(BLOCKS.get(kinds.block)(config, index, layer_prefix.format(index), kinds, shared))
    final_norm = NORMS.get(final_norm_kind)(config, config.hidden, final_norm_name, shared)
    if make_head:
        head = make_head(config, embedding)
    elif getattr(config, "tie_word_embeddings", False):
        head = LMHead(config.vocab, config.hidden, None, tied_to=embedding)
    else:
        head = LMHead(config.vocab, config.hidden, head_name)
    return DecoderModel(config, embedding, blocks, config.schedule(), final_norm, head,
                        shared_parts=list(encodings.values()))
