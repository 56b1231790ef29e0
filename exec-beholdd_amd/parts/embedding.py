"""Token embedding and the language-model head.

Embedding: hidden[t] = E[token[t]] widened to float32, no scaling
(crates/beholdd-model/src/qwen3moe/forward.rs:954-972).  Head: logits = W_out x on the rows that
are asked for; a tied head is the embedding matrix itself, not a copy
(crates/beholdd-model/src/qwen3moe.rs:948-955).
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .linear import Linear


class Embedding:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    def __init__(self, vocab: int, width: int, name: str):
        self.vocab, self.width, self.name = vocab, width, name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.vocab, self.width), "linear")]

    def load(self, get):
        self.weight = get(self.name)

    def working_bytes(self, step) -> int:
        return step.matrix(step.rows, self.width, 4)      # the float32 residual, which lives as long as the step

    def forward(self, ctx):
        hidden = ctx.new_f32(ctx.n_rows, self.width)
        if ctx.token_src is not None:
            ctx.kernels.embed(ctx.tokens, self.weight, hidden, token_src=ctx.token_src, fed_tokens=ctx.fed_tokens)
        else:
            ctx.kernels.embed(ctx.tokens, self.weight, hidden)
        return hidden


class LMHead:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    def __init__(self, vocab: int, width: int, name: str | None, tied_to: Embedding | None = None):
        if (name is None) == (tied_to is None):
            raise ValueError("a head has either its own tensor or an embedding it is tied to")
        self.vocab, self.width, self.tied_to = vocab, width, tied_to
        self.linear = Linear(width, vocab, name or tied_to.name)

    def tensor_specs(self):
        return [] if self.tied_to is not None else self.linear.tensor_specs()

    def load(self, get):
        if self.tied_to is not None:
            self.linear.use(self.tied_to.weight)
        else:
            self.linear.load(get)

    def prepare(self, kernels):
        self.linear.prepare(kernels)        # a tied head keeps the embedding's own matrix

    @property
    def input_reader(self):
        return self.linear.reader()    # x goes to that product and nowhere else

    def working_bytes(self, step) -> int:
        return self.linear.working_bytes(step, step.wanted, out_size=4)

    def forward(self, ctx, x):
        """x [n, width] -> float32 logits [n, vocab]."""
        return self.linear.forward(ctx, x, out_dtype=torch.float32)
