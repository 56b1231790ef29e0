"""RMSNorm: y = (x * inv) * w with inv = 1/sqrt(mean(x^2) + eps).

crates/beholdd-kernel/src/vecops.rs:54-64: the weight is a plain multiplier (no 1 + w) and the
order of the two multiplications is (x * inv) * w.  The statistic is computed in float32 on
the float32 residual; only the result is rounded to the activation type.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import NORMS, NormRequest


class RMSNorm:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    def __init__(self, width: int, eps: float, name: str):
        if not (eps > 0.0):
            raise ValueError(f"RMSNorm epsilon must be positive, got {eps}")
        self.width, self.eps, self.name = int(width), float(eps), name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self):
        return [TensorSpec(self.name, (self.width,), "norm")]

    def load(self, get):
        self.weight = get(self.name)

    serves_reader = True   # forward and request take the product that reads the output

    def forward(self, ctx, hidden, rows=None, reader=None):
        n = hidden.shape[0] if rows is None else rows.shape[0]
        out = ctx.new_activations(n, self.width, reader=reader)
        ctx.kernels.rmsnorm(hidden, self.weight, self.eps, out, rows=rows)
        return out

    def working_bytes(self, step, rows: int | None = None, reader=None) -> int:
        return step.matrix(step.rows if rows is None else rows, self.width, reader=reader)

    def request(self, reader=None):
        """This norm as the product that completes its input may prepare it."""
        return NormRequest(self.weight, self.eps, reader)


@NORMS.register("rmsnorm")
def _build_rmsnorm(config, width, name, shared):
    return RMSNorm(width, config.rms_eps, name)
