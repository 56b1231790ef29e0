"""Dense SwiGLU feed-forward: out = Wd (silu(Wg x) * (Wu x)), added to the residual.

crates/beholdd-model/src/qwen3moe/forward.rs:1270-1298 with silu(x) = x / (1 + exp(-x)) and no
clamp (crates/beholdd-kernel/src/vecops.rs:91-110, limit 0 at forward.rs:1288).  The gate and
up matrices are stacked so that one product computes both.
"""

from __future__ import annotations

from .base import FEED_FORWARDS
from .linear import Linear


class SwiGLU:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    prepares_next_norm = True      # the down projection can carry the norm that follows
    takes_prepared_input = True    # x goes to the gate/up product untouched
    def __init__(self, hidden: int, intermediate: int, prefix: str):
        self.hidden, self.intermediate = hidden, intermediate
        self.gate_up = Linear(hidden, [intermediate, intermediate],
                              [prefix + "gate_proj.weight", prefix + "up_proj.weight"])
        self.down = Linear(intermediate, hidden, prefix + "down_proj.weight")

    @property
    def input_reader(self):
        return self.gate_up.reader(swiglu=True)    # x goes to that product and nowhere else

    def tensor_specs(self):
        return self.gate_up.tensor_specs() + self.down.tensor_specs()

    def load(self, get):
        self.gate_up.load(get)
        self.down.load(get)

    def prepare(self, kernels):
        self.gate_up.prepare(kernels)
        self.down.prepare(kernels)

    def working_bytes(self, step) -> int:
        activated = step.matrix(step.rows, self.intermediate, reader=self.down.reader_for_plan(step.act_size))
        return (activated + self.gate_up.working_bytes(step, step.rows, accumulate=True, swiglu=True)
                + self.down.working_bytes(step, step.rows, accumulate=True, then_norm=True))

    def forward(self, ctx, x, hidden, then_norm=None):
        activated = ctx.new_activations(x.shape[0], self.intermediate, reader=self.down.reader())
        ctx.kernels.gemm_swiglu(x, self.gate_up.weight, activated)     # both products and the gate in one pass
        return self.down.add_into(ctx, activated, hidden, then_norm)


@FEED_FORWARDS.register("swiglu")
def _build_swiglu(config, layer_index, prefix, shared):
    return SwiGLU(config.hidden, config.intermediate, prefix + "mlp.")
