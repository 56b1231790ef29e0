"""Grouped-query attention over the paged cache.

Formulas in the reference's order (crates/beholdd-model/src/qwen3moe/forward.rs:1086-1252):
q, k, v projections without bias; per-head RMSNorm of q and k with one [head_dim] weight each,
BEFORE the rotation (:1130-1156); split-half rotation of q and k at the absolute position
(:1161-1189); keys (normed, rotated) and raw values appended to the cache (:1196); for query
head h the kv head h // (heads / kv_heads) (crates/beholdd-backend/src/cpu.rs:806); scores
scaled by `scale`, causal by position, softmax in float32 (cpu.rs:810-833); output projection
added to the residual (:1236-1252).

Every size and constant is a constructor parameter; the q/k norm, the rotation and a window
are optional, so the same part serves other stacks.
"""

from __future__ import annotations

import math

from ..weights.binder import TensorSpec
from .base import MIXERS, CacheNeed
from .linear import Linear


class GQAAttention:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    prepares_next_norm = True      # the output projection can carry the norm that follows
    takes_prepared_input = True    # x goes to the q/k/v product untouched
    def __init__(self, hidden: int, n_heads: int, n_kv_heads: int, head_dim: int, prefix: str, *,
                 position_encoding=None, qk_norm_eps: float | None = None, scale: float | None = None,
                 window: int = 0):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads do not group evenly into {n_kv_heads} kv heads")
        self.hidden, self.n_heads, self.n_kv_heads, self.head_dim = hidden, n_heads, n_kv_heads, head_dim
        self.prefix = prefix
        self.position_encoding = position_encoding
        self.qk_norm_eps = qk_norm_eps
        # the reference computes the scale in float32: (head_dim as f32).sqrt().recip() (forward.rs:1192)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.window = int(window)
        q_width, kv_width = n_heads * head_dim, n_kv_heads * head_dim
        self.qkv = Linear(hidden, [q_width, kv_width, kv_width],
                          [prefix + "q_proj.weight", prefix + "k_proj.weight", prefix + "v_proj.weight"])
        self.out = Linear(q_width, hidden, prefix + "o_proj.weight")
        self.q_norm = self.k_norm = None

    @property
    def input_reader(self):
        return self.qkv.reader()    # x goes to that product and nowhere else

    def tensor_specs(self):
        specs = self.qkv.tensor_specs() + self.out.tensor_specs()
        if self.qk_norm_eps is not None:
            specs += [TensorSpec(self.prefix + "q_norm.weight", (self.head_dim,), "norm"),
                      TensorSpec(self.prefix + "k_norm.weight", (self.head_dim,), "norm")]
        return specs

    def load(self, get):
        self.qkv.load(get)
        self.out.load(get)
        if self.qk_norm_eps is not None:
            self.q_norm = get(self.prefix + "q_norm.weight")
            self.k_norm = get(self.prefix + "k_norm.weight")
            if self.q_norm.dtype != self.k_norm.dtype:
                self.q_norm, self.k_norm = self.q_norm.float(), self.k_norm.float()

    def prepare(self, kernels):
        self.qkv.prepare(kernels)
        self.out.prepare(kernels)

    def cache_need(self):
        return CacheNeed(kind="kv", kv_heads=self.n_kv_heads, head_dim=self.head_dim, window=self.window)

    def working_bytes(self, step) -> int:
        q_width = self.n_heads * self.head_dim
        total = self.qkv.working_bytes(step, step.rows)
        total += step.matrix(step.rows, q_width, reader=self.out.reader_for_plan(step.act_size))     # attended
        total += step.matrix(step.rows, q_width)                                                     # normed, rotated queries
        if step.sizes is not None:
            total += step.sizes.attention_working_bytes(step.rows, step.seqs, step.max_rows_per_seq, self.n_heads,
                                                        self.n_kv_heads, self.head_dim, step.max_position, step.act_size)
        return total + self.out.working_bytes(step, step.rows, accumulate=True, then_norm=True)

    def forward(self, ctx, x, hidden, cache, then_norm=None):
        k = ctx.kernels
        cos, sin = self.position_encoding.tables() if self.position_encoding is not None else (None, None)
        qkv = None
        # a step of many rows: the projection may stay the sums of K's parts, which the norm/rotation kernel adds up
        takes_sums = getattr(k, "qk_norm_rope_takes_sums", None)
        if not ctx.is_decode and takes_sums is not None and takes_sums(ctx.n_rows, self.head_dim, 2 * cos.shape[1] if cos is not None else 0):
            qkv = self.qkv.forward_bare(ctx, x)
        if qkv is None:
            qkv = self.qkv.forward(ctx, x)
        attended = ctx.new_activations(ctx.n_rows, self.n_heads * self.head_dim, reader=self.out.reader())
        # a decode step: norm, rotation, cache write and attention in one launch where the kernels offer it
        one_launch = getattr(k, "attention_decode_fused", None)
        if ctx.is_decode and one_launch is not None and one_launch(
                qkv, attended, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin, ctx.positions,
                cache.k_pages, cache.v_pages, cache.page_table, self.n_heads, self.n_kv_heads, self.head_dim,
                self.scale, self.window, cache.writes, ctx):
            return self.out.add_into(ctx, attended, hidden, then_norm)
        q = ctx.new_activations(ctx.n_rows, self.n_heads * self.head_dim)
        k.qk_norm_rope_cache(qkv, q, self.q_norm, self.k_norm, self.qk_norm_eps or 0.0, cos, sin,
                             ctx.positions, ctx.row_seq, cache.k_pages, cache.v_pages, cache.page_table,
                             self.n_heads, self.n_kv_heads, self.head_dim, cache.writes, ctx.max_position)
        k.attention(q, attended, cache.k_pages, cache.v_pages, cache.page_table, ctx.row_seq, ctx.positions,
                    self.n_heads, self.n_kv_heads, self.head_dim, self.scale, self.window, layout=ctx)
        return self.out.add_into(ctx, attended, hidden, then_norm)


@MIXERS.register("gqa_attention")
def _build_gqa_attention(config, layer_index, prefix, shared):
    return GQAAttention(config.hidden, config.n_heads, config.n_kv_heads, config.head_dim,
                        prefix + "self_attn.", position_encoding=shared["position_encoding"],
                        qk_norm_eps=config.rms_eps)
