"""A bias-free linear map y = W x with W stored [out, in], as checkpoints store it.

The reference applies every weight this way, without transposing or permuting
(crates/beholdd-backend/src/lib.rs:178, crates/beholdd-backend/src/cpu.rs:206-211).  Several
checkpoint tensors with the same input may be stacked into one matrix at load time, so that
one product serves them all; each output row is computed exactly as it would be alone.
"""

from __future__ import annotations

import torch

from ..weights.binder import TensorSpec
from .base import ProductReader


class Linear:
    graph_safe = True      # forward reads only the step's device tensors
    graph_safe_rows = None # ... whatever the number of tokens a sequence brings
    def __init__(self, in_features: int, out_features, names):
        """`names` and `out_features` are one name and size, or equal-length lists to stack."""
        self.in_features = int(in_features)
        self.names = [names] if isinstance(names, str) else list(names)
        self.splits = [int(out_features)] if isinstance(out_features, int) else [int(o) for o in out_features]
        if len(self.names) != len(self.splits):
            raise ValueError("one output size per stacked tensor")
        self.out_features = sum(self.splits)
        self.weight = None          # a tensor, or the kernel library's packed form of it
        self.shared = False

    def tensor_specs(self):
        return [TensorSpec(name, (rows, self.in_features), "linear") for name, rows in zip(self.names, self.splits)]

    def load(self, get):
        pieces = [get(name) for name in self.names]
        if len(pieces) == 1:
            self.weight = pieces[0]
        else:
            dtype = pieces[0].dtype
            if any(p.dtype != dtype for p in pieces):
                pieces = [p.to(torch.float32) for p in pieces]   # mixed storage: keep the wider one
            self.weight = torch.cat(pieces, dim=0).contiguous()

    def use(self, weight: torch.Tensor):
        """Share another part's matrix (a tied head)."""
        if tuple(weight.shape) != (self.out_features, self.in_features):
            raise ValueError(f"shared weight has shape {tuple(weight.shape)}, expected "
                             f"{(self.out_features, self.in_features)}")
        self.weight = weight
        self.shared = True

    def reader(self, swiglu: bool = False) -> ProductReader:
        """This map as the only reader of an activation matrix (`swiglu`: its rows are gate rows, then up rows)."""
        return ProductReader(self.out_features // 2 if swiglu else self.out_features, swiglu,
                             packed=self.weight is not None and not isinstance(self.weight, torch.Tensor))

    def packs(self, act_size: int) -> bool:
        """Whether `prepare` regroups this matrix in an engine of that element size."""
        return not self.shared and act_size == 2 and self.in_features % 64 == 0

    def reader_for_plan(self, act_size: int, swiglu: bool = False) -> ProductReader:
        """`reader()` as it will be once the weights are loaded and prepared."""
        return ProductReader(self.out_features // 2 if swiglu else self.out_features, swiglu, packed=self.packs(act_size))

    def working_bytes(self, step, rows: int, out_size: int | None = None, accumulate: bool = False,
                      then_norm: bool = False, swiglu: bool = False) -> int:
        """Bytes one product of `rows` rows allocates: its output unless it adds into one, and what the
        kernel library allocates on the way."""
        outputs = self.out_features // 2 if swiglu else self.out_features
        total = 0 if accumulate else step.matrix(rows, outputs, out_size)
        return total + step.product(rows, outputs, self.in_features, self.packs(step.act_size), swiglu, then_norm)

    def prepare(self, kernels):
        """Let the kernel library regroup the matrix into the layout it reads fastest."""
        if not self.shared and hasattr(kernels, "pack_weight"):
            self.weight = kernels.pack_weight(self.weight)

    def forward(self, ctx, x, out=None, accumulate=False, out_dtype=None):
        """x [n, in] -> out [n, out]; with accumulate the product is added into `out`."""
        if out is None:
            out = torch.empty((x.shape[0], self.out_features), dtype=out_dtype or ctx.act_dtype, device=x.device)
        ctx.kernels.gemm(x, self.weight, out, accumulate=accumulate)
        return out

    def forward_bare(self, ctx, x):
        """W x as the kernel library's unfinished form of it (the sums of the parts that K was cut into), for a
        consumer that says it takes that form; None where the library has no such form for these operands or
        does not cut this product (then call `forward`)."""
        bare = getattr(ctx.kernels, "gemm_bare", None)
        return bare(x, self.weight) if bare is not None else None

    def add_into(self, ctx, x, residual, then_norm=None):
        """residual += W x.  With `then_norm` (a NormRequest for the norm that reads the residual next)
        returns what the product prepared of that norm's output, or None."""
        if then_norm is None:
            ctx.kernels.gemm(x, self.weight, residual, accumulate=True)
            return None
        return ctx.kernels.gemm(x, self.weight, residual, accumulate=True, then_norm=then_norm)
