"""Choosing the next token: greedy, or temperature sampling with optional top-k / top-p.

Greedy is the reference's rule: the largest logit, ties to the lowest id, and a non-finite
logit is an error (crates/beholdd-model/src/qwen3moe/forward.rs:1822-1842).  The reference
samples with nothing else (its server refuses a non-zero temperature,
crates/beholdd-server/src/lib.rs:329-335); temperature, top-k and top-p are this library's own.
The uniform number of a draw depends only on (seed, request index, step), never on the
batch a request happens to be in.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

_MASK = (1 << 64) - 1


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0     # 0 = greedy
    top_k: int = 0               # 0 = off
    top_p: float = 1.0           # 1 = off
    seed: int = 0

    def __post_init__(self):
        if not (self.temperature >= 0.0):
            raise ValueError(f"temperature must not be negative, got {self.temperature}")
        if self.top_k < 0:
            raise ValueError(f"top_k must not be negative, got {self.top_k}")
        if not (0.0 < self.top_p <= 1.0):
            raise ValueError(f"top_p must be in (0, 1], got {self.top_p}")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0


def _mix(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


def uniform(seed: int, request: int, step: int) -> float:
    """A number in [0, 1) with 24 random bits, a pure function of its three arguments."""
    value = _mix(_mix(_mix(seed & _MASK) ^ (request & _MASK)) ^ (step & _MASK))
    return (value >> 40) / float(1 << 24)


class SamplingError(RuntimeError):
    pass


class Sampler:
    """Runs the selection kernel on rows of float32 logits."""

    def __init__(self, kernels, device):
        self.kernels, self.device = kernels, torch.device(device)

    def select(self, logits: torch.Tensor, params: list, requests: list, steps: list) -> list:
        """One token per row of `logits`; row i belongs to request `requests[i]` at step `steps[i]`."""
        n_rows = logits.shape[0]
        if not (len(params) == len(requests) == len(steps) == n_rows):
            raise ValueError("one sampling parameter set, request index and step per row")
        both = torch.empty((2, n_rows), dtype=torch.int32, device=self.device)   # one copy brings both back
        tokens, bad = both[0], both[1]
        if all(p.greedy for p in params):
            self.kernels.sample(logits, tokens, bad)
        else:
            host = torch.tensor([[p.temperature, p.top_p, uniform(p.seed, r, s)]
                                 for p, r, s in zip(params, requests, steps)], dtype=torch.float32)
            columns = host.t().contiguous().to(self.device)
            top_k = torch.tensor([p.top_k for p in params], dtype=torch.int32).to(self.device)
            self.kernels.sample(logits, tokens, bad, temperature=columns[0], top_k=top_k, top_p=columns[1],
                                uniform=columns[2])
        result = both.cpu()
        for row in range(n_rows):
            if int(result[1, row]):
                raise SamplingError(f"request {requests[row]}, step {steps[row]}: a logit is not finite")
        return [int(t) for t in result[0]]
