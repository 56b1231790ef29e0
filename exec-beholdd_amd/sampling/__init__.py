"""Choosing the next token: greedy, or temperature sampling with optional top-k / top-p.

Greedy is the reference's rule: the largest logit, ties to the lowest id, and a non-finite
logit is an error (crates/beholdd-model/src/qwen3moe/forward.rs:1822-1842).  The reference
samples with nothing else (its server refuses a non-zero temperature,
crates/beholdd-server/src/lib.rs:329-335); temperature, top-k and top-p are this library's own.
The uniform number of a draw depends only on (seed, request index, step), never on the
batch a request happens to be in.
"""

from __future__ import annotations

import numbers
from dataclasses import dataclass

import torch

_MASK = (1 << 64) - 1
_MOST_TOP_K = (1 << 31) - 1     # the kernel takes it as a 32-bit integer; beyond the vocabulary it filters nothing


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0     # 0 = greedy
    top_k: int = 0               # 0 = off
    top_p: float = 1.0           # 1 = off
    seed: int = 0

    def __post_init__(self):
        for name in ("temperature", "top_p"):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, numbers.Real):
                raise ValueError(f"{name} is a number, got {value!r}")
        for name in ("top_k", "seed"):
            value = getattr(self, name)
            if isinstance(value, bool) or not isinstance(value, numbers.Integral):
                raise ValueError(f"{name} is an integer, got {value!r}")
        if not (0.0 <= self.temperature < float("inf")):
            raise ValueError(f"temperature must be finite and not negative, got {self.temperature}")
        if not (0 <= self.top_k <= _MOST_TOP_K):
            raise ValueError(f"top_k must be in 0 .. {_MOST_TOP_K} (0 = off), got {self.top_k}")
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


class Selection:
    """Tokens that the selection kernel has chosen, or is still choosing, for some rows.

    `result()` waits for them and returns them as a list (raising for a row whose logits were not
    finite).  Until then, and afterwards, the tokens also stand in the sampler's device buffer:
    element i at row `device_rows[i]`, where the next step can read them without the host
    (`StepEntry.fed_row`).  A selection is good until the sampler has made a few more."""

    def __init__(self, host, event, device_rows, requests, steps):
        self._host, self._event = host, event
        self.device_rows, self.requests, self.steps = list(device_rows), list(requests), list(steps)

    def __len__(self):
        return len(self.device_rows)

    def take(self, positions):
        """The selection restricted to some of its elements."""
        return Selection(self._host, self._event, [self.device_rows[i] for i in positions],
                         [self.requests[i] for i in positions], [self.steps[i] for i in positions])

    def token_at(self, device_row: int) -> int:
        """The token at a row of the device buffer, waited for; no check of the row's flag."""
        if self._event is not None:
            self._event.synchronize()
        return int(self._host[0, device_row])

    def result(self) -> list:
        if self._event is not None:
            self._event.synchronize()
        tokens = []
        for row, request, step in zip(self.device_rows, self.requests, self.steps):
            if int(self._host[1, row]):
                raise SamplingError(f"request {request}, step {step}: a logit is not finite")
            tokens.append(int(self._host[0, row]))
        return tokens


class Sampler:
    """Runs the selection kernel on rows of float32 logits."""

    RING = 4      # host buffers in turn: a selection stays readable while the next few are made

    def __init__(self, kernels, device, capacity: int = 64):
        self.kernels, self.device = kernels, torch.device(device)
        self._allocate(int(capacity))

    def _allocate(self, capacity):
        # row 0: tokens, row 1: the not-finite flags.  Captured graphs read row 0; the engine sizes the sampler
        # for its largest batch, so this buffer is replaced only when a caller selects for more rows than the
        # engine has slots.  The new buffer then takes over what the old one held (a selection whose tokens
        # the next step reads on the device stays good), and captures that read the old one are made again.
        before = getattr(self, "out", None)
        self.capacity = capacity
        self.out = torch.zeros((2, capacity), dtype=torch.int32, device=self.device)
        if before is not None:
            self.out[:, :before.shape[1]].copy_(before)
        pin = self.device.type == "cuda"
        self._hosts = [torch.zeros((2, capacity), dtype=torch.int32, pin_memory=pin) for _ in range(self.RING)]
        self._turn = 0
        # A draw's numbers (temperature, top-p, the uniform number; top-k) go to the device from pinned memory without
        # a wait: a copy from ordinary memory would hold the host until the stream has run everything before it, and
        # the loop that works a step ahead of the device would lose its lead at every step.
        self._draw_hosts = [(torch.zeros((3, capacity), dtype=torch.float32, pin_memory=pin),
                             torch.zeros(capacity, dtype=torch.int32, pin_memory=pin)) for _ in range(self.RING)]
        self._draw_sent = [None] * self.RING      # the event behind each pair's last copy
        self._draw_turn = 0
        self._draw = (torch.zeros((3, capacity), dtype=torch.float32, device=self.device),
                      torch.zeros(capacity, dtype=torch.int32, device=self.device))

    @property
    def device_tokens(self) -> torch.Tensor:
        return self.out[0]

    def select_async(self, logits: torch.Tensor, params: list, requests: list, steps: list) -> Selection:
        """Start choosing one token per row of `logits` (row i belongs to request `requests[i]` at step
        `steps[i]`) and bring them to the host without waiting for either."""
        n_rows = logits.shape[0]
        if not (len(params) == len(requests) == len(steps) == n_rows):
            raise ValueError("one sampling parameter set, request index and step per row")
        if n_rows > self.capacity:
            self._allocate(n_rows)
        tokens, bad = self.out[0, :n_rows], self.out[1, :n_rows]
        if all(p.greedy for p in params):
            self.kernels.sample(logits, tokens, bad)
        else:
            turn = self._draw_turn
            self._draw_turn = (turn + 1) % self.RING
            if self._draw_sent[turn] is not None:
                self._draw_sent[turn].synchronize()      # (made RING selections ago: long done)
            numbers, counts = self._draw_hosts[turn]
            numbers[:, :n_rows] = torch.tensor([[p.temperature for p in params], [p.top_p for p in params],
                                                [uniform(p.seed, r, s) for p, r, s in zip(params, requests, steps)]],
                                               dtype=torch.float32)
            counts[:n_rows] = torch.tensor([p.top_k for p in params], dtype=torch.int32)
            on_device, counts_on_device = self._draw
            if self.device.type == "cuda":
                on_device.copy_(numbers, non_blocking=True)
                counts_on_device.copy_(counts, non_blocking=True)
                self._draw_sent[turn] = torch.cuda.Event()
                self._draw_sent[turn].record()
            else:
                on_device.copy_(numbers)
                counts_on_device.copy_(counts)
            # a filter that no row uses is left out: the kernels then spread the rows' work over the chip where they can
            # (a draw from the whole distribution over chunks of the row, a top-k through the chunks' candidates)
            any_k = any(p.top_k > 0 for p in params)
            any_p = any(p.top_p < 1.0 for p in params)
            self.kernels.sample(logits, tokens, bad, temperature=on_device[0, :n_rows],
                                top_k=counts_on_device[:n_rows] if any_k else None,
                                top_p=on_device[1, :n_rows] if any_p else None, uniform=on_device[2, :n_rows])
        host = self._hosts[self._turn]
        self._turn = (self._turn + 1) % self.RING
        event = None
        if self.device.type == "cuda":
            host.copy_(self.out, non_blocking=True)
            event = torch.cuda.Event()
            event.record()
        else:
            host.copy_(self.out)
        return Selection(host, event, range(n_rows), requests, steps)

    def select(self, logits: torch.Tensor, params: list, requests: list, steps: list) -> list:
        """One token per row of `logits`, on the host."""
        return self.select_async(logits, params, requests, steps).result()
