"""Trace replay: given token ids go through the engine's step function; logits come out.

The reference's counterpart is its capture-and-compare tooling: `decode --logits-out`
(crates/beholdd-model/examples/decode.rs:78-82, :343-345) records logits and
tools/compare_logits.py compares two captures.  This program instead takes the schedule from
its input, so the same requests can be replayed whole, token by token, or in batches of
unequal lengths, and every cut must give the same logits.  It has no forward pass, cache or
loader of its own: it calls `Engine.step`.
"""

from __future__ import annotations

import json
import os
import sys

import numpy as np

from .engine import Engine, MemoryBudgetError
from ..cache.sequence_cache import CacheError
from .step import StepEntry, StepError


class TraceError(ValueError):
    pass


def _arguments(argv: list) -> dict:
    wanted = {"--model": None, "--dtype": None, "--out": None, "--max-tokens": None}
    optional = {"--capture": None}
    wanted.update(optional)
    index = 0
    while index < len(argv):
        flag = argv[index]
        if flag not in wanted:
            raise TraceError(f"unexpected argument {flag!r}")
        if wanted[flag] is not None:
            raise TraceError(f"{flag} may be given once")
        if index + 1 >= len(argv):
            raise TraceError(f"{flag} needs a value")
        wanted[flag] = argv[index + 1]
        index += 2
    missing = [flag for flag, value in wanted.items() if value is None and flag not in optional]
    if missing:
        raise TraceError("missing " + ", ".join(missing))
    try:
        wanted["--max-tokens"] = int(wanted["--max-tokens"])
    except ValueError:
        raise TraceError("--max-tokens must be an integer") from None
    if wanted["--max-tokens"] <= 0:
        raise TraceError("--max-tokens must be positive")
    if wanted["--dtype"] not in ("bfloat16", "float32"):
        raise TraceError("--dtype must be bfloat16 or float32")
    return wanted


class _NoCapture:
    _rows = ()

    def feed(self, name, tokens):
        return 0

    def add(self, step, places, logits):
        pass

    def close(self):
        pass

    abandon = close


class Replayer:
    """Maps request ids to cache slots and runs steps as they are read.

    The output folder gets `<step>.f32` (the bare rows) and nothing else.  With `capture` (a path; `--capture` on
    the command line) the replay also writes one capture file (version 2 of engine/artifact.py) when the input
    ends: every request's tokens, and for every logits row its request, position and step, so that two replays can
    be compared without knowing how either was cut (`beholdd compare`).  A run owns its output folder: a
    `<step>.f32` of an earlier run is replaced; within a run a step number may occur once; a capture is never
    written over another file."""

    def __init__(self, engine, out_dir: str, capture: str | None = None, notes: dict | None = None):
        from .artifact import PositionCaptureWriter

        self.engine, self.out_dir = engine, out_dir
        self.slot_of: dict = {}
        self.steps_seen: set = set()
        os.makedirs(out_dir, exist_ok=True)
        self.capture = PositionCaptureWriter(capture, engine.model.vocab, notes) if capture else _NoCapture()
        self.fed: dict = {}         # request id -> tokens fed so far (kept for the capture after the request ends)
        self.generation: dict = {}  # request id -> how many requests of that id have ended before

    def _name(self, request_id) -> str:
        """The capture's name of a request: its id, with a suffix when the id is used again after it ended."""
        again = self.generation.get(request_id, 0)
        return str(request_id) if again == 0 else f"{request_id}#{again}"

    def run_step(self, record: dict) -> None:
        if not isinstance(record, dict) or "step" not in record or "entries" not in record:
            raise TraceError("a step is an object with 'step' and 'entries'")
        step = record["step"]
        if isinstance(step, bool) or not isinstance(step, int) or step < 0:
            raise TraceError(f"'step' must be a non-negative integer, got {step!r}")
        if step in self.steps_seen:
            raise TraceError(f"step {step} occurs twice")
        if not isinstance(record["entries"], list) or not isinstance(record.get("end", []), list):
            raise TraceError(f"step {step}: 'entries' and 'end' are lists")
        seen = set()
        for index, item in enumerate(record["entries"]):      # refuse a malformed entry before anything is started
            if not isinstance(item, dict) or "id" not in item or "tokens" not in item:
                raise TraceError(f"step {step}: entry {index} is an object with 'id' and 'tokens' (and maybe 'want')")
            if not isinstance(item["id"], (str, int)) or isinstance(item["id"], bool):
                raise TraceError(f"step {step}: entry {index}: 'id' is a string or an integer, got {item['id']!r}")
            if not isinstance(item["tokens"], list) or not isinstance(item.get("want", []), list):
                raise TraceError(f"step {step}: entry {index} (request {item['id']!r}): 'tokens' and 'want' are lists")
            if item["id"] in seen:
                raise TraceError(f"step {step}: request {item['id']!r} occurs twice")
            seen.add(item["id"])
        ended = set()
        for name in record.get("end", []):      # and an end that cannot be, before anything has run
            if not isinstance(name, (str, int)) or isinstance(name, bool):
                raise TraceError(f"step {step}: 'end' lists request ids (strings or integers), got {name!r}")
            if name in ended:
                raise TraceError(f"step {step}: request {name!r} ends twice")
            if name not in self.slot_of and name not in seen:
                raise TraceError(f"step {step}: request {name!r} ends but was never started")
            ended.add(name)
        entries, fresh, places = [], [], []
        for item in record["entries"]:
            name = item["id"]
            if name not in self.slot_of:
                self.slot_of[name] = self.engine.alloc_slot()
                fresh.append(name)
            entries.append(StepEntry(self.slot_of[name], list(item["tokens"]), list(item.get("want", []))))
        try:
            logits = self.engine.step(entries) if entries else None
        except BaseException:
            for name in fresh:          # a refused step leaves no trace of the requests it would have started
                self.engine.free_slot(self.slot_of.pop(name))
            raise
        self.steps_seen.add(step)
        for item, entry in zip(record["entries"], entries):
            first = self.capture.feed(self._name(item["id"]), entry.tokens)
            places.extend((self._name(item["id"]), first + int(place)) for place in entry.want)
        if logits is not None:
            data = np.ascontiguousarray(logits.float().cpu().numpy().astype("<f4", copy=False))
            path = os.path.join(self.out_dir, f"{step}.f32")
            with open(path + ".tmp", "wb") as handle:
                handle.write(data.tobytes())
            os.replace(path + ".tmp", path)
            self.capture.add(step, places, data)
        for name in record.get("end", []):
            self.engine.free_slot(self.slot_of.pop(name))
            self.generation[name] = self.generation.get(name, 0) + 1

    def close(self) -> None:
        """The input has ended: complete the capture (no rows were wanted: no capture)."""
        if self.capture._rows:
            self.capture.close()
        else:
            self.capture.abandon()


def main(argv=None, stdin=None, stdout=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    stdin, stdout = stdin or sys.stdin, stdout or sys.stdout
    try:
        args = _arguments(argv)
    except TraceError as error:
        print(f"trace_run: {error}\nusage: trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N "
              "[--capture FILE]", file=sys.stderr)
        return 2
    from ..kernels import KernelError
    from ..kernels.build import BuildError
    try:
        engine = Engine(args["--model"], dtype=args["--dtype"], max_tokens=args["--max-tokens"])
        replayer = Replayer(engine, args["--out"], args["--capture"],
                            notes={"dtype": args["--dtype"], "max_tokens": args["--max-tokens"], "tool": "trace_run"})
    except (ValueError, OSError, CacheError, MemoryBudgetError, KernelError, BuildError) as error:
        print(f"trace_run: {error}", file=sys.stderr)      # no such model, a tensor that does not fit, no GPU: its reason
        return 1
    try:
        for line in stdin:
            line = line.strip()
            if not line:
                continue
            try:
                record = json.loads(line)
            except json.JSONDecodeError as error:
                print(f"trace_run: input line is not JSON: {error}", file=sys.stderr)
                return 1
            try:
                replayer.run_step(record)
            except (TraceError, StepError, CacheError) as error:      # a refused step: its reason, not a traceback
                print(f"trace_run: {error}", file=sys.stderr)
                return 1
            print(f"done {record['step']}", file=stdout, flush=True)
        replayer.close()
        return 0
    finally:
        replayer.capture.abandon()      # a run that ends early leaves no half-written capture (no-op once closed)
