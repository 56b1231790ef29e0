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

from .engine import Engine
from .step import StepEntry


class TraceError(ValueError):
    pass


def _arguments(argv: list) -> dict:
    wanted = {"--model": None, "--dtype": None, "--out": None, "--max-tokens": None}
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
    missing = [flag for flag, value in wanted.items() if value is None]
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


class Replayer:
    """Maps request ids to cache slots and runs steps as they are read."""

    def __init__(self, engine, out_dir: str):
        self.engine, self.out_dir = engine, out_dir
        self.slot_of: dict = {}
        os.makedirs(out_dir, exist_ok=True)

    def run_step(self, record: dict) -> None:
        if not isinstance(record, dict) or "step" not in record or "entries" not in record:
            raise TraceError("a step is an object with 'step' and 'entries'")
        step = record["step"]
        entries, fresh = [], []
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
        if logits is not None:
            data = logits.float().cpu().numpy().astype("<f4", copy=False)
            path = os.path.join(self.out_dir, f"{step}.f32")
            with open(path + ".tmp", "wb") as handle:
                handle.write(np.ascontiguousarray(data).tobytes())
            os.replace(path + ".tmp", path)
        for name in record.get("end", []):
            if name not in self.slot_of:
                raise TraceError(f"step {step}: request {name!r} ends but was never started")
            self.engine.free_slot(self.slot_of.pop(name))


def main(argv=None, stdin=None, stdout=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    stdin, stdout = stdin or sys.stdin, stdout or sys.stdout
    try:
        args = _arguments(argv)
    except TraceError as error:
        print(f"trace_run: {error}\nusage: trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N",
              file=sys.stderr)
        return 2
    engine = Engine(args["--model"], dtype=args["--dtype"], max_tokens=args["--max-tokens"])
    replayer = Replayer(engine, args["--out"])
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        try:
            record = json.loads(line)
        except json.JSONDecodeError as error:
            print(f"trace_run: input line is not JSON: {error}", file=sys.stderr)
            return 1
        replayer.run_step(record)
        print(f"done {record['step']}", file=stdout, flush=True)
    return 0
