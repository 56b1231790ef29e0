"""Command line: `beholdd generate`, `beholdd random-model`, `beholdd plan`.

In the manner of the reference's command lines: flags are parsed by hand, every flag may be
given once, a flag's value may not look like another flag, and an unknown argument is an error
(crates/beholdd-cli/src/lib.rs:136-190, :288-304).  `generate` stands where the reference has
its `decode` example (crates/beholdd-model/examples/decode.rs:45-161): `--logits-out`,
`--step-timing-out`, `--memory-budget-bytes` and `--plan-only` keep their names and meanings;
the prompt is token ids, since text and tokenizers are outside this library.  Its report
follows the example's lines (:359-386): prompt ids, generated ids, every step's token and
logit, seconds per generated token.
"""

from __future__ import annotations

import json
import sys
import time

USAGE = """usage:
  beholdd generate --model DIR [--dtype bfloat16|float32] --prompt-ids 1,2,3 [--prompt-ids 4,5 ...]
                   [--prompt-ids-file FILE] [--max-new-tokens N] [--temperature X] [--top-k K] [--top-p P]
                   [--seed N] [--stop-token-ids a,b] [--max-tokens N] [--slots N] [--batch-size N]
                   [--max-rows-per-step N] [--logits-out PATH] [--step-timing-out PATH] [--memory-budget-bytes N] [--plan-only]
  beholdd random-model --config FILE --out DIR [--seed N] [--dtype bfloat16|float32]
  beholdd compare REFERENCE CANDIDATE [--tolerance X]
  beholdd architectures"""


class UsageError(ValueError):
    pass


def _parse_flags(args: list, valued: set, switches: set, repeatable: set = frozenset()) -> dict:
    found: dict = {}
    index = 0
    while index < len(args):
        flag = args[index]
        if flag in switches:
            if flag in found:
                raise UsageError(f"{flag} may be given once")
            found[flag] = True
            index += 1
            continue
        if flag not in valued:
            raise UsageError(f"unexpected argument {flag!r}")
        if index + 1 >= len(args) or args[index + 1].startswith("--"):
            raise UsageError(f"{flag} needs a value")
        value = args[index + 1]
        if flag in repeatable:
            found.setdefault(flag, []).append(value)
        elif flag in found:
            raise UsageError(f"{flag} may be given once")
        else:
            found[flag] = value
        index += 2
    return found


def _ids(text: str, flag: str) -> list:
    try:
        ids = [int(part) for part in text.replace(" ", "").split(",") if part != ""]
    except ValueError:
        raise UsageError(f"{flag}: {text!r} is not a comma-separated list of token ids") from None
    if any(i < 0 for i in ids):
        raise UsageError(f"{flag}: token ids are not negative")
    return ids


def _number(flags: dict, flag: str, default, kind=int):
    if flag not in flags:
        return default
    try:
        return kind(flags[flag])
    except ValueError:
        raise UsageError(f"{flag}: {flags[flag]!r} is not a valid {kind.__name__}") from None


def _generate(args: list, out) -> int:
    import os

    flags = _parse_flags(
        args,
        valued={"--model", "--dtype", "--prompt-ids", "--prompt-ids-file", "--max-new-tokens", "--temperature",
                "--top-k", "--top-p", "--seed", "--stop-token-ids", "--max-tokens", "--slots", "--batch-size",
                "--logits-out", "--step-timing-out", "--memory-budget-bytes", "--max-rows-per-step"},
        switches={"--plan-only"}, repeatable={"--prompt-ids"})
    if "--model" not in flags:
        raise UsageError("--model DIR is required")
    prompts = [_ids(text, "--prompt-ids") for text in flags.get("--prompt-ids", [])]
    if "--prompt-ids-file" in flags:
        with open(flags["--prompt-ids-file"], "r", encoding="utf-8") as handle:
            for line in handle:
                if line.strip():
                    prompts.append(_ids(line.strip(), "--prompt-ids-file"))
    if not prompts or any(len(p) == 0 for p in prompts):
        raise UsageError("give at least one non-empty prompt with --prompt-ids or --prompt-ids-file")
    max_new = _number(flags, "--max-new-tokens", 16)
    temperature = _number(flags, "--temperature", 0.0, float)
    top_k = _number(flags, "--top-k", 0)
    top_p = _number(flags, "--top-p", 1.0, float)
    seed = _number(flags, "--seed", 0)
    stops = _ids(flags["--stop-token-ids"], "--stop-token-ids") if "--stop-token-ids" in flags else None
    from .kernels.build import source_page_size

    page = source_page_size()
    default_tokens = sum(-(-(len(p) + max_new) // page) * page for p in prompts)
    max_tokens = _number(flags, "--max-tokens", default_tokens)
    slots = _number(flags, "--slots", None)
    batch_size = _number(flags, "--batch-size", None)
    budget = _number(flags, "--memory-budget-bytes", None)
    step_rows = _number(flags, "--max-rows-per-step", None)
    if step_rows is not None and step_rows <= 0:
        raise UsageError("--max-rows-per-step is positive")
    for path_flag in ("--logits-out", "--step-timing-out"):
        if path_flag in flags and os.path.lexists(flags[path_flag]):
            raise UsageError(f"{path_flag}: {flags[path_flag]} exists and is never overwritten")

    from .config.base import read_config_json
    from .registry import resolve_architecture

    data, path = read_config_json(flags["--model"])
    entry = resolve_architecture(data, path)
    config = entry.config_class.from_dict(data, path)
    dtype = flags.get("--dtype", "bfloat16")

    if "--plan-only" in flags:
        import torch

        from .cache import SequenceCache
        from .engine import open_model, parse_dtype
        from .engine.engine import GRAPH_LIMIT
        from .engine.memory import plan_memory
        from .kernels import KernelSizes

        model, weights = open_model(flags["--model"], dtype, "cpu")      # the header only: no tensor is read
        try:
            weight_bytes = weights.planned_bytes(model.tensor_specs())
        finally:
            weights.reader.close()
        cache = SequenceCache(model.entry_needs, max_tokens, parse_dtype(dtype), "cpu", page, max_slots=slots,
                              max_position=model.max_position)
        capacity = cache.n_pages * cache.page_size
        # the kernel library's own account of what its calls allocate: host code, no GPU is touched
        plan = plan_memory(model, weight_bytes, cache.plan(), 2 if parse_dtype(dtype) == torch.bfloat16 else 4,
                           KernelSizes(), min(step_rows or capacity, capacity), cache.max_slots, cache.max_position,
                           page, GRAPH_LIMIT)
        total = plan.total_bytes
        print(plan.describe() + (f" (budget {budget}: {'fits' if total <= budget else 'does not fit'})"
                                 if budget is not None else ""), file=out)
        print(cache.plan().describe(), file=out)
        return 0 if budget is None or total <= budget else 1

    from .engine import Engine
    from .engine.artifact import write_logits_artifact

    engine = Engine(flags["--model"], dtype=dtype, max_tokens=max_tokens, max_slots=slots,
                    memory_limit_bytes=budget, max_rows_per_step=step_rows)
    if stops is None:
        stops = list(getattr(config, "eos_token_ids", ()))
    # Without a capture the loop runs one step ahead of the host and nothing waits per token; the per-step
    # report (each token's logit, each step's duration) needs the logits row and a wait per step, so it is
    # made only where --logits-out or --step-timing-out asks for it.
    keep = "--logits-out" in flags
    per_step = keep or "--step-timing-out" in flags
    step_logits = {i: [] for i in range(len(prompts))}
    stamps = []

    def on_logits(index, step, row):
        step_logits[index].append(row.float().cpu().numpy() if keep else float(row.max()))

    def control():
        import torch
        torch.cuda.synchronize()
        stamps.append(time.perf_counter())

    import torch
    torch.cuda.synchronize()
    started = time.perf_counter()
    stamps.append(started)
    results = engine.generate(prompts, max_new, temperature=temperature, top_k=top_k, top_p=top_p, seed=seed,
                              stop_token_ids=stops, batch_size=batch_size, control=control if per_step else None,
                              on_logits=on_logits if per_step else None)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - started
    stamps.append(started + elapsed)
    print(flags["--model"], file=out)
    for index, (prompt, result) in enumerate(zip(prompts, results)):
        print(f"  request {index}", file=out)
        print(f"  prompt:    {prompt}", file=out)
        print(f"  generated: {result.token_ids}", file=out)
        for step, token in enumerate(result.token_ids if per_step else ()):
            row = step_logits[index][step]
            value = float(row[token]) if keep else row
            note = "" if keep or temperature == 0.0 else " (largest logit of the step)"
            print(f"    step {step:>3}: token {token:>6}, logit {value:.7f}{note}", file=out)
        reason = result.finish_reason + (f" (token {result.stop_token})" if result.stop_token is not None else "")
        print(f"  finish:    {reason}", file=out)
    total = sum(r.completion_tokens for r in results)
    print(f"  device:    {engine.device} ({dtype})", file=out)
    if total:
        print(f"  decode:     {elapsed:.2f}s ({elapsed / total:.4f}s / generated token, {total / elapsed:.1f} generated "
              f"tokens/s, prompts included)", file=out)
    else:
        print(f"  decode:     {elapsed:.2f}s (no generated tokens)", file=out)
    if keep:
        for index, result in enumerate(results):
            if not result.token_ids:
                continue
            path = flags["--logits-out"] if len(prompts) == 1 else f"{flags['--logits-out']}.{index}"
            write_logits_artifact(path, prompts[index], result.token_ids, step_logits[index][:len(result.token_ids)],
                                  check_argmax=(temperature == 0.0))
    if "--step-timing-out" in flags:
        with open(flags["--step-timing-out"], "x", encoding="utf-8") as handle:
            handle.write("step\tduration_ms\n")
            for step in range(1, len(stamps) - 1):
                handle.write(f"{step - 1}\t{(stamps[step + 1] - stamps[step]) * 1e3:.3f}\n")
    return 0


def _random_model(args: list, out) -> int:
    flags = _parse_flags(args, valued={"--config", "--out", "--seed", "--dtype"}, switches=set())
    if "--config" not in flags or "--out" not in flags:
        raise UsageError("random-model needs --config FILE and --out DIR")
    from .weights.random_init import write_random_model

    with open(flags["--config"], "r", encoding="utf-8") as handle:
        data = json.load(handle)
    folder = write_random_model(flags["--out"], data, _number(flags, "--seed", 0), flags.get("--dtype", "bfloat16"))
    print(folder, file=out)
    return 0


def _compare(args: list, out) -> int:
    """Two logits captures: equal descriptors, then
    equal bytes, or with --tolerance X logits within X of the largest logit.  In the manner of the reference's
    tools/compare_logits.py:291-316: FAIL with the reason, or the shape, the SHA-256 and PASS."""
    paths = [a for a in args[:2] if not a.startswith("--")]
    if len(paths) != 2:
        raise UsageError("compare needs two captures")
    flags = _parse_flags(args[2:], valued={"--tolerance"}, switches=set())
    tolerance = _number(flags, "--tolerance", 0.0, float)
    if not tolerance >= 0.0:
        raise UsageError("--tolerance is not negative")
    from .engine.artifact import ArtifactError
    from .engine.compare import CompareError, compare
    try:
        report = compare(paths[0], paths[1], tolerance)
    except (CompareError, ArtifactError, OSError) as error:
        print(f"FAIL: {error}", file=out)
        return 1
    print(f"  shape: requests={report['requests']}, rows={report['rows']}, vocab={report['vocab']}", file=out)
    if tolerance == 0.0:
        print(f"  SHA-256: {report['sha256']}", file=out)
        print("  Exact logit comparison: PASS", file=out)
    else:
        print(f"  largest difference: {report['error']:.3e} of the largest logit ({report['worst']})", file=out)
        print(f"  Logit comparison within {tolerance:g}: PASS", file=out)
    return 0


def main(argv=None, out=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    out = out or sys.stdout
    try:
        if not argv or argv[0] in ("-h", "--help", "help"):
            print(USAGE, file=out)
            return 0 if argv else 2
        command, rest = argv[0], argv[1:]
        if command == "generate":
            return _generate(rest, out)
        if command == "random-model":
            return _random_model(rest, out)
        if command == "compare":
            return _compare(rest, out)
        if command == "architectures":
            from .registry import registered_architectures
            print("\n".join(registered_architectures()), file=out)
            return 0
        raise UsageError(f"unknown command {command!r}")
    except UsageError as error:
        print(f"error: {error}\n{USAGE}", file=sys.stderr)
        return 2
    except (ValueError, OSError, *_library_errors()) as error:
        # a value that some part refuses, a file that is not there, a model that does not fit: one line, not a traceback
        print(f"error: {error}", file=sys.stderr)
        return 1


def _library_errors() -> tuple:
    from .cache import CacheError
    from .engine.engine import MemoryBudgetError
    from .kernels import KernelError
    from .kernels.build import BuildError
    from .sampling import SamplingError
    return (CacheError, MemoryBudgetError, BuildError, KernelError, SamplingError)
