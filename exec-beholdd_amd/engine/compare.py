"""Comparing two logits captures.

The reference's tools/compare_logits.py validates two captures, requires equal descriptors (:233-256) and
then equal bytes, reporting the first differing offset and both SHA-256 sums (:259-288).  Here the same with
a tolerance: captures of replays that cut the same requests differently hold the same positions in another
order and agree within rounding, not bit for bit.  `compare(a, b, tolerance)`:
  both files are validated by their readers;
  descriptors must agree: vocabulary, the requests' names and tokens, and the set of (request, position) rows;
  tolerance 0: the rows must come in the same order and the files must be equal byte for byte;
  tolerance > 0: max |a - b| over all rows, divided by max |a|, must not exceed it; the worst row is named.
Version-1 captures (one request's generated steps) compare the same way, prompt and generated ids being the
descriptor.
"""

from __future__ import annotations

import hashlib

import numpy as np

from .artifact import ArtifactError, read_logits_artifact, read_position_capture


class CompareError(ValueError):
    """The two captures do not describe the same thing, or differ by more than allowed."""


def _version(path: str) -> int:
    with open(path, "rb") as handle:
        head = handle.read(10)
    if len(head) < 10 or head[:8] != b"BHDLOGIT":
        raise ArtifactError(f"{path}: not a logits capture")
    return int.from_bytes(head[8:10], "little")


def _first_byte_difference(left: bytes, right: bytes):
    size = 1 << 20
    for start in range(0, min(len(left), len(right)), size):
        a, b = left[start:start + size], right[start:start + size]
        if a != b:
            for offset, (x, y) in enumerate(zip(a, b)):
                if x != y:
                    return start + offset, x, y
    return None


def _compare_bytes(path_a: str, path_b: str) -> str:
    with open(path_a, "rb") as handle:
        left = handle.read()
    with open(path_b, "rb") as handle:
        right = handle.read()
    sums = (hashlib.sha256(left).hexdigest(), hashlib.sha256(right).hexdigest())
    if left == right:
        return sums[0]
    hashes = f"reference SHA-256 {sums[0]}, candidate SHA-256 {sums[1]}"
    difference = _first_byte_difference(left, right)
    if difference is None:
        raise CompareError(f"file bytes differ in length: {len(left)} vs {len(right)}; {hashes}")
    offset, x, y = difference
    raise CompareError(f"file bytes differ at offset {offset}: reference 0x{x:02x}, candidate 0x{y:02x}; {hashes}")


def _relative(a: np.ndarray, b: np.ndarray):
    """(max |a - b| / max |a|, index of the worst row)."""
    difference = np.abs(a.astype(np.float64) - b.astype(np.float64)).max(axis=1)
    return float(difference.max() / max(float(np.abs(a).max()), 1e-30)), int(difference.argmax())


def compare(path_a: str, path_b: str, tolerance: float = 0.0) -> dict:
    """Compare two captures (see the module's text).  Returns a report; raises CompareError on a mismatch and
    ArtifactError for a file that is no valid capture."""
    if tolerance < 0:
        raise ValueError("the tolerance is not negative")
    versions = (_version(path_a), _version(path_b))
    if versions[0] != versions[1]:
        raise CompareError(f"descriptor mismatch: capture versions differ: {versions[0]} vs {versions[1]}")
    if versions[0] == 1:
        prompt_a, generated_a, logits_a = read_logits_artifact(path_a, check_argmax=False)
        prompt_b, generated_b, logits_b = read_logits_artifact(path_b, check_argmax=False)
        for label, left, right in (("prompt ids", prompt_a, prompt_b), ("generated ids", generated_a, generated_b)):
            if left != right:
                raise CompareError(f"descriptor mismatch: {label} differ: {left} vs {right}")
        if logits_a.shape != logits_b.shape:
            raise CompareError(f"descriptor mismatch: logits are {logits_a.shape} vs {logits_b.shape}")
        report = {"rows": logits_a.shape[0], "vocab": logits_a.shape[1], "requests": 1}
        if tolerance == 0:
            report["sha256"] = _compare_bytes(path_a, path_b)
            report["error"] = 0.0
            return report
        error, worst = _relative(logits_a, logits_b)
        report.update(error=error, worst=f"step {worst}")
    else:
        a, b = read_position_capture(path_a), read_position_capture(path_b)
        if a.vocab != b.vocab:
            raise CompareError(f"descriptor mismatch: vocabulary size differs: {a.vocab} vs {b.vocab}")
        if sorted(a.requests) != sorted(b.requests):
            raise CompareError(f"descriptor mismatch: requests differ: {sorted(a.requests)} vs {sorted(b.requests)}")
        for name in a.requests:
            if a.requests[name] != b.requests[name]:
                raise CompareError(f"descriptor mismatch: the tokens of request {name!r} differ")
        keys_a = [(name, position) for name, position, _ in a.rows]
        keys_b = [(name, position) for name, position, _ in b.rows]
        if len(set(keys_a)) != len(keys_a) or len(set(keys_b)) != len(keys_b):
            raise CompareError("descriptor mismatch: a capture holds a position twice")
        if set(keys_a) != set(keys_b):
            only = sorted(set(keys_a) ^ set(keys_b))[:5]
            raise CompareError(f"descriptor mismatch: the captures hold different positions, for instance {only}")
        report = {"rows": len(keys_a), "vocab": a.vocab, "requests": len(a.requests)}
        if tolerance == 0:
            if a.rows != b.rows:
                raise CompareError("descriptor mismatch: the rows come in another order or from other steps; "
                                   "an exact comparison needs the same schedule")
            report["sha256"] = _compare_bytes(path_a, path_b)
            report["error"] = 0.0
            return report
        where = {key: row for row, key in enumerate(keys_b)}
        order = np.asarray([where[key] for key in keys_a])
        error, worst = _relative(a.logits, b.logits[order])
        report.update(error=error, worst=f"request {keys_a[worst][0]!r}, position {keys_a[worst][1]}")
    if report["error"] > tolerance:
        raise CompareError(f"logits differ by {report['error']:.3e} of the largest logit at {report['worst']}; "
                           f"the tolerance is {tolerance:g}")
    return report
