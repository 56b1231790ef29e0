"""The logits capture file: prompt ids, generated ids and the logits row of every step.

Layout as the reference defines it (crates/beholdd-model/src/artifact.rs:18-22, :136-158, read
back by tools/compare_logits.py:14-24), all little-endian:
  header  64 bytes: magic "BHDLOGIT", u16 version 1, u16 header length 64, u32 scalar encoding
                    (1 = float32), u64 prompt length, u64 step count, u64 vocabulary,
                    u64 logit count (= steps x vocabulary), u64 body length in bytes, u64 zero
  body    prompt ids u32, generated ids u32, logits float32 bits row-major [steps, vocabulary]
  footer  u64 total length, magic "BHDLEND!"
The writer refuses to overwrite and publishes the finished file under its name at once; the
reader re-derives the argmax of every row (ties to the lowest id) and compares it with the
recorded token (artifact.rs:182-250).
"""

from __future__ import annotations

import os
import struct

import numpy as np

MAGIC, FOOTER_MAGIC = b"BHDLOGIT", b"BHDLEND!"
VERSION, HEADER_LEN, SCALAR_F32 = 1, 64, 1
_HEADER = struct.Struct("<8sHHIQQQQQQ")


class ArtifactError(ValueError):
    pass


def write_logits_artifact(path: str, prompt: list, generated: list, step_logits, check_argmax: bool = True):
    logits = np.ascontiguousarray(np.asarray(step_logits, dtype="<f4"))
    steps = len(generated)
    if logits.ndim != 2 or logits.shape[0] != steps:
        raise ArtifactError(f"{steps} generated tokens need {steps} logits rows, got shape {logits.shape}")
    if len(prompt) == 0 or steps == 0:
        raise ArtifactError("a capture needs a prompt and at least one step")
    vocab = logits.shape[1]
    if not np.isfinite(logits).all():
        raise ArtifactError("a logit is not finite")
    ids = np.asarray(list(prompt) + list(generated), dtype="<u4")
    if ids.max() >= vocab:
        raise ArtifactError("a token id is outside the vocabulary")
    if check_argmax:
        for step, token in enumerate(generated):
            if int(np.argmax(logits[step])) != int(token):
                raise ArtifactError(f"step {step}: token {token} is not the argmax of its logits row")
    if os.path.lexists(path):
        raise ArtifactError(f"{path} exists; a capture is never overwritten")
    body_len = ids.nbytes + logits.nbytes
    total = HEADER_LEN + body_len + 16
    tmp = f"{path}.tmp{os.getpid()}"
    with open(tmp, "wb") as handle:
        handle.write(_HEADER.pack(MAGIC, VERSION, HEADER_LEN, SCALAR_F32, len(prompt), steps, vocab,
                                  steps * vocab, body_len, 0))
        handle.write(ids.tobytes())
        handle.write(logits.tobytes())
        handle.write(struct.pack("<Q8s", total, FOOTER_MAGIC))
        handle.flush()
        os.fsync(handle.fileno())
    try:
        os.link(tmp, path)      # fails if another writer got there first
    finally:
        os.remove(tmp)


def read_logits_artifact(path: str, check_argmax: bool = True):
    """Returns (prompt ids, generated ids, logits [steps, vocab]) after validating the file."""
    with open(path, "rb") as handle:
        data = handle.read()
    if len(data) < HEADER_LEN + 16:
        raise ArtifactError(f"{path}: too short for a capture")
    magic, version, header_len, scalar, n_prompt, steps, vocab, count, body_len, reserved = _HEADER.unpack_from(data)
    if magic != MAGIC or version != VERSION or header_len != HEADER_LEN or scalar != SCALAR_F32 or reserved != 0:
        raise ArtifactError(f"{path}: not a version-{VERSION} float32 logits capture")
    if n_prompt == 0 or steps == 0 or vocab == 0:
        raise ArtifactError(f"{path}: sizes must be non-zero")
    if count != steps * vocab or body_len != 4 * (n_prompt + steps + count):
        raise ArtifactError(f"{path}: the header's counts do not agree")
    total, footer = struct.unpack_from("<Q8s", data, HEADER_LEN + body_len)
    if footer != FOOTER_MAGIC or total != len(data) or total != HEADER_LEN + body_len + 16:
        raise ArtifactError(f"{path}: bad footer or length")
    ids = np.frombuffer(data, dtype="<u4", count=n_prompt + steps, offset=HEADER_LEN)
    logits = np.frombuffer(data, dtype="<f4", count=count, offset=HEADER_LEN + 4 * (n_prompt + steps))
    logits = logits.reshape(steps, vocab)
    if ids.max() >= vocab:
        raise ArtifactError(f"{path}: a token id is outside the vocabulary")
    if not np.isfinite(logits).all():
        raise ArtifactError(f"{path}: a logit is not finite")
    generated = [int(t) for t in ids[n_prompt:]]
    if check_argmax:
        for step, token in enumerate(generated):
            if int(np.argmax(logits[step])) != token:
                raise ArtifactError(f"{path}: step {step}: token {token} is not the argmax of its row")
    return [int(t) for t in ids[:n_prompt]], generated, logits
