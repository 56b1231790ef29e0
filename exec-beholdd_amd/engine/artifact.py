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


# ---- version 2: the logits of given positions of several requests ---------------------------------------------
# What a replay writes: the reference's capture holds one request's generated steps only; a replay feeds given
# tokens in any schedule, so its capture names, for every logits row, the request, the position in it and the
# step that computed it, and holds every request's tokens.  Layout (little-endian):
#   header  64 bytes: magic "BHDLOGIT", u16 version 2, u16 header length 64, u32 scalar encoding (1 = float32),
#                     u64 kind (2 = positions), u64 request count, u64 vocabulary, u64 row count,
#                     u64 offset of the tables, u64 zero
#   logits  float32 bits, row-major [rows, vocabulary], from byte 64
#   tables  per row: u32 request index, u32 position, u32 step number;
#           per request: u32 length of its name in bytes, the name (UTF-8) padded with zeros to a multiple of 4,
#                        u32 token count, token ids u32;
#           u32 length of a JSON text of notes (engine dtype and the like), the text padded likewise
#   footer  u64 total length, magic "BHDLEND!"
# Rows are appended while the replay runs; tables, footer and the final header are written when it ends, and only
# then does the file appear under its name.

KIND_POSITIONS = 2
_HEADER2 = struct.Struct("<8sHHIQQQQQQ")


def _padded(data: bytes) -> bytes:
    return data + b"\0" * (-len(data) % 4)


class PositionCaptureWriter:
    """Appends logits rows step by step; `close()` completes and publishes the file (never over another)."""

    def __init__(self, path: str, vocab: int, notes: dict | None = None):
        if os.path.lexists(path):
            raise ArtifactError(f"{path} exists; a capture is never overwritten")
        self.path, self.vocab, self.notes = path, int(vocab), dict(notes or {})
        self._tmp = f"{path}.tmp{os.getpid()}"
        self._file = open(self._tmp, "wb")
        self._file.write(b"\0" * HEADER_LEN)
        self._rows: list = []          # (request index, position, step)
        self._requests: dict = {}      # name -> [index, tokens]

    def feed(self, name: str, tokens) -> int:
        """Note that `tokens` were appended to request `name`; returns the position of the first of them."""
        entry = self._requests.setdefault(str(name), [len(self._requests), []])
        first = len(entry[1])
        entry[1].extend(int(t) for t in tokens)
        return first

    def add(self, step: int, places: list, logits) -> None:
        """`logits` [len(places), vocab] float32 for `places` = [(request name, position)]."""
        rows = np.ascontiguousarray(np.asarray(logits, dtype="<f4"))
        if rows.ndim != 2 or rows.shape != (len(places), self.vocab):
            raise ArtifactError(f"{len(places)} places need logits [{len(places)}, {self.vocab}], got {rows.shape}")
        if not np.isfinite(rows).all():
            raise ArtifactError(f"step {step}: a logit is not finite")
        for name, position in places:
            index, tokens = self._requests[str(name)]
            if not 0 <= position < len(tokens):
                raise ArtifactError(f"step {step}: request {name!r} has no position {position}")
            self._rows.append((index, int(position), int(step)))
        self._file.write(rows.tobytes())

    def close(self) -> None:
        if self._file is None:
            return
        handle, self._file = self._file, None
        try:
            table_offset = HEADER_LEN + 4 * self.vocab * len(self._rows)
            handle.write(np.asarray(self._rows, dtype="<u4").reshape(-1, 3).tobytes())
            for name, (_, tokens) in sorted(self._requests.items(), key=lambda item: item[1][0]):
                raw = name.encode("utf-8")
                if any(t >= self.vocab for t in tokens):
                    raise ArtifactError(f"request {name!r}: a token id is outside the vocabulary")
                handle.write(struct.pack("<I", len(raw)) + _padded(raw) + struct.pack("<I", len(tokens)))
                handle.write(np.asarray(tokens, dtype="<u4").tobytes())
            import json
            notes = json.dumps(self.notes, sort_keys=True).encode("utf-8")
            handle.write(struct.pack("<I", len(notes)) + _padded(notes))
            total = handle.tell() + 16
            handle.write(struct.pack("<Q8s", total, FOOTER_MAGIC))
            handle.seek(0)
            handle.write(_HEADER2.pack(MAGIC, 2, HEADER_LEN, SCALAR_F32, KIND_POSITIONS, len(self._requests),
                                       self.vocab, len(self._rows), table_offset, 0))
            handle.flush()
            os.fsync(handle.fileno())
            handle.close()
            os.link(self._tmp, self.path)      # fails if another writer got there first
        finally:
            if not handle.closed:
                handle.close()
            os.remove(self._tmp)

    def abandon(self) -> None:
        if self._file is not None:
            self._file.close()
            self._file = None
            os.remove(self._tmp)


class PositionCapture:
    """A validated version-2 capture: `requests` {name: token ids}, `rows` [(name, position, step)],
    `logits` [rows, vocab], `notes`, and the file's `sha256`."""

    def __init__(self, path, requests, rows, logits, notes, sha256):
        self.path, self.requests, self.rows, self.logits, self.notes, self.sha256 = path, requests, rows, logits, notes, sha256
        self.vocab = logits.shape[1]


def read_position_capture(path: str) -> PositionCapture:
    import hashlib
    import json

    with open(path, "rb") as handle:
        data = handle.read()
    if len(data) < HEADER_LEN + 16:
        raise ArtifactError(f"{path}: too short for a capture")
    magic, version, header_len, scalar, kind, n_requests, vocab, n_rows, table_offset, reserved = _HEADER2.unpack_from(data)
    if magic != MAGIC or version != 2 or header_len != HEADER_LEN or scalar != SCALAR_F32 or kind != KIND_POSITIONS \
            or reserved != 0:
        raise ArtifactError(f"{path}: not a version-2 float32 capture of positions")
    if vocab == 0 or n_rows == 0 or n_requests == 0:
        raise ArtifactError(f"{path}: sizes must be non-zero")
    total, footer = struct.unpack_from("<Q8s", data, len(data) - 16)
    if footer != FOOTER_MAGIC or total != len(data):
        raise ArtifactError(f"{path}: bad footer or length")
    if table_offset != HEADER_LEN + 4 * vocab * n_rows or table_offset + 12 * n_rows > len(data) - 16:
        raise ArtifactError(f"{path}: the header's counts do not agree")
    logits = np.frombuffer(data, dtype="<f4", count=n_rows * vocab, offset=HEADER_LEN).reshape(n_rows, vocab)
    if not np.isfinite(logits).all():
        raise ArtifactError(f"{path}: a logit is not finite")
    table = np.frombuffer(data, dtype="<u4", count=3 * n_rows, offset=table_offset).reshape(n_rows, 3)
    at, end = table_offset + 12 * n_rows, len(data) - 16

    def take(count):
        nonlocal at
        if at + count > end:
            raise ArtifactError(f"{path}: the tables run past the end of the file")
        piece = data[at:at + count]
        at += count
        return piece

    names, requests = [], {}
    for _ in range(n_requests):
        (length,) = struct.unpack("<I", take(4))
        name = take(length + (-length % 4))[:length].decode("utf-8")
        (count,) = struct.unpack("<I", take(4))
        tokens = np.frombuffer(take(4 * count), dtype="<u4")
        if name in requests:
            raise ArtifactError(f"{path}: request {name!r} is listed twice")
        if count and tokens.max() >= vocab:
            raise ArtifactError(f"{path}: request {name!r}: a token id is outside the vocabulary")
        names.append(name)
        requests[name] = [int(t) for t in tokens]
    (length,) = struct.unpack("<I", take(4))
    notes = json.loads(take(length + (-length % 4))[:length].decode("utf-8") or "{}")
    if at != end:
        raise ArtifactError(f"{path}: {end - at} bytes between the tables and the footer")
    rows = []
    for index, position, step in table.tolist():
        if index >= n_requests or position >= len(requests[names[index]]):
            raise ArtifactError(f"{path}: a row names request {index}, position {position}, which does not exist")
        rows.append((names[index], position, step))
    return PositionCapture(path, requests, rows, logits, notes, hashlib.sha256(data).hexdigest())
