"""The greedy selection that allocates nothing (`bh_sample_greedy_static`), called through ctypes as a
caller without an allocator would, against the entry point it is a variant of (`bh_sample`)."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from beholdd.kernels import build

    lib = ctypes.CDLL(build.ensure_built(verbose=False))
    p, i = ctypes.c_void_p, ctypes.c_int
    lib.bh_last_error.restype = ctypes.c_char_p
    lib.bh_sample_scratch.argtypes, lib.bh_sample_scratch.restype = [i, i], i
    lib.bh_sample.argtypes, lib.bh_sample.restype = [p, p, p, p, p, p, p, p, i, i, p], i
    lib.bh_sample_greedy_static.argtypes, lib.bh_sample_greedy_static.restype = [p, p, p, i, i, p], i
    return lib


def _existing(lib, logits):
    rows, vocab = logits.shape
    tokens = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    bad = torch.full((rows,), -7, dtype=torch.int32, device=logits.device)
    words = lib.bh_sample_scratch(rows, vocab)
    scratch = torch.empty(max(words, 1), dtype=torch.float32, device=logits.device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    status = lib.bh_sample(logits.data_ptr(), None, None, None, None, tokens.data_ptr(), bad.data_ptr(),
                           scratch.data_ptr() if words else None, rows, vocab, stream)
    assert status == 0, lib.bh_last_error()
    torch.cuda.synchronize()
    return tokens.cpu(), bad.cpu()


def _static(lib, logits, tokens, bad):
    rows, vocab = logits.shape
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    status = lib.bh_sample_greedy_static(logits.data_ptr(), tokens.data_ptr(), bad.data_ptr(), rows, vocab, stream)
    assert status == 0, lib.bh_last_error()
    torch.cuda.synchronize()
    return tokens[:rows].cpu(), bad[:rows].cpu()


def _logits(rows, vocab, seed):
    generator = torch.Generator().manual_seed(seed)
    logits = torch.randn(rows, vocab, generator=generator)
    logits[0, vocab - 1] = logits[0, 5] = logits[0].max() + 1.0     # a tie: the lower id wins
    if rows > 2:
        logits[2, vocab // 2] = float("nan")                        # a row that is refused
    if rows > 3:
        logits[3, 0] = float("inf")
    return logits.to("cuda:0")


def test_two_calls_in_a_row_agree_with_the_allocating_entry_point():
    lib = _library()
    # outputs made once, before the calls: the entry point itself is given nothing to allocate with
    tokens = torch.empty(64, dtype=torch.int32, device="cuda:0")
    bad = torch.empty(64, dtype=torch.int32, device="cuda:0")
    first = _logits(7, 151_936, seed=1)          # 75 chunks per row
    second = _logits(3, 5_000, seed=2)           # smaller in both directions: the array still holds the first call's parts
    for logits in (first, second):
        tokens.fill_(-7)
        bad.fill_(-7)
        got_tokens, got_bad = _static(lib, logits, tokens, bad)
        want_tokens, want_bad = _existing(lib, logits)
        assert torch.equal(got_tokens, want_tokens), (got_tokens, want_tokens)
        assert torch.equal(got_bad, want_bad), (got_bad, want_bad)
        assert int(got_tokens[0]) == 5 and int(got_bad[0]) == 0
        assert int(got_tokens[2]) == -1 and int(got_bad[2]) == 1
        clean = torch.nan_to_num(logits.cpu(), nan=-1e30, posinf=-1e30)
        assert int(got_tokens[1]) == int(clean[1].argmax())


def test_sizes_beyond_the_static_array_are_refused_with_a_clear_error():
    lib = _library()
    logits = torch.zeros(4, 64, device="cuda:0")
    tokens = torch.full((4,), -7, dtype=torch.int32, device="cuda:0")
    bad = torch.full((4,), -7, dtype=torch.int32, device="cuda:0")
    # 300 rows x 75 chunks x 2 words > 32768: refused before anything is launched or read
    status = lib.bh_sample_greedy_static(logits.data_ptr(), tokens.data_ptr(), bad.data_ptr(), 300, 151_936, None)
    assert status != 0
    message = lib.bh_last_error().decode()
    assert "static array" in message and "45000" in message
    torch.cuda.synchronize()
    assert tokens.cpu().tolist() == [-7] * 4


_CAPTURE = r"""
import ctypes, sys
import torch
sys.path.insert(0, {root!r})
from beholdd.kernels import build
lib = ctypes.CDLL(build.ensure_built(verbose=False))
p, i = ctypes.c_void_p, ctypes.c_int
lib.bh_last_error.restype = ctypes.c_char_p
lib.bh_sample_scratch.argtypes, lib.bh_sample_scratch.restype = [i, i], i
lib.bh_sample.argtypes, lib.bh_sample.restype = [p, p, p, p, p, p, p, p, i, i, p], i
lib.bh_sample_greedy_static.argtypes, lib.bh_sample_greedy_static.restype = [p, p, p, i, i, p], i
rows, vocab = 6, 40_000
logits = torch.randn(rows, vocab, device="cuda:0")
tokens = torch.full((rows,), -7, dtype=torch.int32, device="cuda:0")
bad = torch.full((rows,), -7, dtype=torch.int32, device="cuda:0")
def static(stream):
    status = lib.bh_sample_greedy_static(logits.data_ptr(), tokens.data_ptr(), bad.data_ptr(), rows, vocab, ctypes.c_void_p(stream))
    assert status == 0, lib.bh_last_error()
if {warm}:
    static(torch.cuda.current_stream().cuda_stream)      # an eager call first: the array's address is known before the capture
    torch.cuda.synchronize()
graph = torch.cuda.CUDAGraph()
with torch.cuda.graph(graph):
    static(torch.cuda.current_stream().cuda_stream)
words = lib.bh_sample_scratch(rows, vocab)
scratch = torch.empty(max(words, 1), dtype=torch.float32, device="cuda:0")
want, want_bad = torch.empty_like(tokens), torch.empty_like(bad)
for replay in range(4):                # other work and synchronisations between the replays; every replay is checked
    logits.normal_()
    logits[replay % rows, 17] = 50.0
    if replay == 2:
        logits[1, 9] = float("nan")
    tokens.fill_(-7)
    torch.cuda.synchronize()
    graph.replay()
    status = lib.bh_sample(logits.data_ptr(), None, None, None, None, want.data_ptr(), want_bad.data_ptr(),
                           scratch.data_ptr() if words else None, rows, vocab, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert status == 0, lib.bh_last_error()
    torch.cuda.synchronize()
    assert torch.equal(tokens, want) and torch.equal(bad, want_bad), (replay, tokens, want)
    assert int(tokens[replay % rows]) in (17, -1)
print("capture ok")
"""


@pytest.mark.parametrize("warm", [False, True])
def test_the_call_inside_a_captured_graph(warm):
    """What the entry point is for: the call recorded into a HIP graph, in a process of its own so that the capture
    can be the very first call on the device (the array's address is asked for inside it), and after an eager call;
    four replays with other work between them against the allocating entry point."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = subprocess.run([sys.executable, "-c", _CAPTURE.format(root=root, warm=warm)], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and "capture ok" in run.stdout, run.stderr[-2000:]
