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
