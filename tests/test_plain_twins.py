"""The kernels' plain C++ twins: their self-test under the host sanitizers, and the twins against the plain
implementation's functions of the same formulas on random data."""

import subprocess

import numpy as np
import pytest

import plain_qwen3 as plain
import twins as twins_module
from beholdd.kernels import build

RNG = np.random.default_rng(77)


@pytest.fixture(scope="module")
def twins(tmp_path_factory):
    return twins_module.Twins(tmp_path_factory.mktemp("twins"))


def test_self_test_under_the_address_and_undefined_behaviour_sanitizers(tmp_path):
    program = build.build_plain_twins(str(tmp_path), selftest=True)
    run = subprocess.run([program], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and "self-test ok" in run.stdout, run.stdout + run.stderr


def test_elementwise_twins_are_the_plain_functions(twins):
    x = RNG.normal(size=(5, 200)).astype(np.float32) * 3
    w = (1 + 0.3 * RNG.normal(size=200)).astype(np.float32)
    assert np.allclose(twins.rmsnorm(x, w, 1e-5), plain.rmsnorm(x, w, 1e-5), rtol=1e-6, atol=1e-7)
    assert np.allclose(twins.rmsnorm(x, w, 1e-5, rows=[4, 0]), plain.rmsnorm(x[[4, 0]], w, 1e-5), rtol=1e-6, atol=1e-7)
    gate_up = RNG.normal(size=(3, 2 * 37)).astype(np.float32) * 4
    assert np.allclose(twins.swiglu(gate_up), plain.swiglu(gate_up[:, :37], gate_up[:, 37:]), rtol=1e-6, atol=1e-7)
    a, m = RNG.normal(size=(4, 120)).astype(np.float32), RNG.normal(size=(7, 120)).astype(np.float32)
    assert np.allclose(twins.gemm(a, m), plain.linear(a, m), rtol=1e-6, atol=1e-6)
    assert np.allclose(twins.gemm(a, m, c=np.ones((4, 7), np.float32)), plain.linear(a, m) + 1, rtol=1e-6, atol=1e-6)
    table = RNG.normal(size=(11, 6)).astype(np.float32)
    status, rows = twins.embed([3, 10, 0], table)
    assert status == 0 and np.array_equal(rows, plain.embed([3, 10, 0], table))
    logits = RNG.normal(size=(3, 50)).astype(np.float32)
    logits[1, 7] = logits[1, 40] = 9.0
    logits[2, 3] = np.nan
    tokens, bad = twins.argmax(logits)
    assert tokens.tolist() == [plain.greedy_token(logits[0]), 7, -1] and bad.tolist() == [0, 0, 1]
    # bfloat16 storage: the twin rounds what it stores and computes on the rounded values
    rounded = twins_module.from_bf16_bits(twins_module.to_bf16_bits(gate_up))
    assert np.allclose(twins.swiglu(gate_up, twins_module.BF16), plain.swiglu(rounded[:, :37], rounded[:, 37:]), rtol=8e-3)


@pytest.mark.parametrize("order,head_dim,rot", [(0, 24, 24), (0, 32, 16), (1, 32, 32), (1, 64, 0)])
def test_cache_write_and_attention_twins_are_the_plain_functions(twins, order, head_dim, rot):
    """Three sequences with pasts of 0, 70 and 5 tokens get 9, 3 and 130 more: norm, rotation, cache write through
    shuffled pages, then attention over the pages, against the plain functions on whole sequences."""
    n_heads, kv_heads, eps, theta, window = 6, 2, 1e-5, 10000.0, 0
    lengths = [(0, 9), (70, 3), (5, 130)]
    n_pages = 9
    pages = RNG.permutation(n_pages).tolist()
    table = np.zeros((3, 3), np.int32)
    for s, (past, new) in enumerate(lengths):
        for j in range(-(-(past + new) // 64)):
            table[s, j] = pages.pop()
    fused = (n_heads + 2 * kv_heads) * head_dim
    whole = [RNG.normal(size=(past + new, fused)).astype(np.float32) for past, new in lengths]
    qw, kw = (1 + 0.3 * RNG.normal(size=head_dim)).astype(np.float32), (1 + 0.3 * RNG.normal(size=head_dim)).astype(np.float32)
    freqs = plain.rope_frequencies(theta, rot) if rot else None
    top = max(past + new for past, new in lengths)
    cos = np.stack([plain.rope_cos_sin(freqs, p)[0] for p in range(top)]) if rot else None
    sin = np.stack([plain.rope_cos_sin(freqs, p)[1] for p in range(top)]) if rot else None
    k_pages = v_pages = None
    q_new = []
    for phase in (0, 1):       # the pasts first, then the new rows: two steps onto the same pages
        rows, positions, row_seq = [], [], []
        for s, (past, new) in enumerate(lengths):
            lo, hi = (0, past) if phase == 0 else (past, past + new)
            rows.append(whole[s][lo:hi])
            positions.extend(range(lo, hi))
            row_seq.extend([s] * (hi - lo))
        q_out, k_pages, v_pages = twins.qk_norm_rope_cache(np.concatenate(rows), qw, kw, eps, cos, sin, positions, row_seq, table,
                                                           n_pages, n_heads, kv_heads, head_dim, order, k_pages=k_pages, v_pages=v_pages)
        if phase == 1:
            q_new, new_positions, new_row_seq = q_out, positions, row_seq
    scale = 1 / np.sqrt(head_dim)
    got = twins.attention(q_new, k_pages, v_pages, table, new_row_seq, new_positions, n_heads, kv_heads, head_dim, scale, window, order)
    at = 0
    for s, (past, new) in enumerate(lengths):
        total = past + new
        q = plain.rmsnorm(whole[s][:, :n_heads * head_dim].reshape(total, n_heads, head_dim), qw, eps)
        k = plain.rmsnorm(whole[s][:, n_heads * head_dim:(n_heads + kv_heads) * head_dim].reshape(total, kv_heads, head_dim), kw, eps)
        v = whole[s][:, (n_heads + kv_heads) * head_dim:]
        for t in range(total if rot else 0):
            cs = plain.rope_cos_sin(freqs, t)
            q[t, :, :rot], k[t, :, :rot] = plain.rope_split_half(q[t, :, :rot], *cs), plain.rope_split_half(k[t, :, :rot], *cs)
        # the cache holds the rotated keys and the raw values where the page table says
        for t in (0, total - 1, min(64, total - 1)):
            page = table[s, t // 64]
            assert np.allclose(twins.key(k_pages, order, page, 1, t % 64, head_dim), k[t, 1], rtol=1e-5, atol=1e-6)
            assert np.allclose(twins.value(v_pages, order, page, 0, t % 64, head_dim), v[t, :head_dim], rtol=1e-6, atol=1e-7)
        want = plain.causal_attention(q[past:].reshape(new, -1), k.reshape(total, -1), v, n_heads, kv_heads, head_dim, scale,
                                      query_start=past)
        assert np.allclose(got[at:at + new], want, rtol=2e-5, atol=2e-6), s
        at += new


@pytest.mark.parametrize("block_rows", [8, 16])
def test_rows_in_blocks_are_a_permutation_in_operand_order(twins, block_rows):
    """Every element of a matrix whose rows lie in blocks has a place of its own within the whole blocks; a block is
    32 columns of `block_rows` rows, and inside it eight columns of a row lie together, the rows of those eight
    columns one after the other, then the next eight columns: what one matrix-core operand load takes."""
    rows, width = 2 * block_rows + 3, 96
    index = twins.rows_index(block_rows, rows, width)
    padded = -(-rows // block_rows) * block_rows
    assert len(set(index.ravel().tolist())) == rows * width and index.min() == 0 and index.max() < padded * width
    assert np.array_equal(twins.rows_index(0, rows, width), np.arange(rows * width).reshape(rows, width))
    for r in (0, 1, block_rows - 1, block_rows, rows - 1):
        for c in (0, 7, 8, 31, 32, 95):
            block = (r // block_rows) * (width // 32) + c // 32
            want = block * 32 * block_rows + (((c % 32) // 8) * block_rows + r % block_rows) * 8 + c % 8
            assert index[r, c] == want


def test_the_draws_twin_is_an_inverse_cdf_over_the_kept_tokens(twins):
    """The sampler's twin against NumPy and SciPy: the distribution it draws from is softmax(logits / temperature)
    cut to the top k and to the smallest most likely set that reaches top_p, in index order."""
    from scipy.special import softmax
    rng = np.random.default_rng(3)
    vocab = 200
    logits = (rng.normal(size=(1, vocab)) * 2).astype(np.float32)
    for temperature, k, p in ((1.0, 0, 1.0), (0.6, 0, 1.0), (1.3, 10, 1.0), (1.5, 0, 0.7), (1.6, 25, 0.9)):
        masses = softmax(logits[0].astype(np.float64) / temperature)
        keep = np.ones(vocab, bool)
        if k:
            keep &= logits[0] >= np.sort(logits[0])[-k]
        if p < 1.0:
            order = np.argsort(-masses * keep, kind="stable")
            reached = np.cumsum((masses * keep)[order]) >= p * (masses * keep).sum()
            keep &= masses >= masses[order[np.argmax(reached)]]
        edges = np.concatenate([[0.0], np.cumsum(masses * keep)]) / (masses * keep).sum()
        draws = rng.random(400).astype(np.float32)
        got, bad, margin = twins.sample(np.repeat(logits, 400, axis=0), np.full(400, temperature), draws,
                                        top_k=np.full(400, k, np.int32), top_p=np.full(400, p, np.float32))
        want = np.searchsorted(edges, draws.astype(np.float64), side="right") - 1
        sure = margin > 1e-9
        assert bad.sum() == 0 and sure.sum() > 390 and np.array_equal(got[sure], want[sure])
        assert keep[got].all() and len(set(got.tolist())) > 3
    greedy, _, _ = twins.sample(logits, np.zeros(1), np.zeros(1, np.float32))
    assert greedy[0] == int(np.argmax(logits[0]))
