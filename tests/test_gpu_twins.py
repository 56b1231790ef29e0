"""Every kernel beside its plain C++ twin (exec-beholdd_amd/csrc/plain_twins.cpp): the same arguments, the same
cache pages element for element, in float32 and in bfloat16."""

import math

import numpy as np
import pytest
import torch

import twins as twins_module
from twins import BF16, F32

pytestmark = pytest.mark.gpu
DEVICE = "cuda:0"
RNG = np.random.default_rng(5)


@pytest.fixture(scope="module")
def K():
    from beholdd.kernels import HipKernels
    return HipKernels(DEVICE)


@pytest.fixture(scope="module")
def twins(tmp_path_factory):
    return twins_module.Twins(tmp_path_factory.mktemp("twins"))


def dev(array, dtype=None):
    tensor = torch.from_numpy(np.ascontiguousarray(array)).to(DEVICE)
    return tensor.to(dtype) if dtype is not None else tensor


def host(tensor):
    return tensor.float().cpu().numpy()


def rel(got, want):
    return float(np.abs(got.astype(np.float64) - want).max() / max(np.abs(want).max(), 1e-30))


@pytest.mark.parametrize("block_rows,rows", [(8, 5), (8, 8), (16, 16), (16, 21), (16, 300)])
def test_rows_in_blocks_lie_where_the_twin_says(K, twins, block_rows, rows):
    """The regrouping kernel and the norm that writes blocks itself put every element where the index function
    that host and device code share says."""
    width = 96
    x = RNG.normal(size=(rows, width)).astype(np.float32)
    index = twins.rows_index(block_rows, rows, width)
    blocked = K.to_blocked(dev(x, torch.bfloat16), block_rows=block_rows)
    assert np.array_equal(host(blocked.data)[index], host(dev(x, torch.bfloat16)))
    from beholdd.kernels.library import BlockedRows
    normed = BlockedRows(torch.zeros_like(blocked.data), rows, width, block_rows)
    weight = RNG.normal(size=width).astype(np.float32)
    K.rmsnorm(dev(x), dev(weight), 1e-5, normed)
    as_rows = torch.empty(rows, width, dtype=torch.bfloat16, device=DEVICE)
    K.rmsnorm(dev(x), dev(weight), 1e-5, as_rows)
    assert np.array_equal(host(normed.data)[index], host(as_rows))


def test_embed_rmsnorm_swiglu_argmax_and_their_twins(K, twins):
    table = RNG.normal(size=(331, 96)).astype(np.float32)
    tokens = RNG.integers(0, 331, size=37).astype(np.int32)
    out = torch.empty(37, 96, device=DEVICE)
    K.embed(dev(tokens), dev(table, torch.bfloat16), out)
    assert np.array_equal(host(out), twins.embed(tokens, table, BF16)[1])
    x = RNG.normal(size=(33, 1000)).astype(np.float32) * 2
    w = (1 + 0.3 * RNG.normal(size=1000)).astype(np.float32)
    for out_dtype, code, bound in ((torch.float32, F32, 2e-6), (torch.bfloat16, BF16, 8e-3)):
        got = torch.empty(33, 1000, device=DEVICE, dtype=out_dtype)
        K.rmsnorm(dev(x), dev(w), 1e-5, got)
        assert rel(host(got), twins.rmsnorm(x, w, 1e-5, out_code=code)) < bound
    gate_up = RNG.normal(size=(7, 400)).astype(np.float32) * 3
    for dtype, code, bound in ((torch.float32, F32, 2e-6), (torch.bfloat16, BF16, 8e-3)):
        got = torch.empty(7, 200, device=DEVICE, dtype=dtype)
        K.swiglu(dev(gate_up, dtype), got)
        assert rel(host(got), twins.swiglu(gate_up, code)) < bound
    logits = RNG.normal(size=(5, 10000)).astype(np.float32)
    logits[1, 77] = logits[1, 9000] = 50.0
    logits[3, 5] = np.inf
    tokens_out = torch.empty(5, dtype=torch.int32, device=DEVICE)
    bad = torch.empty(5, dtype=torch.int32, device=DEVICE)
    K.sample(dev(logits), tokens_out, bad)
    want_tokens, want_bad = twins.argmax(logits)
    assert tokens_out.cpu().tolist() == want_tokens.tolist() and bad.cpu().tolist() == want_bad.tolist()


@pytest.mark.parametrize("m,n,k", [(1, 96, 128), (8, 331, 192), (40, 130, 320), (200, 64, 448)])
def test_products_and_their_twin(K, twins, m, n, k):
    a, w = RNG.normal(size=(m, k)).astype(np.float32), RNG.normal(size=(n, k)).astype(np.float32) * 0.1
    got32 = torch.zeros(m, n, device=DEVICE)
    K.gemm(dev(a), dev(w), got32)
    assert rel(host(got32), twins.gemm(a, w)) < 5e-6
    got16 = torch.ones(m, n, device=DEVICE)          # bfloat16 operands (the matrix cores), added into a float32 residual
    K.gemm(dev(a, torch.bfloat16), K.pack_weight(dev(w, torch.bfloat16)), got16, accumulate=True)
    assert rel(host(got16), twins.gemm(a, w, BF16, c=np.ones((m, n), np.float32))) < 5e-6


class Layout:
    def __init__(self, seq_start, n_seqs, max_rows_per_seq, max_position):
        self.seq_start, self.n_seqs, self.max_rows_per_seq, self.max_position = seq_start, n_seqs, max_rows_per_seq, max_position


@pytest.mark.parametrize("dtype,code,head_dim,rot,window", [(torch.float32, F32, 48, 48, 0), (torch.float32, F32, 80, 32, 70),
                                                            (torch.bfloat16, BF16, 64, 64, 0), (torch.bfloat16, BF16, 128, 128, 100),
                                                            (torch.bfloat16, BF16, 48, 0, 0)])
def test_cache_write_and_attention_and_their_twins(K, twins, dtype, code, head_dim, rot, window):
    """Sequences with pasts of 0, 70 and 5 tokens get 9, 1 and 130 more rows in one step: the writing kernel fills
    the same places of the same pages as its twin, and the attention kernel (the generic one, or the matrix-core
    ones for bfloat16 heads in steps of 32) gives what the twin gives over those pages."""
    n_heads, kv_heads, eps = 6, 2, 1e-5
    lengths = [(0, 9), (70, 1), (5, 130)]
    n_pages = 8
    order = K.kv_order(dtype, head_dim)
    assert order == (1 if dtype == torch.bfloat16 and head_dim % 32 == 0 else 0)
    pages = RNG.permutation(n_pages).tolist()
    table = np.zeros((3, 3), np.int32)
    for s, (past, new) in enumerate(lengths):
        for j in range(-(-(past + new) // 64)):
            table[s, j] = pages.pop()
    fused = (n_heads + 2 * kv_heads) * head_dim
    qw = (1 + 0.3 * RNG.normal(size=head_dim)).astype(np.float32)
    kw = (1 + 0.3 * RNG.normal(size=head_dim)).astype(np.float32)
    top = max(past + new for past, new in lengths)
    angles = np.arange(top)[:, None] * (1.0 / 10000.0 ** (2 * np.arange(max(rot, 2) // 2) / max(rot, 2)))[None, :]
    cos, sin = (np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)) if rot else (None, None)
    kind = torch.float32 if code == F32 else torch.bfloat16
    k_dev = torch.zeros(n_pages, kv_heads, 64, head_dim, device=DEVICE, dtype=kind)
    v_dev = torch.zeros(n_pages, kv_heads, head_dim, 64, device=DEVICE, dtype=kind)
    k_twin = v_twin = None
    for phase in (0, 1):
        rows, positions, row_seq, starts = [], [], [], [0]
        for s, (past, new) in enumerate(lengths):
            lo, hi = (0, past) if phase == 0 else (past, past + new)
            rows.append(RNG.normal(size=(hi - lo, fused)).astype(np.float32))
            positions.extend(range(lo, hi))
            row_seq.extend([s] * (hi - lo))
            starts.append(len(positions))
        qkv = np.concatenate(rows)
        q_twin, k_twin, v_twin = twins.qk_norm_rope_cache(qkv, qw, kw, eps, cos, sin, positions, row_seq, table, n_pages, n_heads,
                                                          kv_heads, head_dim, order, code, k_pages=k_twin, v_pages=v_twin)
        q_dev = torch.empty(len(positions), n_heads * head_dim, device=DEVICE, dtype=kind)
        K.qk_norm_rope_cache(dev(qkv, kind), q_dev, dev(qw), dev(kw), eps, None if cos is None else dev(cos),
                             None if sin is None else dev(sin), dev(np.asarray(positions, np.int32)),
                             dev(np.asarray(row_seq, np.int32)), k_dev, v_dev, dev(table), n_heads, kv_heads, head_dim, True,
                             max(positions))
    bound = 2e-6 if code == F32 else 8e-3
    assert rel(host(q_dev), q_twin) < bound
    # the pages, element for element in the library's own order: the values are copies, the keys are within rounding
    k_got, v_got = host(k_dev.reshape(n_pages, kv_heads, -1)), host(v_dev.reshape(n_pages, kv_heads, -1))
    k_want = k_twin if code == F32 else twins_module.from_bf16_bits(k_twin)
    v_want = v_twin if code == F32 else twins_module.from_bf16_bits(v_twin)
    assert np.array_equal(v_got, v_want)
    assert rel(k_got, k_want) < bound
    scale = 1 / math.sqrt(head_dim)
    out = torch.empty_like(q_dev)
    layout = Layout(dev(np.asarray(starts, np.int32)), 3, max(new for _, new in lengths), max(positions))
    K.attention(q_dev, out, k_dev, v_dev, dev(table), dev(np.asarray(row_seq, np.int32)), dev(np.asarray(positions, np.int32)),
                n_heads, kv_heads, head_dim, scale, window, layout=layout)
    want = twins.attention(host(q_dev), k_twin, v_twin, table, row_seq, positions, n_heads, kv_heads, head_dim, scale, window, order, code)
    assert rel(host(out), want) < (1e-5 if code == F32 else 1.2e-2)


def test_the_draws_thresholds_on_rows_made_to_trip_them(K, twins):
    """Rows on which a search for the k-th largest logit or for top-p's threshold digit by digit could go wrong: all
    logits equal (every token ties at every threshold), two values only, logits of both signs around zero and far
    apart, a vocabulary that fills no trip of the draw, k one below the vocabulary, p so small that only the
    largest logit stays, p just below one.  Against the plain twin, row by row."""
    rng = np.random.default_rng(11)
    vocab = 5003
    shapes = [np.full(vocab, 1.25, np.float32),
              np.where(rng.random(vocab) < 0.01, 3.0, -2.0).astype(np.float32),
              (rng.normal(size=vocab) * 1e-3).astype(np.float32),
              (rng.normal(size=vocab) * 40).astype(np.float32),
              np.concatenate([np.full(vocab - 3, -1e30, np.float32), np.asarray([0.5, 0.5, 0.25], np.float32)]),
              (-np.abs(rng.normal(size=vocab)) * 5 - 100).astype(np.float32),
              np.where(rng.random(vocab) < 0.5, np.float32(0.0), np.float32(-0.0)).astype(np.float32)]     # zero and minus zero tie
    settings = [(0, 1.0), (5, 1.0), (vocab - 1, 1.0), (0, 1e-6), (0, 0.999999), (0, 0.5), (40, 0.7), (1, 0.3)]
    logits = np.stack([shape for shape in shapes for _ in settings])
    rows = logits.shape[0]
    top_k = np.asarray([k for _ in shapes for k, _ in settings], np.int32)
    top_p = np.asarray([p for _ in shapes for _, p in settings], np.float32)
    temperature = rng.choice([0.6, 1.0, 1.5], size=rows).astype(np.float32)
    for seed in range(3):
        uniform = np.random.default_rng(seed).random(rows).astype(np.float32)
        tokens, bad = torch.empty(rows, dtype=torch.int32, device=DEVICE), torch.empty(rows, dtype=torch.int32, device=DEVICE)
        K.sample(dev(logits), tokens, bad, temperature=dev(temperature), top_k=dev(top_k), top_p=dev(top_p), uniform=dev(uniform))
        want, want_bad, margin = twins.sample(logits, temperature, uniform, top_k, top_p)
        got = tokens.cpu().numpy()
        assert bad.cpu().tolist() == want_bad.tolist() == [0] * rows
        sure = margin > 1e-5
        assert sure.sum() > 0.8 * rows and np.array_equal(got[sure], want[sure]), (got[sure != (got == want)], want[sure != (got == want)])
    # k = 1 and a tiny p keep the largest logit alone, whatever the uniform number
    alone = [i for i in range(rows) if (top_k[i] == 1 or top_p[i] < 1e-5) and len(set(logits[i].tolist())) > 2]
    assert alone and all(int(got[i]) == int(np.argmax(logits[i])) for i in alone)


def test_a_draw_from_the_whole_distribution_goes_chunk_by_chunk_and_keeps_index_order(K, twins):
    """A draw at a temperature without top-k and top-p is spread over chunks of the row.  Rows made so that a fault of
    that shows: three tokens in three different chunks (one in the ragged last chunk) hold all of the weight, 0.5, 0.3
    and 0.2 of it, and uniform numbers step through [0, 1): the token follows the cumulative weights in index order.
    Then shapes against the plain twin: all logits equal, one chunk far above the others, a very low temperature, a
    greedy row among drawn ones, and a logit that is not finite in a chunk that is not the first."""
    vocab = 4 * 2048 + 808
    assert K.lib.bh_sample_draw_scratch(4, vocab) > 0
    places, shares = [700, 2048 + 1999, 4 * 2048 + 807], [0.5, 0.3, 0.2]
    steps = 200
    logits = np.full((steps, vocab), -1e4, np.float32)
    for place, share in zip(places, shares):
        logits[:, place] = np.log(share)
    uniform = ((np.arange(steps) + 0.5) / steps).astype(np.float32)
    temperature = np.ones(steps, np.float32)
    tokens, bad = torch.empty(steps, dtype=torch.int32, device=DEVICE), torch.empty(steps, dtype=torch.int32, device=DEVICE)
    K.sample(dev(logits), tokens, bad, temperature=dev(temperature), uniform=dev(uniform))
    want = [places[0] if u < 0.5 else places[1] if u < 0.8 else places[2] for u in uniform]
    assert tokens.cpu().tolist() == want and bad.cpu().tolist() == [0] * steps

    rng = np.random.default_rng(23)
    lifted = (rng.normal(size=vocab) * 2).astype(np.float32)
    lifted[3 * 2048:4 * 2048] += 30.0
    shapes = [np.full(vocab, -3.5, np.float32), lifted, (rng.normal(size=vocab) * 3).astype(np.float32),
              (rng.normal(size=vocab) * 1e-3).astype(np.float32), (rng.normal(size=vocab) * 40).astype(np.float32)]
    logits = np.stack([shape for shape in shapes for _ in range(12)])
    rows = logits.shape[0]
    temperature = rng.choice([0.01, 0.3, 1.0, 2.5], size=rows).astype(np.float32)
    temperature[7] = 0.0
    for seed in range(3):
        uniform = np.random.default_rng(seed).random(rows).astype(np.float32)
        tokens, bad = torch.empty(rows, dtype=torch.int32, device=DEVICE), torch.empty(rows, dtype=torch.int32, device=DEVICE)
        K.sample(dev(logits), tokens, bad, temperature=dev(temperature), uniform=dev(uniform))
        want, want_bad, margin = twins.sample(logits, temperature, uniform)
        got = tokens.cpu().numpy()
        assert bad.cpu().tolist() == want_bad.tolist() == [0] * rows
        sure = margin > 1e-5
        assert sure.sum() > 0.8 * rows and np.array_equal(got[sure], want[sure]), (got[sure & (got != want)], want[sure & (got != want)])
        assert int(got[7]) == int(np.argmax(logits[7]))
    spoiled = logits.copy()
    spoiled[3, 2 * 2048 + 5] = np.nan
    spoiled[4, vocab - 1] = np.inf
    K.sample(dev(spoiled), tokens, bad, temperature=dev(temperature), uniform=dev(uniform))
    assert bad.cpu().tolist() == [int(i in (3, 4)) for i in range(rows)]
    assert tokens.cpu().tolist()[3:5] == [-1, -1] and np.array_equal(tokens.cpu().numpy()[5:], got[5:])


def test_a_top_k_draw_goes_through_the_candidates_of_the_rows_chunks(K, twins):
    """With a top-k the row's chunks hand in their own k largest and the draw is made among those.  Rows made for what
    could go wrong there: the k largest all in one chunk (the first, or the ragged last one, which has fewer tokens
    than k), ties at the threshold within a chunk and across chunks (more of them than a chunk has places for sends
    the row down the other path), all logits equal, k of 1, the largest k that goes this way and the first that does
    not, k off in some rows.  The token must be the one that the one-block kernel draws from the whole row, for every
    row, and the plain twin's wherever the target is not at an interval's very end."""
    rng = np.random.default_rng(31)
    vocab = 4 * 2048 + 30
    assert K.lib.bh_sample_top_k_scratch(4, vocab) > 0
    ramp = np.linspace(8.0, -8.0, vocab).astype(np.float32)
    coarse = (np.round(rng.normal(size=vocab) * 4) / 4).astype(np.float32)
    few_ties = (rng.normal(size=vocab) * 3).astype(np.float32)
    few_ties[[5, 2048 + 17, 3 * 2048 + 1, vocab - 2]] = np.sort(few_ties)[-20]      # the 20th largest, in four chunks
    signed_zeros = np.where(rng.random(vocab) < 0.5, np.float32(0.0), np.float32(-0.0)).astype(np.float32)
    signed_zeros[[9, 5000]] = 1.0          # two tokens above a sea of zeros of both signs, which all tie
    shapes = [(rng.normal(size=vocab) * 3).astype(np.float32), ramp, ramp[::-1].copy(), coarse, few_ties,
              np.full(vocab, 0.75, np.float32), np.where(rng.random(vocab) < 0.01, 3.0, -2.0).astype(np.float32), signed_zeros]
    settings = [(1, 1.0), (5, 0.9), (20, 1.0), (40, 0.3), (50, 0.9), (128, 1.0), (129, 0.9), (0, 0.5), (vocab - 1, 1.0)]
    logits = np.stack([shape for shape in shapes for _ in settings])
    rows = logits.shape[0]
    top_k = np.asarray([k for _ in shapes for k, _ in settings], np.int32)
    top_p = np.asarray([p for _ in shapes for _, p in settings], np.float32)
    temperature = rng.choice([0.6, 1.0, 1.5], size=rows).astype(np.float32)
    temperature[3] = 0.0
    on_device = dict(logits=dev(logits), temperature=dev(temperature), top_k=dev(top_k), top_p=dev(top_p))
    for seed in range(4):
        uniform = np.random.default_rng(seed).random(rows).astype(np.float32)
        tokens, bad = torch.empty(rows, dtype=torch.int32, device=DEVICE), torch.empty(rows, dtype=torch.int32, device=DEVICE)
        K.sample(on_device["logits"], tokens, bad, temperature=on_device["temperature"], top_k=on_device["top_k"],
                 top_p=on_device["top_p"] if seed % 2 else None, uniform=dev(uniform))
        whole, whole_bad = torch.empty_like(tokens), torch.empty_like(bad)
        K._check(K.lib.bh_sample(K._ptr(on_device["logits"], "logits"), K._ptr(on_device["temperature"], "temperature"),
                                 K._ptr(on_device["top_k"], "top_k"), K._ptr(on_device["top_p"] if seed % 2 else None, "top_p", None, True),
                                 K._ptr(dev(uniform), "uniform"), K._ptr(whole, "tokens"), K._ptr(whole_bad, "bad"),
                                 K._ptr(None, "scratch", None, True), rows, vocab, K._stream()))
        got = tokens.cpu().numpy()
        assert np.array_equal(got, whole.cpu().numpy())
        want, want_bad, margin = twins.sample(logits, temperature, uniform, top_k, top_p if seed % 2 else None)
        assert bad.cpu().tolist() == want_bad.tolist() == [0] * rows
        sure = margin > 1e-5
        assert sure.sum() > 0.8 * rows and np.array_equal(got[sure], want[sure]), (got[sure & (got != want)], want[sure & (got != want)])
        assert int(got[3]) == int(np.argmax(logits[3]))
    spoiled = logits.copy()
    spoiled[2, 3 * 2048 + 5] = np.nan
    K.sample(dev(spoiled), tokens, bad, temperature=on_device["temperature"], top_k=on_device["top_k"], uniform=dev(uniform))
    assert bad.cpu().tolist() == [int(i == 2) for i in range(rows)] and int(tokens[2]) == -1


def test_a_top_p_draw_goes_through_the_candidates_where_its_share_lies_within_them(K, twins):
    """A top-p without a top-k: the chunks hand in their 128 largest and their tokens' weight, and the row's block stays
    among the candidates if top-p's share of the whole row's weight lies within the row's 128 largest, else it goes
    through the whole row.  Rows on both sides of that (peaked ones, flat ones, one whose share ends exactly around the
    128th largest token, all logits equal, two values), rows with a top-k as well and rows with no filter in the same call.
    The token must be the one-block kernel's for every row, and the plain twin's wherever the target is not at an
    interval's very end."""
    rng = np.random.default_rng(37)
    vocab = 5 * 2048 + 100
    base = rng.normal(size=vocab).astype(np.float32)
    edge = np.full(vocab, -30.0, np.float32)             # 256 equal tokens carry all the weight: p = 0.5 ends at the 128th
    edge[rng.choice(vocab, size=256, replace=False)] = 2.0
    shapes = [base * 12, base * 6, base * 3, base, base * 0.05, edge, np.full(vocab, -1.5, np.float32),
              np.where(rng.random(vocab) < 0.002, 4.0, -4.0).astype(np.float32)]
    settings = [(0, 0.9), (0, 0.5), (0, 0.1), (0, 0.999), (0, 1.0), (20, 0.9), (50, 1.0), (200, 0.7)]
    logits = np.stack([shape for shape in shapes for _ in settings])
    rows = logits.shape[0]
    top_k = np.asarray([k for _ in shapes for k, _ in settings], np.int32)
    top_p = np.asarray([p for _ in shapes for _, p in settings], np.float32)
    temperature = rng.choice([0.6, 1.0, 1.5], size=rows).astype(np.float32)
    temperature[9] = 0.0
    device = dict(logits=dev(logits), temperature=dev(temperature), top_k=dev(top_k), top_p=dev(top_p))
    for seed in range(4):
        with_k = seed % 2 == 1
        uniform = np.random.default_rng(seed).random(rows).astype(np.float32)
        tokens, bad = torch.empty(rows, dtype=torch.int32, device=DEVICE), torch.empty(rows, dtype=torch.int32, device=DEVICE)
        uniform_device = dev(uniform)
        for some in (slice(0, 32), slice(32, rows)):      # (a top-p alone goes this way for up to 64 rows a call; here in two calls)
            K.sample(device["logits"][some], tokens[some], bad[some], temperature=device["temperature"][some],
                     top_k=device["top_k"][some] if with_k else None, top_p=device["top_p"][some], uniform=uniform_device[some])
        whole, whole_bad = torch.empty_like(tokens), torch.empty_like(bad)
        K._check(K.lib.bh_sample(K._ptr(device["logits"], "logits"), K._ptr(device["temperature"], "temperature"),
                                 K._ptr(device["top_k"] if with_k else None, "top_k", None, True), K._ptr(device["top_p"], "top_p"),
                                 K._ptr(dev(uniform), "uniform"), K._ptr(whole, "tokens"), K._ptr(whole_bad, "bad"),
                                 K._ptr(None, "scratch", None, True), rows, vocab, K._stream()))
        got = tokens.cpu().numpy()
        assert np.array_equal(got, whole.cpu().numpy()), np.nonzero(got != whole.cpu().numpy())
        want, want_bad, margin = twins.sample(logits, temperature, uniform, top_k if with_k else None, top_p)
        assert bad.cpu().tolist() == want_bad.tolist() == [0] * rows
        sure = margin > 1e-5
        assert sure.sum() > 0.7 * rows and np.array_equal(got[sure], want[sure]), (got[sure & (got != want)], want[sure & (got != want)])
        assert int(got[9]) == int(np.argmax(logits[9]))
    spoiled = logits.copy()
    spoiled[2, 3 * 2048 + 5] = np.inf
    K.sample(dev(spoiled[:32]), tokens[:32], bad[:32], temperature=device["temperature"][:32], top_p=device["top_p"][:32],
             uniform=uniform_device[:32])
    assert bad[:32].cpu().tolist() == [int(i == 2) for i in range(32)] and int(tokens[2]) == -1
    assert K.lib.bh_sample_top_k_scratch(32, vocab) > 0


@pytest.mark.parametrize("vocab", [50, 1000, 4133, 151936])
def test_the_draw_and_its_twin(K, twins, vocab):
    """Temperature, top-k and top-p draws of the kernel against the plain twin's, row by row: the same token wherever the
    draw's target lies further from the ends of its token's interval than float32 sums can move it."""
    rng = np.random.default_rng(vocab)
    rows = 96
    logits = (rng.normal(size=(rows, vocab)) * 2.5).astype(np.float32)
    logits[5, 7] = logits[5, 9]                    # ties at a threshold are kept
    temperature = rng.choice([0.0, 0.5, 0.8, 1.0, 1.7], size=rows).astype(np.float32)
    uniform = rng.random(rows).astype(np.float32)
    for top_k, top_p in ((None, None), (rng.choice([0, 1, 5, 40, vocab], size=rows).astype(np.int32), None),
                         (None, rng.choice([1.0, 0.9, 0.5, 0.05], size=rows).astype(np.float32)),
                         (rng.choice([0, 3, 40], size=rows).astype(np.int32), rng.choice([1.0, 0.8, 0.3], size=rows).astype(np.float32))):
        tokens, bad = torch.empty(rows, dtype=torch.int32, device=DEVICE), torch.empty(rows, dtype=torch.int32, device=DEVICE)
        K.sample(dev(logits), tokens, bad, temperature=dev(temperature), top_k=None if top_k is None else dev(top_k),
                 top_p=None if top_p is None else dev(top_p), uniform=dev(uniform))
        want, want_bad, margin = twins.sample(logits, temperature, uniform, top_k, top_p)
        got = tokens.cpu().numpy()
        assert bad.cpu().tolist() == want_bad.tolist() == [0] * rows
        sure = margin > 1e-5      # (of 151,936 tokens most have intervals of that size: fewer rows are sure there)
        assert sure.sum() > (0.9 if vocab < 10000 else 0.6) * rows and np.array_equal(got[sure], want[sure])
        assert len(set(want.tolist())) > rows // 4
