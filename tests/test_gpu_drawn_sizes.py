"""The kernels' public entry points at sizes drawn from a seeded generator, so that no dispatch rule is tested only at
the sizes someone thought of: products through every path the library chooses between (rows from 1 to 1,100, widths
in steps of 16, K in steps of 64, each output mode), ragged attention steps (head sizes 32 to 256, any grouping, a
window or none, new rows on top of a past), and the many-row cache write (bit for bit, with nothing else touched).
The draws are fixed by their seeds; each case prints its sizes before it runs."""

import math
import random

import numpy as np
import pytest
import torch

import test_gpu_kernels as T
from beholdd.kernels.library import BlockedRows, NormedRows
from beholdd.parts.base import NormRequest

pytestmark = pytest.mark.gpu
DEVICE = "cuda:0"


@pytest.fixture(scope="module")
def K():
    from beholdd.kernels import HipKernels
    return HipKernels(DEVICE)


def rel(got, want):
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30))


def rows_of(K, out):
    return K.from_blocked(out) if isinstance(out, BlockedRows) else out


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_products_at_drawn_sizes(K, seed):
    rng = random.Random(seed)
    for case in range(24):
        m = rng.choice([rng.randint(1, 70), rng.randint(1, 300), rng.randint(250, 1100)])
        n = 16 * rng.choice([rng.randint(1, 40), rng.randint(30, 300)])
        k = 64 * rng.choice([rng.randint(1, 8), rng.randint(2, 40), rng.randint(30, 70)])
        mode = rng.choice(["bf16", "f32", "accumulate", "accumulate_then_norm", "swiglu", "swiglu_to_blocks", "norm_ahead"])
        packed = rng.random() < 0.85
        print(f"seed {seed} case {case}: m={m} n={n} k={k} {mode} packed={packed}", flush=True)
        g = torch.Generator().manual_seed(1000 * seed + case)
        a = torch.randn(m, k, generator=g).to(torch.bfloat16)
        w = (torch.randn(2 * n if mode.startswith("swiglu") else n, k, generator=g) * 0.05).to(torch.bfloat16)
        w_dev = K.pack_weight(w.to(DEVICE)) if packed else w.to(DEVICE)
        want = a.double() @ w.double().t()
        f32_bound = 8 * math.sqrt(k) * 2.0 ** -24
        if mode == "bf16":
            out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEVICE)
            K.gemm(a.to(DEVICE), w_dev, out)
            assert rel(out, want) < 6e-3
        elif mode == "f32":
            out = torch.full((m, n), float("nan"), dtype=torch.float32, device=DEVICE)
            K.gemm(a.to(DEVICE), w_dev, out)
            assert rel(out, want) < f32_bound
        elif mode.startswith("accumulate"):
            base = torch.randn(m, n, generator=g)
            out = base.to(DEVICE).clone()
            weight = 1 + 0.3 * torch.randn(n, generator=g)
            request = NormRequest(weight.to(DEVICE), 1e-6) if mode == "accumulate_then_norm" else None
            prepared = K.gemm(a.to(DEVICE), w_dev, out, accumulate=True, then_norm=request)
            total = want + base.double()
            assert rel(out, total) < f32_bound
            normed = total * torch.rsqrt((total ** 2).mean(-1, keepdim=True) + 1e-6) * weight.double()
            if isinstance(prepared, NormedRows):                     # the norm's rows came with the product, but for each row's factor
                factor = torch.rsqrt(prepared.ss.double().sum(-1, keepdim=True).cpu() / n + 1e-6)
                assert rel(rows_of(K, prepared.rows).double().cpu() * factor, normed) < 1e-2
            elif isinstance(prepared, (BlockedRows, torch.Tensor)):  # or whole
                assert rel(rows_of(K, prepared), normed) < 1e-2
        elif mode.startswith("swiglu"):
            gate, up = want[:, :n], want[:, n:]
            activated = gate / (1 + torch.exp(-gate)) * up
            if mode == "swiglu_to_blocks" and n % 32 == 0:
                out = K.new_rows(m, n, torch.bfloat16, reader_outputs=rng.choice([n, 4096]), reader_swiglu=False, reader_packed=True)
            else:
                out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEVICE)
            K.gemm_swiglu(a.to(DEVICE), w_dev, out)
            assert rel(rows_of(K, out), activated) < 8e-3
        else:      # a norm's output in whatever form the library hands the product that reads it
            x = torch.randn(m, k, generator=g)
            weight = 1 + 0.3 * torch.randn(k, generator=g)
            normed = x.double() * torch.rsqrt((x.double() ** 2).mean(-1, keepdim=True) + 1e-6) * weight.double()
            normed_dev = K.new_rows(m, k, torch.bfloat16, reader_outputs=n, reader_swiglu=False, reader_packed=packed)
            K.rmsnorm(x.to(DEVICE), weight.to(DEVICE), 1e-6, normed_dev)
            out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEVICE)
            K.gemm(normed_dev, w_dev, out)
            assert rel(out, normed @ w.double().t()) < 1.2e-2


@pytest.mark.parametrize("seed", [1, 2])
def test_attention_at_drawn_sizes(K, seed):
    rng = random.Random(seed)
    for case in range(16):
        kv_heads = rng.choice([1, 2, 4, 8])
        n_heads = kv_heads * rng.choice([1, 2, 4, 8])
        head_dim = rng.choice([32, 64, 96, 128, 128, 128, 160, 256])
        window = rng.choice([0, 0, rng.randint(1, 300)])
        n_seqs = rng.randint(1, 6)
        longest = 600 if rng.random() < 0.6 else 40
        news = [rng.randint(1, longest) for _ in range(n_seqs)]
        pasts = [rng.choice([0, rng.randint(0, 300)]) for _ in range(n_seqs)]
        print(f"seed {seed} case {case}: heads {n_heads}/{kv_heads} of {head_dim}, window {window}, new {news}, past {pasts}", flush=True)
        lengths = [p + n for p, n in zip(pasts, news)]
        kp, vp, table, keys, values = T.make_cache(n_seqs, lengths, kv_heads, head_dim, torch.bfloat16, seed=100 * seed + case)
        for s, n in enumerate(lengths):       # what lies behind a sequence's end in its last page must not matter
            if n % T.PAGE:
                page = int(table[s, (n - 1) // T.PAGE])
                kp[page, :, n % T.PAGE:, :] = float("nan")
                vp[page, :, :, n % T.PAGE:] = float("nan")
        g = torch.Generator().manual_seed(100 * seed + case)
        n_rows = sum(news)
        q = torch.randn(n_rows, n_heads * head_dim, generator=g).to(torch.bfloat16)
        positions = torch.tensor([p + t for p, n in zip(pasts, news) for t in range(n)], dtype=torch.int32)
        row_seq = torch.tensor([s for s, n in enumerate(news) for _ in range(n)], dtype=torch.int32)
        starts = torch.tensor(np.concatenate([[0], np.cumsum(news)]), dtype=torch.int32)
        out = torch.full((n_rows, n_heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEVICE)
        scale = 1 / math.sqrt(head_dim)
        K.attention(T.dev(q), out, *T.stored(K, kp, vp), T.dev(table), T.dev(row_seq), T.dev(positions), n_heads, kv_heads,
                    head_dim, scale, window, layout=T.Layout(False, T.dev(starts), n_seqs, max(news), max(lengths) - 1))
        for s in range(n_seqs):
            r = slice(int(starts[s]), int(starts[s + 1]))
            want = T.attention_reference_rows(q[r], keys[s], values[s], positions[r].long(), n_heads, kv_heads, head_dim, scale, window)
            assert T.rel(out[r], want) < 1.2e-2, f"sequence {s}"


@pytest.mark.parametrize("seed", [1, 2])
def test_cache_write_of_many_rows_at_drawn_sizes(K, seed):
    """Without norm and rotation the kernel only moves values: queries, keys and values must arrive bit for bit, and
    every other element of the pages must keep what it held."""
    rng = random.Random(seed)
    page_size = T.PAGE
    for case in range(20):
        kv_heads = rng.choice([1, 2, 3, 4, 8])
        n_heads = kv_heads * rng.choice([1, 2, 4])
        head_dim = rng.choice([64, 128, 256])
        n_seqs = rng.randint(1, 6)
        news = [rng.randint(1, 120) for _ in range(n_seqs)]
        if sum(news) < 64:
            news[0] += 64
        pasts = [rng.randint(0, 70) for _ in range(n_seqs)]
        write_kv = rng.random() < 0.8
        print(f"seed {seed} case {case}: heads {n_heads}/{kv_heads} of {head_dim}, new {news}, past {pasts}, write {write_kv}", flush=True)
        pages_per = [-(-(p + n) // page_size) for p, n in zip(pasts, news)]
        n_pages = sum(pages_per) + 2
        order = list(range(n_pages))
        rng.shuffle(order)
        table = torch.zeros(n_seqs, max(pages_per), dtype=torch.int32)
        for s in range(n_seqs):
            for i in range(pages_per[s]):
                table[s, i] = order.pop()
        g = torch.Generator().manual_seed(100 * seed + case)
        n_rows = sum(news)
        qkv = torch.randn(n_rows, (n_heads + 2 * kv_heads) * head_dim, generator=g).to(torch.bfloat16)
        positions = torch.tensor([p + t for p, n in zip(pasts, news) for t in range(n)], dtype=torch.int32)
        row_seq = torch.tensor([s for s, n in enumerate(news) for _ in range(n)], dtype=torch.int32)
        kp = torch.full((n_pages, kv_heads, page_size, head_dim), 768.0).to(torch.bfloat16)
        vp = torch.full((n_pages, kv_heads, head_dim, page_size), 768.0).to(torch.bfloat16)
        kp_dev, vp_dev = T.stored(K, kp, vp)
        q_out = torch.empty(n_rows, n_heads * head_dim, dtype=torch.bfloat16, device=DEVICE)
        K.qk_norm_rope_cache(T.dev(qkv), q_out, None, None, 0.0, None, None, T.dev(positions), T.dev(row_seq), kp_dev, vp_dev,
                             T.dev(table), n_heads, kv_heads, head_dim, write_kv, int(positions.max()))
        k_rows, v_rows = T.as_rows(K, kp_dev, vp_dev)
        want_k, want_v = kp.clone(), vp.clone()
        if write_kv:
            for row in range(n_rows):
                pos, seq = int(positions[row]), int(row_seq[row])
                page = int(table[seq, pos // page_size])
                want_k[page, :, pos % page_size] = qkv[row, n_heads * head_dim:(n_heads + kv_heads) * head_dim].reshape(kv_heads, head_dim)
                want_v[page, :, :, pos % page_size] = qkv[row, (n_heads + kv_heads) * head_dim:].reshape(kv_heads, head_dim)
        assert torch.equal(q_out.cpu(), qkv[:, :n_heads * head_dim])
        assert torch.equal(k_rows.cpu(), want_k) and torch.equal(v_rows.cpu(), want_v)


def test_decode_attention_at_drawn_batches_and_lengths(K):
    """One new row per sequence over caches of drawn lengths: the number of key splits follows the batch, the heads
    and the longest cache, so batches and lengths that nobody picked go through it, with NaN behind every
    sequence's end."""
    rng = random.Random(4)
    seen_splits = set()
    for case in range(10):
        kv_heads = rng.choice([1, 2, 4, 8])
        n_heads = kv_heads * rng.choice([1, 2, 4, 8])
        head_dim = rng.choice([64, 96, 128, 128, 256])
        n_seqs = rng.choice([rng.randint(1, 8), rng.randint(5, 24), rng.randint(25, 70)])
        longest = rng.choice([300, 1200, 2600])
        lengths = [rng.randint(1, max(1, min(longest, 24000 // n_seqs))) for _ in range(n_seqs)]
        window = rng.choice([0, 0, rng.randint(1, 500)])
        splits = K.lib.bh_attention_bf16_splits(n_seqs, 1, n_heads, kv_heads, max(lengths) - 1)
        seen_splits.add(splits)
        print(f"case {case}: heads {n_heads}/{kv_heads} of {head_dim}, window {window}, {n_seqs} sequences up to {max(lengths)}, "
              f"{splits} splits", flush=True)
        kp, vp, table, keys, values = T.make_cache(n_seqs, lengths, kv_heads, head_dim, torch.bfloat16, seed=case)
        for s, n in enumerate(lengths):
            if n % T.PAGE:
                page = int(table[s, (n - 1) // T.PAGE])
                kp[page, :, n % T.PAGE:, :] = float("nan")
                vp[page, :, :, n % T.PAGE:] = float("nan")
        g = torch.Generator().manual_seed(case)
        q = torch.randn(n_seqs, n_heads * head_dim, generator=g).to(torch.bfloat16)
        positions = torch.tensor([n - 1 for n in lengths], dtype=torch.int32)
        row_seq = torch.arange(n_seqs, dtype=torch.int32)
        out = torch.full((n_seqs, n_heads * head_dim), float("nan"), dtype=torch.bfloat16, device=DEVICE)
        scale = 1 / math.sqrt(head_dim)
        layout = T.Layout(True, T.dev(torch.arange(n_seqs + 1, dtype=torch.int32)), n_seqs, 1, max(lengths) - 1)
        K.attention(T.dev(q), out, *T.stored(K, kp, vp), T.dev(table), T.dev(row_seq), T.dev(positions), n_heads, kv_heads,
                    head_dim, scale, window, layout=layout)
        for s, n in enumerate(lengths):
            want = T.attention_reference(q[s].reshape(n_heads, head_dim), keys[s], values[s], n - 1, n_heads, kv_heads,
                                         head_dim, scale, window)
            assert T.rel(out[s].reshape(n_heads, head_dim), want) < 1.2e-2, (s, n)
    assert len(seen_splits) >= 3, seen_splits
