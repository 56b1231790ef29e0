"""The engine on the GPU against the plain implementation, in float32 and in bfloat16:
every request alone and whole; with its last 32 tokens one by one; in batches of unequal
lengths whose shorter requests end earlier, one batch after another so that slots and pages are
used again; long decoding; the first tokens of a sequence; generation through the entry
point; trace replay as a program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import schedules

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# float32: the acceptance bound.  bfloat16: activations carry 8 bits of mantissa (half an ulp is
# 2^-9 = 0.002 of a value) through a dozen roundings per layer; the bound is on max|diff| / max|logit|.
TOLERANCE = {"float32": 1e-4, "bfloat16": 2e-2}

LENGTHS = {"A": [5, 11, 17, 70, 33, 128], "B": [1, 7, 23, 40, 90, 200, 64], "C": [3, 65, 130, 400, 31],
           "D": [2, 50, 129, 300], "E": [4, 66, 150]}


def engine_for(folder, dtype, max_tokens=4096):
    from beholdd.engine import Engine
    return Engine(folder, dtype=dtype, max_tokens=max_tokens)


@pytest.fixture(scope="module")
def expected(model_dirs):
    cache = {}

    def get(name):
        if name not in cache:
            folder = model_dirs(name, "bfloat16")
            cfg, weights = plain.load_plain(folder)
            requests = schedules.random_requests(cfg.vocab, LENGTHS[name], seed=11)
            cache[name] = (folder, requests, [plain.forward_logits(cfg, weights, r) for r in requests])
        return cache[name]

    return get


def check(label, got, want, tolerance):
    for index, (g, e) in enumerate(zip(got, want)):
        assert g.shape == e.shape, (label, index, g.shape, e.shape)
        assert np.isfinite(g).all(), (label, index)
        error = schedules.relative_error(g, e)
        if error >= tolerance:
            per_row = np.abs(g.astype(np.float64) - e).max(axis=1) / np.abs(e).max()
            first = int(np.argmax(per_row >= tolerance))
            pytest.fail(f"{label}: request {index} (length {len(g)}): error {error:.3e} >= {tolerance}; "
                        f"first wrong position {first}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_every_cut_matches_the_plain_implementation(expected, name, dtype):
    folder, requests, want = expected(name)
    engine = engine_for(folder, dtype)
    tolerance = TOLERANCE[dtype]
    whole = schedules.whole(engine, requests)
    check("whole", whole, want, tolerance)
    tail = schedules.tail_one_by_one(engine, requests, tail=32)
    check("last 32 one by one", tail, want, tolerance)
    for batch_size in (3, len(requests)):
        batched = schedules.batches(engine, requests, batch_size=batch_size)
        check(f"batches of {batch_size}", batched, want, tolerance)
    in_portions = schedules.portions(engine, requests)
    check("portions", in_portions, want, tolerance)
    # the cuts agree with each other more closely than with another implementation
    check("tail vs whole", tail, whole, tolerance / 2)
    check("batches vs whole", batched, whole, tolerance / 2)
    check("portions vs whole", in_portions, whole, tolerance / 2)
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == [] and engine.cache.free_page_count() == engine.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_batches_of_many_sequences(model_dirs, dtype):
    """Twenty-odd and forty sequences decode together: steps of 17 to 64 rows take other matrix-product
    kernels than steps of a few rows do, also inside the replayed graphs.  Configuration D has the sizes
    that let every fast path run (widths in multiples of 64, head size 128)."""
    folder = model_dirs("D", "bfloat16")
    cfg, weights = plain.load_plain(folder)
    lengths = [5 + (7 * i) % 23 for i in range(40)]
    requests = schedules.random_requests(cfg.vocab, lengths, seed=3)
    want = [plain.forward_logits(cfg, weights, r) for r in requests]
    engine = engine_for(folder, dtype, max_tokens=8192)
    for batch_size in (23, 40):
        got = schedules.batches(engine, requests, batch_size=batch_size, prompt_fraction=0.4)
        check(f"batches of {batch_size}", got, want, TOLERANCE[dtype])
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == []


# (layers, hidden, query heads, kv heads, feed-forward width, prompt lengths)
LARGE_SHAPES = {"8b": (2, 4096, 32, 8, 12288, [70, 9, 131, 300]), "14b": (1, 5120, 40, 8, 17408, [70, 9, 131]),
                "32b": (1, 5120, 64, 8, 25600, [70, 9, 131]),
                # narrower layers of the same make: other counts of weight blocks per compute unit, other tile plans
                "w1024": (2, 1024, 16, 8, 3072, [70, 9, 131]), "w2048": (2, 2048, 16, 8, 6144, [70, 9, 131]),
                "w2560": (1, 2560, 32, 8, 9728, [70, 9, 131, 300])}


@pytest.fixture(scope="module")
def large_expected(tmp_path_factory):
    """Per shape: the model folder, the requests and the plain implementation's logits, made once."""
    import beholdd
    cache = {}

    def get(shape):
        if shape not in cache:
            layers, hidden, heads, kv_heads, intermediate, lengths = LARGE_SHAPES[shape]
            config = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": layers, "hidden_size": hidden,
                      "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": 128,
                      "intermediate_size": intermediate, "vocab_size": 1000, "rope_theta": 1000000.0,
                      "rms_norm_eps": 1e-6, "max_position_embeddings": 8192, "tie_word_embeddings": False}
            folder = str(tmp_path_factory.mktemp(f"layers_{shape}"))
            beholdd.write_random_model(folder, config, seed=1, dtype="bfloat16")
            cfg, weights = plain.load_plain(folder)
            requests = schedules.random_requests(cfg.vocab, lengths, seed=5)
            many = schedules.random_requests(cfg.vocab, [3 + i % 9 for i in range(24)], seed=6)
            cache[shape] = (folder, requests, [plain.forward_logits(cfg, weights, r) for r in requests],
                            many, [plain.forward_logits(cfg, weights, r) for r in many])
        return cache[shape]

    return get


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("shape", ["8b", "14b", "32b", "w1024", "w2048", "w2560"])
def test_layers_of_the_large_models_sizes(large_expected, shape, dtype):
    """The layer sizes of Qwen3-8B, 14B and 32B (five and eight query heads per kv head, heads that do not
    add up to the width) in one or two layers with a small vocabulary: the kernels at the shapes they are
    tuned for (steps of 1, 9, 24, 70, 131 and 300 rows take different matrix-product kernels and tile
    shapes), whole, token by token and in batches, against the plain implementation."""
    folder, requests, want, many, want_many = large_expected(shape)
    engine = engine_for(folder, dtype, max_tokens=4096)
    check("whole", schedules.whole(engine, requests), want, TOLERANCE[dtype])
    check("last 8 one by one", schedules.tail_one_by_one(engine, requests, tail=8), want, TOLERANCE[dtype])
    check("batch", schedules.batches(engine, requests[:3], batch_size=3, prompt_fraction=0.9), want[:3], TOLERANCE[dtype])
    check("24 together", schedules.batches(engine, many, batch_size=24, prompt_fraction=0.5), want_many, TOLERANCE[dtype])


def test_prompts_of_many_rows(large_expected):
    """Steps of 400 to 2,200 rows at the Qwen3-8B layer sizes, where the bfloat16 products go to the kernel whose
    wave groups take turns (a tile of its own, K in parts, the finishing kernel that also finishes the norm):
    three prompts in one step and each alone, against the float32 engine, which the test above holds to
    the plain implementation at these sizes."""
    folder = large_expected("8b")[0]
    requests = schedules.random_requests(1000, [700, 1100, 400], seed=9)
    engine32 = engine_for(folder, "float32", max_tokens=4096)
    want = schedules.whole(engine32, requests)
    del engine32
    engine = engine_for(folder, "bfloat16", max_tokens=4096)
    alone = schedules.whole(engine, requests)
    check("each alone", alone, want, TOLERANCE["bfloat16"])
    together = schedules.batches(engine, requests, batch_size=3, prompt_fraction=1.0)
    check("one step of 2,200 rows", together, want, TOLERANCE["bfloat16"])
    check("together against alone", together, alone, TOLERANCE["bfloat16"] / 2)


@pytest.mark.parametrize("batch", [1, 8, 24])
def test_every_product_gets_its_rows_the_way_it_reads_them(large_expected, batch):
    """At the Qwen3-8B layer sizes the products of a prompt of 1,500 rows and of decode steps of 1, 8 and 24
    sequences read their activations from blocks.  Every kernel before them knows its reader and writes the blocks
    itself: the binding's regrouping kernel, which would make up for a part that does not, never runs."""
    from beholdd.engine import StepEntry
    folder = large_expected("8b")[0]
    engine = engine_for(folder, "bfloat16", max_tokens=4096)
    kernels, calls = engine.kernels, []
    to_blocked, from_blocked, new_rows = kernels.to_blocked, kernels.from_blocked, kernels.new_rows
    kinds = set()

    def watched_new_rows(*args, **kwargs):
        out = new_rows(*args, **kwargs)
        kinds.add(getattr(out, "block_rows", 0))
        return out

    kernels.to_blocked = lambda *a, **k: (calls.append("to_blocked"), to_blocked(*a, **k))[1]
    kernels.from_blocked = lambda *a, **k: (calls.append("from_blocked"), from_blocked(*a, **k))[1]
    kernels.new_rows = watched_new_rows
    try:
        requests = schedules.random_requests(1000, [1500 if i == 0 else 20 + i for i in range(batch)], seed=40)
        slots = [engine.alloc_slot() for _ in requests]
        engine.step([StepEntry(s, r[:-2], [len(r) - 3]) for s, r in zip(slots, requests)])
        assert 16 in kinds                                   # the prompt step's products of many rows
        kinds.clear()
        for back in (2, 1):                                  # the first decode step runs as it is, the second is captured
            engine.step([StepEntry(s, [r[-back]], [0]) for s, r in zip(slots, requests)])
        assert kinds == {8 if batch <= 8 else 16, 0}         # 0: matrices that no product reads (queries for the attention)
        assert calls == []
    finally:
        kernels.to_blocked, kernels.from_blocked, kernels.new_rows = to_blocked, from_blocked, new_rows
        for slot in slots:
            engine.free_slot(slot)


def _prompt_then_one_by_one(engine, tokens, tail, keep):
    """The first len - tail tokens in one step (the logits of its last `keep` rows wanted), the rest one by one."""
    from beholdd.engine import StepEntry
    cut = len(tokens) - tail
    slot = engine.alloc_slot()
    rows = [engine.step([StepEntry(slot, tokens[:cut], list(range(cut - keep, cut)))]).float().cpu().numpy()]
    for token in tokens[cut:]:
        rows.append(engine.step([StepEntry(slot, [token], [0])]).float().cpu().numpy())
    engine.free_slot(slot)
    return np.concatenate(rows)


def test_the_benchmark_context_at_the_large_layer_sizes(large_expected):
    """Where the benchmark runs: the Qwen3-8B layer sizes (two layers, a small vocabulary) at a context of
    8,100 tokens, the prompt whole and the last 32 tokens one by one through the captured graphs (127 pages, the
    keys split over workgroups); and eight requests of 256 to 1,024 tokens decoding 64 tokens together.  bfloat16
    against the float32 engine, which test_layers_of_the_large_models_sizes holds to the plain implementation at
    these sizes, and which is held to itself here: whole against one by one."""
    from beholdd.engine import StepEntry
    folder = large_expected("8b")[0]
    long_one = schedules.random_requests(1000, [8100], seed=31)[0]
    lengths = [256, 1024, 700, 333, 512, 961, 640, 449]
    batch = schedules.random_requests(1000, [n + 64 for n in lengths], seed=32)
    got = {}
    for dtype in ("float32", "bfloat16"):
        engine = engine_for(folder, dtype, max_tokens=8192)
        long_rows = _prompt_then_one_by_one(engine, long_one, tail=32, keep=4)
        if dtype == "float32":
            slot = engine.alloc_slot()
            whole = engine.step([StepEntry(slot, long_one, list(range(8100 - 36, 8100)))]).float().cpu().numpy()
            engine.free_slot(slot)
            check("float32 whole against one by one", [long_rows], [whole], TOLERANCE["float32"] / 2)
        slots = [engine.alloc_slot() for _ in batch]
        rows = [engine.step([StepEntry(s, r[:n], [n - 1]) for s, r, n in zip(slots, batch, lengths)]).float().cpu().numpy()]
        for step in range(64):
            rows.append(engine.step([StepEntry(s, [r[n + step]], [0]) for s, r, n in zip(slots, batch, lengths)])
                        .float().cpu().numpy())
        for slot in slots:
            engine.free_slot(slot)
        if dtype == "bfloat16":
            assert engine.graphs is not None and len(engine.graphs.graphs) >= 2
        engine.cache.check_invariants()
        got[dtype] = (long_rows, np.stack(rows, axis=1))       # [request, step, vocab]
        del engine
    check("8,100 tokens", [got["bfloat16"][0]], [got["float32"][0]], TOLERANCE["bfloat16"])
    check("batch of 8", list(got["bfloat16"][1]), list(got["float32"][1]), TOLERANCE["bfloat16"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_float32_storage_and_slot_reuse_in_a_small_cache(model_dirs, dtype):
    """Weights stored in 32-bit; a cache of three pages, so every request runs in pages and slots
    that earlier requests used."""
    folder = model_dirs("B", "float32")
    cfg, weights = plain.load_plain(folder)
    requests = schedules.random_requests(cfg.vocab, [100, 64, 130, 1, 65], seed=4)
    want = [plain.forward_logits(cfg, weights, r) for r in requests]
    engine = engine_for(folder, dtype, max_tokens=192)
    assert engine.cache.n_pages == 3
    check("whole", schedules.whole(engine, requests), want, TOLERANCE[dtype])
    check("tail", schedules.tail_one_by_one(engine, requests, tail=32), want, TOLERANCE[dtype])
    check("pairs", schedules.batches(engine, [requests[1], requests[3], requests[4], requests[3]], batch_size=2),
          [want[1], want[3], want[4], want[3]], TOLERANCE[dtype])      # 64 + 1, then 65 + 1 tokens: 2, then 3 pages
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(model_dirs, dtype):
    """Ten prompt tokens, then 500 tokens one by one (several pages, several key chunks)."""
    folder = model_dirs("C", "bfloat16")
    cfg, weights = plain.load_plain(folder)
    tokens = schedules.random_requests(cfg.vocab, [510], seed=21)[0]
    want = plain.forward_logits(cfg, weights, tokens)
    engine = engine_for(folder, dtype)
    got = schedules.tail_one_by_one(engine, [tokens], tail=500)[0]
    check("long decoding", [got], [want], TOLERANCE[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens_of_a_sequence(model_dirs, name, dtype):
    folder = model_dirs(name, "bfloat16")
    cfg, weights = plain.load_plain(folder)
    engine = engine_for(folder, dtype)
    for length in (1, 2, 3):
        tokens = schedules.random_requests(cfg.vocab, [length], seed=length)[0]
        want = plain.forward_logits(cfg, weights, tokens)
        check(f"whole {length}", schedules.whole(engine, [tokens]), [want], TOLERANCE[dtype])
        check(f"one by one {length}", schedules.tail_one_by_one(engine, [tokens], tail=length), [want], TOLERANCE[dtype])


def test_capture_is_safe_from_the_garbage_collector(model_dirs):
    """No garbage collection runs while a stream is capturing (freeing another engine's graphs there is
    refused by the runtime), and an engine that nobody holds is freed at once, with no collection."""
    import gc
    import weakref
    from beholdd.engine import Engine, StepEntry
    engine = Engine(model_dirs("A", "bfloat16"), dtype="bfloat16", max_tokens=256)
    seen, forward = [], engine.model.forward

    def watched(*args, **kwargs):
        seen.append((torch.cuda.is_current_stream_capturing(), gc.isenabled()))
        return forward(*args, **kwargs)

    engine.model.forward = watched
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, [1, 2, 3], [2])])
    engine.step([StepEntry(slot, [4], [0])])
    engine.step([StepEntry(slot, [5], [0])])
    assert gc.isenabled()
    assert (True, False) in seen and not any(capturing and collecting for capturing, collecting in seen), seen
    engine.model.forward = forward
    del watched, forward
    alive = weakref.ref(engine)
    del engine
    assert alive() is None


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(model_dirs, dtype):
    """Decode steps replayed from captured HIP graphs against the same steps launched one kernel at
    a time: every replay is checked, with other work (a prefill of another request, a sampling
    kernel, synchronisations) between the replays, across a page boundary, across a change of the
    batch and across the page-table bucket (1,024 tokens) that makes a new graph."""
    from beholdd.engine import Engine, StepEntry
    folder = model_dirs("D", "bfloat16")
    graphed = Engine(folder, dtype=dtype, max_tokens=4096)
    eager = Engine(folder, dtype=dtype, max_tokens=4096, use_graphs=False)
    assert graphed.graphs is not None and eager.graphs is None and graphed.model.graph_safe
    requests = schedules.random_requests(1500, [1040, 60, 1075], seed=17)
    prompts = [990, 30, 1]
    worst = 0.0
    for engine in (graphed, eager):
        engine.slots = [engine.alloc_slot() for _ in requests]
        engine.step([StepEntry(s, r[:p], []) for s, r, p in zip(engine.slots, requests, prompts)])
    done = list(prompts)
    live = [0, 1, 2]
    for step in range(40):
        if step == 12:
            live = [0, 2]             # the batch shrinks: another graph
        outs = []
        for engine in (graphed, eager):
            logits = engine.step([StepEntry(engine.slots[i], [requests[i][done[i]]], [0]) for i in live])
            outs.append(logits.float().cpu().numpy())
            if step % 5 == 0:         # other work between replays
                extra = engine.alloc_slot()
                engine.step([StepEntry(extra, requests[1][:33], [32])])
                engine.select(logits, [__import__("beholdd").SamplingParams()] * len(live), live, [step] * len(live))
                engine.free_slot(extra)
                torch.cuda.synchronize()
        for i in live:
            done[i] += 1
        if dtype == "float32":
            assert np.array_equal(outs[0], outs[1]), step
        else:
            worst = max(worst, schedules.relative_error(outs[0], outs[1]))
    assert worst < 5e-3, worst
    assert len(graphed.graphs.graphs) >= 3        # (3, 16 pages), (2, 16 pages), (2, 32 pages)
    cfg, weights = plain.load_plain(folder)
    final = plain.forward_logits(cfg, weights, requests[0][:done[0]])[-1]
    assert schedules.relative_error(outs[0][0], final) < TOLERANCE[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_captured_steps_of_a_few_tokens_per_sequence(model_dirs, dtype):
    """An engine that is told to capture steps of up to four tokens per sequence: steps in which every sequence brings
    three tokens are captured and replayed (across a page boundary and a change of the batch), steps of one token go on
    as before, a step of unequal counts is launched kernel by kernel; logits asked for at some of a step's places only.
    Every step against an engine without captures, the end against the plain implementation."""
    from beholdd.engine import Engine, StepEntry
    folder = model_dirs("D", "bfloat16")
    graphed = Engine(folder, dtype=dtype, max_tokens=4096, graph_rows_per_sequence=4)
    eager = Engine(folder, dtype=dtype, max_tokens=4096, use_graphs=False)
    requests = schedules.random_requests(1500, [400, 300, 200], seed=23)
    done = [50, 30, 1]
    for engine in (graphed, eager):
        engine.slots = [engine.alloc_slot() for _ in requests]
        engine.step([StepEntry(s, r[:p], []) for s, r, p in zip(engine.slots, requests, done)])
    live = [0, 1, 2]
    worst = 0.0
    counts = []
    for step in range(30):
        if step == 14:
            live = [0, 2]
        each = [1, 1, 1] if step % 7 == 3 else [3, 2, 3] if step == 9 else [3, 3, 3]
        want = [[0, 2], [1], [0, 1, 2]] if each == [3, 3, 3] else [[n - 1] for n in each]
        outs = []
        for engine in (graphed, eager):
            logits = engine.step([StepEntry(engine.slots[i], requests[i][done[i]:done[i] + each[i]], want[i]) for i in live])
            outs.append(logits.float().cpu().numpy())
        counts.append(outs[0].shape[0])
        for i in live:
            done[i] += each[i]
        if dtype == "float32":
            assert np.array_equal(outs[0], outs[1]), step
        else:
            worst = max(worst, schedules.relative_error(outs[0], outs[1]))
    assert worst < 5e-3, worst
    assert counts[0] == 6 and counts[3] == 3 and counts[20] == 5
    keys = set(graphed.graphs.graphs)
    assert {(3, 16, 3), (2, 16, 3), (3, 16, 1), (2, 16, 1)} <= keys and not any(key[2] == 2 for key in keys), keys
    assert max(done) > 64           # the steps of three crossed a page's end
    cfg, weights = plain.load_plain(folder)
    final = plain.forward_logits(cfg, weights, requests[0][:done[0]])[-1]
    assert schedules.relative_error(outs[0][1], final) < TOLERANCE[dtype]
    graphed.cache.check_invariants()


def _varied(model_dirs):
    """Tiny configuration B (separate head) with weights of a larger scale: greedy continuations that change
    from token to token, so that a wrong position, a stale page or a wrong length after the prompt changes
    a token.  Returns folder, plain configuration and weights, prompts of 1, 7, 23 and 40 tokens, the numbers
    of new tokens and the plain implementation's greedy tokens."""
    folder = model_dirs("B", "bfloat16", seed=1, std=0.05)
    cfg, weights = plain.load_plain(folder)
    prompts = schedules.random_requests(cfg.vocab, [1, 7, 23, 40], seed=2)
    max_new = [12, 9, 12, 6]
    want = [plain.greedy_generate(cfg, weights, prompt, n)[0] for prompt, n in zip(prompts, max_new)]
    for tokens in want:
        assert len(set(tokens)) >= 3, f"the expected tokens {tokens} would hide a fault after the prompt"
    return folder, cfg, weights, prompts, max_new, want


def test_greedy_generation_through_the_entry_point(model_dirs):
    """Prompts of unequal lengths with unequal numbers of new tokens, token for token against the plain
    implementation; a stop token that one request meets in mid-sequence while the others go on; the loop that
    runs a step ahead against the plain loop; bfloat16 within rounding."""
    import beholdd
    folder, cfg, weights, prompts, max_new, want = _varied(model_dirs)
    engine = beholdd.Engine(folder, dtype="float32", max_tokens=512)
    results = engine.generate(prompts, max_new_tokens=max_new)
    for prompt, result, tokens, n in zip(prompts, results, want, max_new):
        assert result.token_ids == tokens and result.finish_reason == "length"
        assert result.prompt_tokens == len(prompt) and result.completion_tokens == n
    # a stop token that request 2 chooses as its fourth token
    stop = want[2][3]
    cuts = [tokens.index(stop) if stop in tokens else None for tokens in want]
    assert cuts[2] is not None and cuts[2] > 0 and any(cut is None for cut in cuts), (stop, want)
    again = engine.generate(prompts, max_new_tokens=max_new, stop_token_ids=[stop])
    for tokens, cut, after in zip(want, cuts, again):
        if cut is not None:
            assert after.token_ids == tokens[:cut] and after.finish_reason == "stop" and after.stop_token == stop
        else:
            assert after.token_ids == tokens and after.finish_reason == "length" and after.stop_token is None
    # bfloat16: every chosen token is the plain implementation's choice, or as good within rounding
    engine16 = beholdd.Engine(folder, dtype="bfloat16", max_tokens=512)
    results16 = engine16.generate(prompts, max_new_tokens=max_new)
    for prompt, result in zip(prompts, results16):
        tokens = list(prompt)
        for token in result.token_ids:
            logits = plain.forward_logits(cfg, weights, tokens)[-1]
            assert logits[token] >= logits.max() - TOLERANCE["bfloat16"] * np.abs(logits).max()
            tokens.append(token)
    assert any(len(set(r.token_ids)) >= 3 for r in results16)
    # the loop that runs a step ahead of the host and the plain one (which a callback for logits selects) agree,
    # and the logits that the plain loop chose from are the plain implementation's at that position
    for runner, tolerance in ((engine, TOLERANCE["float32"]), (engine16, TOLERANCE["bfloat16"])):
        ahead = runner.generate(prompts, max_new_tokens=max_new, stop_token_ids=[stop])
        seen = {}
        plain_loop = runner.generate(prompts, max_new_tokens=max_new, stop_token_ids=[stop],
                                     on_logits=lambda index, step, row: seen.setdefault((index, step), row.float().cpu().numpy()))
        assert [(r.token_ids, r.finish_reason, r.stop_token) for r in ahead] == \
               [(r.token_ids, r.finish_reason, r.stop_token) for r in plain_loop]
        for index, (prompt, result) in enumerate(zip(prompts, ahead)):
            full = plain.forward_logits(cfg, weights, list(prompt) + result.token_ids)
            for step in range(len(result.token_ids)):
                assert schedules.relative_error(seen[(index, step)], full[len(prompt) - 1 + step]) < tolerance, (index, step)
        runner.cache.check_invariants()
        assert runner.cache.live_slots() == []


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_sampling_is_seeded_and_independent_of_the_batch(model_dirs, dtype):
    """Prompts of 1, 7, 23 and 40 tokens, temperature 0.8, 12 tokens each; then with top-k and top-p.  In
    bfloat16 the decode steps run from captured graphs and the loop a step ahead of the host."""
    import beholdd
    folder = model_dirs("B", "bfloat16", seed=1, std=0.05)
    prompts = schedules.random_requests(384, [1, 7, 23, 40], seed=6)
    engine = beholdd.Engine(folder, dtype=dtype, max_tokens=1024)
    for options in ({"temperature": 0.8}, {"temperature": 1.3, "top_k": 20, "top_p": 0.9}):
        first = engine.generate(prompts, max_new_tokens=12, seed=5, **options)
        again = engine.generate(prompts, max_new_tokens=12, seed=5, **options)
        other = engine.generate(prompts, max_new_tokens=12, seed=6, **options)
        assert [r.token_ids for r in first] == [r.token_ids for r in again]
        assert [r.token_ids for r in first] != [r.token_ids for r in other]
        assert all(len(r.token_ids) == 12 for r in first)
        if dtype == "float32":
            # a request's draws and logits do not depend on its batch-mates (in bfloat16 the products of a step
            # of other rows round differently, so a draw next to a threshold may fall on the other side)
            in_pairs = engine.generate(prompts, max_new_tokens=12, seed=5, batch_size=2, **options)
            assert [r.token_ids for r in in_pairs] == [r.token_ids for r in first]
        greedy = engine.generate(prompts, max_new_tokens=12)
        assert [r.token_ids for r in greedy] != [r.token_ids for r in first]
    if dtype == "bfloat16":
        # every drawn token had a chance: it lies among the 20 largest logits of the plain implementation, give
        # or take rounding
        cfg, weights = plain.load_plain(folder)
        for prompt, result in zip(prompts, first):
            tokens = list(prompt)
            for token in result.token_ids:
                logits = plain.forward_logits(cfg, weights, tokens)[-1]
                assert logits[token] >= np.sort(logits)[-20] - TOLERANCE["bfloat16"] * np.abs(logits).max()
                tokens.append(token)
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == []


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(model_dirs, tmp_path, dtype):
    """bin/trace_run as a user runs it: a batch of three unequal requests, their prompts in one
    step, then one token each; the shortest ends first; then a second batch in the freed room."""
    folder = model_dirs("B", "bfloat16")
    cfg, weights = plain.load_plain(folder)
    requests = dict(zip("abcde", schedules.random_requests(cfg.vocab, [40, 70, 55, 64, 20], seed=9)))
    want = {name: plain.forward_logits(cfg, weights, tokens) for name, tokens in requests.items()}
    steps, expect, number = [], {}, 0

    def run_batch(names, prompt_len):
        nonlocal number
        done = {n: prompt_len[n] for n in names}
        ended = [n for n in names if done[n] == len(requests[n])]
        steps.append({"step": number, "entries": [{"id": n, "tokens": requests[n][:done[n]],
                                                   "want": [done[n] - 1, 0] if done[n] > 1 else [0]} for n in names],
                      "end": ended})
        expect[number] = np.concatenate([want[n][[done[n] - 1, 0] if done[n] > 1 else [0]] for n in names])
        number += 1
        live = [n for n in names if n not in ended]
        while live:
            entries = [{"id": n, "tokens": [requests[n][done[n]]], "want": [0] if done[n] % 2 else []} for n in live]
            rows = [want[n][done[n]:done[n] + 1] for n in live if done[n] % 2]
            for n in live:
                done[n] += 1
            ended = [n for n in live if done[n] == len(requests[n])]
            steps.append({"step": number, "entries": entries, "end": ended})
            if rows:
                expect[number] = np.concatenate(rows)
            number += 1
            live = [n for n in live if n not in ended]

    run_batch(["a", "b", "c"], {"a": 30, "b": 50, "c": 55})
    run_batch(["d", "e"], {"d": 60, "e": 5})
    out_dir = tmp_path / "out"
    trace = "\n".join(json.dumps(s) for s in steps) + "\n"
    # live tokens, each request rounded up to 64: a 64 + b 128 + c 64 = 256 at most
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                          "--out", str(out_dir), "--max-tokens", "256", "--capture", str(tmp_path / "capture")],
                         input=trace, capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [line for line in run.stdout.splitlines() if line.startswith("done")] == [f"done {s['step']}" for s in steps]
    assert sorted(os.listdir(out_dir)) == sorted(f"{n}.f32" for n in expect)
    for number, rows in expect.items():
        got = np.fromfile(out_dir / f"{number}.f32", dtype="<f4").reshape(-1, cfg.vocab)
        assert got.shape == rows.shape
        assert schedules.relative_error(got, rows) < TOLERANCE[dtype], number
    from beholdd.engine.artifact import read_position_capture
    capture = read_position_capture(str(tmp_path / "capture"))
    assert capture.requests == requests and len(capture.rows) == sum(len(rows) for rows in expect.values())
    assert np.array_equal(capture.logits[:len(expect[0])], np.fromfile(out_dir / "0.f32", dtype="<f4").reshape(-1, cfg.vocab))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replays_of_different_cuts_compare_through_the_tool(model_dirs, tmp_path, dtype):
    """Capture, then compare: the same requests replayed whole, in batches of unequal lengths and in portions;
    every replay leaves a capture that says which request and position each row belongs to, and `beholdd compare`
    holds any two of them, and the plain implementation's logits written as such a capture, to the tolerance;
    the same schedule replayed twice compares equal byte for byte."""
    import io
    from beholdd import cli
    from beholdd.engine import replay
    from beholdd.engine.artifact import PositionCaptureWriter

    folder = model_dirs("B", "bfloat16")
    cfg, weights = plain.load_plain(folder)
    requests = schedules.random_requests(cfg.vocab, [40, 70, 9, 64, 130], seed=12)
    traces = {"whole": schedules.trace_of(schedules.whole, requests),
              "batches": schedules.trace_of(schedules.batches, requests, batch_size=3),
              "again": schedules.trace_of(schedules.batches, requests, batch_size=3),
              "portions": schedules.trace_of(schedules.portions, requests)}
    for name, steps in traces.items():
        lines = io.StringIO("".join(json.dumps(step) + "\n" for step in steps))
        said = io.StringIO()
        code = replay.main(["--model", folder, "--dtype", dtype, "--out", str(tmp_path / f"{name}.out"), "--max-tokens", "512",
                            "--capture", str(tmp_path / name)], stdin=lines, stdout=said)
        assert code == 0 and said.getvalue().splitlines() == [f"done {step['step']}" for step in steps]
    writer = PositionCaptureWriter(str(tmp_path / "plain.bhdlogit"), cfg.vocab, {"tool": "plain implementation"})
    for index, tokens in enumerate(requests):
        writer.feed(f"r{index}", tokens)
        writer.add(index, [(f"r{index}", position) for position in range(len(tokens))], plain.forward_logits(cfg, weights, tokens))
    writer.close()

    def compare(a, b, tolerance):
        out = io.StringIO()
        code = cli.main(["compare", str(tmp_path / a), str(tmp_path / b), "--tolerance", str(tolerance)], out=out)
        return code, out.getvalue()

    between_cuts = 5e-5 if dtype == "float32" else 1e-2
    for name in ("batches", "portions"):
        code, text = compare("whole", name, between_cuts)
        assert code == 0 and "PASS" in text, text
    for name in ("whole", "batches", "portions"):
        code, text = compare("plain.bhdlogit", name, TOLERANCE[dtype])
        assert code == 0 and "PASS" in text, text
    code, text = compare("batches", "again", 0)
    assert code == 0 and "Exact logit comparison: PASS" in text, text
    code, text = compare("whole", "batches", 0)
    assert code == 1 and "same schedule" in text
    code, text = compare("whole", "batches", 1e-12)
    assert code == 1 and "logits differ by" in text


def test_command_line_generate(model_dirs, tmp_path):
    import beholdd
    from beholdd.engine.artifact import read_logits_artifact
    folder, cfg, weights, prompts, _, _ = _varied(model_dirs)
    prompt = prompts[1]
    capture = tmp_path / "logits.bin"
    timing = tmp_path / "steps.tsv"
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "beholdd"), "generate", "--model", folder,
                          "--dtype", "float32", "--prompt-ids", ",".join(str(t) for t in prompt), "--max-new-tokens", "6",
                          "--logits-out", str(capture), "--step-timing-out", str(timing)],
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    want, _ = plain.greedy_generate(cfg, weights, prompt, 6)
    assert len(set(want)) >= 3
    assert f"generated: {want}" in run.stdout
    got_prompt, generated, logits = read_logits_artifact(str(capture))
    assert got_prompt == prompt and generated == want and logits.shape == (6, cfg.vocab)
    full = plain.forward_logits(cfg, weights, prompt + want[:-1])
    assert schedules.relative_error(logits, full[len(prompt) - 1:]) < 1e-4
    assert timing.read_text().splitlines()[0] == "step\tduration_ms"


def test_command_line_generate_without_captures(model_dirs):
    """`beholdd generate` in bfloat16 with three prompts and a temperature, no capture flags: the loop that runs a
    step ahead of the host, no per-step lines; the tokens are those `Engine.generate` draws with the same seed."""
    import re

    import beholdd
    folder, cfg, weights, prompts, _, _ = _varied(model_dirs)
    prompts = prompts[1:]
    command = [sys.executable, os.path.join(ROOT, "bin", "beholdd"), "generate", "--model", folder, "--dtype", "bfloat16",
               "--max-new-tokens", "10", "--temperature", "0.7", "--top-k", "30", "--seed", "9", "--max-tokens", "512"]
    for prompt in prompts:
        command += ["--prompt-ids", ",".join(str(t) for t in prompt)]
    run = subprocess.run(command, capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    engine = beholdd.Engine(folder, dtype="bfloat16", max_tokens=512)
    want = engine.generate(prompts, max_new_tokens=10, temperature=0.7, top_k=30, seed=9)
    printed = re.findall(r"generated: (\[.*\])", run.stdout)
    assert [json.loads(text) for text in printed] == [r.token_ids for r in want]
    assert len({tuple(r.token_ids) for r in want}) == 3 and all(len(r.token_ids) == 10 for r in want)
    assert "step   0" not in run.stdout and "generated tokens/s" in run.stdout
    # every drawn token had a chance by the plain implementation's logits
    for prompt, result in zip(prompts, want):
        tokens = list(prompt)
        for token in result.token_ids:
            logits = plain.forward_logits(cfg, weights, tokens)[-1]
            assert logits[token] >= np.sort(logits)[-30] - TOLERANCE["bfloat16"] * np.abs(logits).max()
            tokens.append(token)
