"""The engine where no small test goes: requests of 8,100 and 16,390 tokens against the plain implementation, the
Qwen3-32B layer sizes at a context of 16,384, the real vocabulary of 151,936 entries, more captured decode steps
than the engine keeps, a selection wider than the sampler's buffer between generations, and the byte plan against
what the allocator saw."""

import numpy as np
import pytest
import torch

import plain_qwen3 as plain
import schedules

pytestmark = pytest.mark.gpu

TOLERANCE = {"float32": 1e-4, "bfloat16": 2e-2}


def _config(**changes):
    config = {"architectures": ["Qwen3ForCausalLM"], "num_hidden_layers": 2, "hidden_size": 320,
              "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 128, "intermediate_size": 640,
              "vocab_size": 1500, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 16400,
              "tie_word_embeddings": False}
    config.update(changes)
    return config


def _sharpen(folder, factor):
    """Multiply every layer's query-norm weight by `factor`: the scores of a head then spread `factor` times
    wider, so that among thousands of keys a few dozen carry the softmax, wherever they stand.  With weights
    as they are drawn the average over 16,000 values would hide a page that is read wrongly."""
    from safetensors import safe_open

    from beholdd.weights.safetensors_io import write_safetensors
    tensors = {}
    path = f"{folder}/model.safetensors"
    with safe_open(path, framework="pt") as handle:
        for name in handle.keys():
            tensor = handle.get_tensor(name)
            tensors[name] = (tensor.float() * factor).to(tensor.dtype) if name.endswith("q_norm.weight") else tensor
    write_safetensors(path, tensors)


def _wanted(n, tail=40, spread=64):
    """The last `tail` positions and `spread` ones spread over the rest."""
    return sorted(set(int(x) for x in np.linspace(0, n - tail - 1, spread)) | set(range(n - tail, n)))


@pytest.fixture(scope="module")
def long_model(tmp_path_factory):
    """The head shape and group of the large models in a narrow two-layer model with a context of 16,400; one
    request of 16,390 tokens and one of 8,100, and the plain implementation's logits at the wanted positions."""
    import beholdd
    folder = str(tmp_path_factory.mktemp("long_context"))
    beholdd.write_random_model(folder, _config(), seed=3, dtype="bfloat16")
    _sharpen(folder, 2.0)
    cfg, weights = plain.load_plain(folder)
    requests = schedules.random_requests(cfg.vocab, [16390, 8100], seed=21)
    wanted = [_wanted(len(r)) for r in requests]
    expected = [plain.forward_logits(cfg, weights, r, rows=w) for r, w in zip(requests, wanted)]
    return folder, requests, wanted, expected


def _prompt_then_one_by_one(engine, tokens, wanted, tail=32):
    from beholdd.engine import StepEntry
    cut = len(tokens) - tail
    slot = engine.alloc_slot()
    rows = [engine.step([StepEntry(slot, tokens[:cut], [w for w in wanted if w < cut])]).float().cpu().numpy()]
    for position in range(cut, len(tokens)):
        logits = engine.step([StepEntry(slot, [tokens[position]], [0] if position in wanted else [])])
        if logits is not None:
            rows.append(logits.float().cpu().numpy())
    engine.free_slot(slot)
    return np.concatenate(rows)


def _check(label, got, want, tolerance):
    assert got.shape == want.shape and np.isfinite(got).all(), label
    per_row = np.abs(got.astype(np.float64) - want).max(axis=1) / np.abs(want).max()
    assert per_row.max() < tolerance, f"{label}: error {per_row.max():.3e} >= {tolerance}, first wrong row {int(np.argmax(per_row >= tolerance))}"
    return float(per_row.max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_requests_against_the_plain_implementation(long_model, dtype):
    """16,390 and 8,100 tokens: the prompt whole in one step (257 and 127 pages), the last 32 tokens one by one
    (through the captured graphs, page tables of 272 and 128 pages, keys split over workgroups), the second
    request in the pages the first gave back."""
    from beholdd.engine import Engine
    folder, requests, wanted, expected = long_model
    engine = Engine(folder, dtype=dtype, max_tokens=16448)
    for tokens, rows, want in zip(requests, wanted, expected):
        error = _check(f"{len(tokens)} tokens", _prompt_then_one_by_one(engine, tokens, rows), want, TOLERANCE[dtype])
        print(f"{dtype}, {len(tokens)} tokens: {error:.2e}")
    if dtype == "bfloat16":
        assert {key[1] for key in engine.graphs.graphs} == {256, 272, 128}
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == []


def test_one_far_page_moves_the_last_logits(long_model):
    """What the test above rests on: other tokens in one page 8,000 positions back (positions 64 to 127 of 8,100)
    move the last position's logits by several times the wider tolerance, so a far page that is read wrongly
    shows in the comparison."""
    folder, requests, wanted, expected = long_model
    cfg, weights = plain.load_plain(folder)
    other = list(requests[1])
    other[64:128] = [(token + 7) % cfg.vocab for token in other[64:128]]
    moved = plain.forward_logits(cfg, weights, other, rows=[len(other) - 1])[0]
    assert wanted[1][-1] == len(other) - 1
    assert np.abs(moved - expected[1][-1]).max() / np.abs(expected[1]).max() > 3 * TOLERANCE["bfloat16"]


def test_the_32b_layer_sizes_at_a_context_of_16384(tmp_path):
    """One layer of Qwen3-32B's sizes (64 query heads on 8 kv heads, heads wider than the model) with positions up
    to 16,384: four requests of 9,000 to 16,300 tokens, their prompts fed in portions of at most 8,192 tokens a
    step, then 16 tokens each decoded together; bfloat16 against the float32 engine."""
    import beholdd
    from beholdd.engine import Engine, StepEntry
    from beholdd.engine.generation import prefill
    folder = str(tmp_path / "m")
    beholdd.write_random_model(folder, _config(num_hidden_layers=1, hidden_size=5120, num_attention_heads=64,
                                               num_key_value_heads=8, intermediate_size=25600, vocab_size=1000,
                                               max_position_embeddings=16384), seed=4, dtype="bfloat16")
    _sharpen(folder, 2.0)
    lengths = [9000, 16300, 12111, 14000]
    requests = schedules.random_requests(1000, [n + 16 for n in lengths], seed=8)
    got = {}
    for dtype in ("float32", "bfloat16"):
        engine = Engine(folder, dtype=dtype, max_tokens=sum(-(-(n + 16) // 64) * 64 for n in lengths), max_rows_per_step=8192)
        slots = [engine.alloc_slot() for _ in requests]
        rows = [prefill(engine, slots, [r[:n] for r, n in zip(requests, lengths)]).float().cpu().numpy()]
        for step in range(16):
            rows.append(engine.step([StepEntry(s, [r[n + step]], [0]) for s, r, n in zip(slots, requests, lengths)])
                        .float().cpu().numpy())
        for slot in slots:
            engine.free_slot(slot)
        engine.cache.check_invariants()
        if dtype == "bfloat16":
            assert engine.graphs.graphs and all(key == (4, 256, 1) for key in engine.graphs.graphs)
        got[dtype] = np.stack(rows, axis=1)
        del engine
    for index, n in enumerate(lengths):
        _check(f"request of {n}", got["bfloat16"][index], got["float32"][index], TOLERANCE["bfloat16"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_real_vocabulary(tmp_path_factory, dtype):
    """A vocabulary of 151,936 entries on one narrow layer: the head's product on the wanted rows, the argmax in two
    steps over chunks of the vocabulary, token ids beyond 2^17; logits and greedy tokens against the plain
    implementation."""
    import beholdd
    folder = str(tmp_path_factory.mktemp("vocabulary"))
    beholdd.write_random_model(folder, _config(num_hidden_layers=1, hidden_size=128, num_attention_heads=2,
                                               num_key_value_heads=1, head_dim=64, intermediate_size=256,
                                               vocab_size=151936, max_position_embeddings=256), seed=6, dtype="bfloat16", std=0.05)
    cfg, weights = plain.load_plain(folder)
    prompts = [[151935, 7, 140000, 65536, 99999], [131072], [5, 151000, 3]]
    engine = beholdd.Engine(folder, dtype=dtype, max_tokens=512)
    from beholdd.engine import StepEntry
    slot = engine.alloc_slot()
    logits = engine.step([StepEntry(slot, prompts[0], list(range(5)))]).float().cpu().numpy()
    engine.free_slot(slot)
    _check("logits", logits, plain.forward_logits(cfg, weights, prompts[0]), TOLERANCE[dtype])
    results = engine.generate(prompts, max_new_tokens=6)
    seen = set()
    for prompt, result in zip(prompts, results):
        tokens = list(prompt)
        for token in result.token_ids:
            row = plain.forward_logits(cfg, weights, tokens)[-1]
            if dtype == "float32":
                assert token == plain.greedy_token(row), (tokens, token)
            else:
                assert row[token] >= row.max() - TOLERANCE[dtype] * np.abs(row).max(), (tokens, token)
            tokens.append(token)
            seen.add(token)
    assert len(seen) >= 6 and max(seen) >= 2048          # tokens from several chunks of the vocabulary
    # Draws at this vocabulary go through chunks of the row (weight sums, the chunks' candidates): every token drawn
    # with a top-k must be among the k largest of the plain logits, with a top-p within the smallest set that holds
    # that share (one token of slack at its end, and the tolerance's worth of logit), and the same seed must give the
    # same tokens again.
    slack = TOLERANCE[dtype]
    for filters in (dict(top_k=5), dict(top_p=0.3), dict(top_k=40, top_p=0.5), dict()):
        drawn = engine.generate(prompts, max_new_tokens=5, temperature=0.7, seed=11, **filters)
        again = engine.generate(prompts, max_new_tokens=5, temperature=0.7, seed=11, **filters)
        assert [r.token_ids for r in drawn] == [r.token_ids for r in again]
        for prompt, result in zip(prompts, drawn):
            tokens = list(prompt)
            for token in result.token_ids:
                row = plain.forward_logits(cfg, weights, tokens)[-1].astype(np.float64)
                order = np.argsort(-row, kind="stable")
                allowed = len(order)
                if filters.get("top_k"):
                    allowed = min(allowed, filters["top_k"])
                floor = row[order[allowed - 1]]
                assert row[token] >= floor - slack * np.abs(row).max(), (filters, tokens, token)
                if filters.get("top_p"):
                    kept = order[:allowed]
                    weights_kept = np.exp((row[kept] - row[kept[0]]) / 0.7)
                    share = np.cumsum(weights_kept) / weights_kept.sum()
                    last = min(int(np.searchsorted(share, filters["top_p"])) + 1, allowed - 1)
                    assert row[token] >= row[kept[last]] - slack * np.abs(row).max(), (filters, tokens, token)
                tokens.append(token)


def test_more_decode_shapes_than_the_engine_keeps(model_dirs):
    """Six requests that end one after the other: decode steps of 6, 5, 4, 3, 2 and 1 sequences in an engine that
    keeps three captures, twice, so that captures are dropped and made again; and between two generations a
    selection for more rows than the sampler's buffer has, after which the captures read the new buffer.  Tokens
    against an engine without captures."""
    import beholdd
    from beholdd.engine import StepEntry
    folder = model_dirs("B", "bfloat16", seed=1, std=0.05)
    prompts = schedules.random_requests(384, [3, 9, 17, 5, 30, 12], seed=13)
    max_new = [4, 6, 8, 10, 12, 14]
    plain_engine = beholdd.Engine(folder, dtype="bfloat16", max_tokens=1024, max_slots=6, use_graphs=False)
    want = [r.token_ids for r in plain_engine.generate(prompts, max_new_tokens=max_new, temperature=0.9, seed=3)]
    assert len({tuple(w) for w in want}) == 6
    engine = beholdd.Engine(folder, dtype="bfloat16", max_tokens=1024, max_slots=6, graph_limit=3)
    for _ in range(2):
        got = [r.token_ids for r in engine.generate(prompts, max_new_tokens=max_new, temperature=0.9, seed=3)]
        assert got == want
        assert len(engine.graphs.graphs) == 3
    # a selection over every row of a prompt: more rows than the engine has slots
    slot = engine.alloc_slot()
    logits = engine.step([StepEntry(slot, prompts[4], list(range(30)))])
    engine.free_slot(slot)
    before = engine.sampler.out
    chosen = engine.select(logits, [beholdd.SamplingParams()] * 30, list(range(30)), [0] * 30)
    assert engine.sampler.out is not before and engine.sampler.capacity == 30
    assert chosen == [int(t) for t in logits.float().argmax(dim=1).cpu()]
    got = [r.token_ids for r in engine.generate(prompts, max_new_tokens=max_new, temperature=0.9, seed=3)]
    assert got == want
    assert all(graph.fed_buffer is engine.sampler.out for graph in engine.graphs.graphs.values())
    engine.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_byte_plan_covers_what_the_allocator_saw(model_dirs, dtype):
    """An engine whose steps take at most 256 tokens: prompts of 1,400 tokens together go through in portions,
    then decode through the captures; the device memory in use never exceeds the plan made before anything was
    allocated, and the plan is no wild overestimate of it."""
    import beholdd
    folder = model_dirs("D", "bfloat16")
    prompts = schedules.random_requests(1500, [500, 3, 700, 200], seed=17)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    base = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    engine = beholdd.Engine(folder, dtype=dtype, max_tokens=2048, max_slots=4, max_rows_per_step=256)
    assert engine.plan.unaccounted == []
    loaded = torch.cuda.max_memory_allocated() - base
    results = engine.generate(prompts, max_new_tokens=[20, 12, 9, 20])
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - base
    assert peak <= engine.plan.total_bytes, (peak, engine.memory_plan())
    assert peak >= 0.25 * engine.plan.total_bytes, (peak, engine.memory_plan())
    print(f"{dtype}: peak {peak} bytes of a plan of {engine.plan.total_bytes} ({loaded} after loading)")
    # the same tokens as an engine that takes every prompt whole
    whole = beholdd.Engine(folder, dtype=dtype, max_tokens=2048, max_slots=4)
    assert whole.max_rows_per_step == 2048
    if dtype == "float32":       # (in bfloat16 a product of other rows rounds differently, and a near tie may fall the other way)
        assert [r.token_ids for r in whole.generate(prompts, max_new_tokens=[20, 12, 9, 20])] == [r.token_ids for r in results]
    # a limit below the plan refuses before anything is read
    with pytest.raises(beholdd.engine.MemoryBudgetError):
        beholdd.Engine(folder, dtype=dtype, max_tokens=2048, max_slots=4, max_rows_per_step=256,
                       memory_limit_bytes=engine.plan.total_bytes - 1)
