"""The engine's own logic on the CPU: step layout, paged cache, slots, registry and loading,
with the kernel library replaced by a torch double (tests/kernel_emulation.py).  What is
compared is the same as on the GPU: every cut of the work against the plain implementation."""

import numpy as np
import pytest
import torch

import beholdd
import plain_qwen3 as plain
import schedules
from beholdd.engine import Engine, StepEntry, StepError
from kernel_emulation import TorchKernels


def make_engine(folder, dtype="float32", max_tokens=1024, **kw):
    return Engine(folder, dtype=dtype, max_tokens=max_tokens, device="cpu", kernels=TorchKernels(), **kw)


@pytest.mark.parametrize("name,lengths", [("A", [5, 11, 17, 70]), ("B", [1, 7, 23, 40, 90])])
def test_every_cut_matches_the_plain_implementation(model_dirs, name, lengths):
    folder = model_dirs(name, "float32")
    cfg, weights = plain.load_plain(folder)
    requests = schedules.random_requests(cfg.vocab, lengths, seed=3)
    expected = [plain.forward_logits(cfg, weights, r) for r in requests]
    engine = make_engine(folder)
    for label, got in (("whole", schedules.whole(engine, requests)),
                       ("tail", schedules.tail_one_by_one(engine, requests, tail=32)),
                       ("batches", schedules.batches(engine, requests, batch_size=3)),
                       ("portions", schedules.portions(engine, requests))):
        for i, (g, e) in enumerate(zip(got, expected)):
            assert g.shape == e.shape, (label, i)
            assert schedules.relative_error(g, e) < 1e-4, (label, i, schedules.relative_error(g, e))
    engine.cache.check_invariants()
    assert engine.cache.live_slots() == []
    assert engine.cache.free_page_count() == engine.cache.n_pages


def test_bfloat16_storage_widens_exactly_in_a_float32_engine(model_dirs):
    folder = model_dirs("A", "bfloat16")
    cfg, weights = plain.load_plain(folder)
    requests = schedules.random_requests(cfg.vocab, [9], seed=1)
    got = schedules.whole(make_engine(folder), requests)[0]
    assert schedules.relative_error(got, plain.forward_logits(cfg, weights, requests[0])) < 1e-4


def test_storage_rule_of_a_bfloat16_engine(model_dirs):
    kept32 = make_engine(model_dirs("A", "float32"), dtype="bfloat16")
    kept16 = make_engine(model_dirs("A", "bfloat16"), dtype="bfloat16")
    assert kept32.model.embedding.weight.dtype == torch.float32      # stored in 32-bit: stays so
    assert kept16.model.embedding.weight.dtype == torch.bfloat16
    assert kept16.model.blocks[0].mixer.qkv.weight.dtype == torch.bfloat16
    assert kept16.cache.groups[0].k.dtype == torch.bfloat16
    tied = kept16.model
    assert tied.head.linear.weight.data_ptr() == tied.embedding.weight.data_ptr()   # tied: the same matrix


def test_step_refuses_bad_entries_without_changing_lengths(model_dirs):
    engine = make_engine(model_dirs("A", "float32"), max_tokens=128)
    slot = engine.alloc_slot()
    engine.step([StepEntry(slot, [1, 2, 3], [2])])
    for bad in ([StepEntry(slot, [], [])], [StepEntry(slot, [256], [0])], [StepEntry(slot, [-1], [0])],
                [StepEntry(slot, [1], [1])], [StepEntry(slot, [1], [0]), StepEntry(slot, [2], [0])],
                [StepEntry(slot + 1, [1], [0])], [],
                # wrong types are refused with a reason too, not with a traceback from the middle of the step
                [StepEntry(slot, 7, [0])], [StepEntry(slot, [1], 0)], [StepEntry([slot], [1], [0])], [StepEntry(True, [1], [0])],
                [StepEntry(slot, [1.5], [0])], [StepEntry(slot, None, [])]):
        with pytest.raises((StepError, beholdd.cache.CacheError)):
            engine.step(bad)
        assert engine.cache.length(slot) == 3
        engine.cache.check_invariants()
    with pytest.raises(beholdd.cache.CacheFull):          # 128 tokens of cache, 126 more do not fit after 3
        engine.step([StepEntry(slot, [1] * 126, [])])
    assert engine.cache.length(slot) == 3
    engine.cache.check_invariants()
    assert engine.step([StepEntry(slot, [4], [])]) is None      # nothing wanted: no logits


def test_a_failing_step_rolls_back_and_a_retry_matches(model_dirs):
    # in the manner of crates/beholdd-model/src/qwen3moe/forward.rs:2937-2998
    folder = model_dirs("B", "float32")
    engine = make_engine(folder)
    slot = engine.alloc_slot()
    tokens = schedules.random_requests(384, [70], seed=5)[0]
    engine.step([StepEntry(slot, tokens[:60], [])])
    real = engine.kernels.swiglu
    calls = {"n": 0}

    def failing(*a, **k):
        calls["n"] += 1
        if calls["n"] == 2:
            raise RuntimeError("injected failure")
        return real(*a, **k)

    engine.kernels.swiglu = failing
    free_before = engine.cache.free_page_count()
    with pytest.raises(RuntimeError, match="injected"):
        engine.step([StepEntry(slot, tokens[60:], [9])])
    engine.kernels.swiglu = real
    assert engine.cache.length(slot) == 60 and engine.cache.free_page_count() == free_before
    engine.cache.check_invariants()
    retried = engine.step([StepEntry(slot, tokens[60:], [9])]).numpy()
    fresh = make_engine(folder)
    s2 = fresh.alloc_slot()
    assert np.array_equal(retried, fresh.step([StepEntry(s2, tokens, [69])]).numpy())


def test_a_reused_slot_gives_the_same_logits_as_a_fresh_cache(model_dirs):
    folder = model_dirs("A", "float32")
    a, b = schedules.random_requests(256, [80, 75], seed=8)
    engine = make_engine(folder, max_tokens=128)
    first = schedules.whole(engine, [a])[0]          # fills and frees pages 0 and 1
    second = schedules.whole(engine, [b])[0]         # runs in the very same slot and pages
    fresh = schedules.whole(make_engine(folder, max_tokens=128), [b])[0]
    assert np.array_equal(second, fresh)
    assert not np.array_equal(first[:75], second)


def test_memory_limit_covers_weights_and_cache_and_is_checked_before_anything_is_read(model_dirs, monkeypatch):
    from beholdd.engine import MemoryBudgetError
    from beholdd.weights import binder

    folder = model_dirs("A", "bfloat16")
    weights = 90_496 * 2                                  # tiny A in bfloat16 (tied head: the embedding once)
    cache = 2 * 2 * 2 * 2 * 64 * 16 * 2                   # 2 layers, keys and values, 2 pages, 2 heads, 64 x 16
    reads = []
    real = binder.BoundWeights.__call__
    monkeypatch.setattr(binder.BoundWeights, "__call__", lambda self, name: reads.append(name) or real(self, name))
    # the plan holds weights and cache, and beyond them what a step of as many rows as the cache holds allocates
    # (the kernel double says nothing about its calls, so the parts' own matrices only)
    with pytest.raises(MemoryBudgetError, match="the engine needs") as refused:
        make_engine(folder, dtype="bfloat16", max_tokens=128, memory_limit_bytes=weights + cache)
    assert reads == [] and f"weights: {weights} bytes" in str(refused.value) and f"cache: {cache} bytes" in str(refused.value)
    total = int(str(refused.value).split("the engine needs ")[1].split()[0])
    assert total > weights + cache
    with pytest.raises(MemoryBudgetError):
        make_engine(folder, dtype="bfloat16", max_tokens=128, memory_limit_bytes=total - 1)
    assert reads == []
    engine = make_engine(folder, dtype="bfloat16", max_tokens=128, memory_limit_bytes=total)
    assert len(reads) == 24 and engine.weight_bytes == weights and engine.cache.allocated_bytes() == cache
    assert f"weights: {weights} bytes" in engine.memory_plan() and engine.plan.total_bytes == total
    assert engine.max_rows_per_step == 128
    assert engine.plan.bytes_of("working memory of a step of 128 rows") > 128 * 64 * 4
    smaller = make_engine(folder, dtype="bfloat16", max_tokens=128, max_rows_per_step=16)
    assert smaller.plan.bytes_of("working memory of a step of 16 rows") < engine.plan.bytes_of("working memory of a step of 128 rows") / 4
    slot = smaller.alloc_slot()
    with pytest.raises(beholdd.engine.step.StepError, match="max_rows_per_step"):
        smaller.step([beholdd.StepEntry(slot, list(range(17)), [16])])
    assert smaller.cache.length(slot) == 0
    smaller.step([beholdd.StepEntry(slot, list(range(16)), [15])])


def test_unknown_architecture_names_the_registered_ones(tmp_path, tiny_configs):
    config = dict(tiny_configs["A"], architectures=["Qwen9ForCausalLM"])
    with pytest.raises(beholdd.ConfigError, match="Qwen3ForCausalLM"):
        beholdd.write_random_model(str(tmp_path), config, seed=0)


def test_no_gpu_means_no_engine(model_dirs):
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(beholdd.kernels.KernelError, match="no CPU fallback"):
        Engine(model_dirs("A", "float32"), dtype="float32", max_tokens=64)


def test_an_engine_refuses_arguments_that_cannot_be_meant(model_dirs):
    folder = model_dirs("A", "float32")
    for number in (0, 1, 64):       # an integer would name an open file of the process, not a folder
        with pytest.raises(beholdd.ConfigError, match="named by a path"):
            make_engine(number)
    for bad in (dict(max_tokens="64"), dict(max_tokens=1 << 70), dict(max_tokens=1.5), dict(max_tokens=0),
                dict(max_slots=-1), dict(max_slots=[1]), dict(max_slots=1 << 39), dict(max_rows_per_step="7"),
                dict(max_rows_per_step=float("inf")), dict(max_rows_per_step=0), dict(graph_rows_per_sequence={}),
                dict(graph_rows_per_sequence=0), dict(graph_limit=None), dict(memory_limit_bytes="1000"),
                dict(memory_limit_bytes=1.5), dict(dtype="float16")):
        with pytest.raises(ValueError):
            make_engine(folder, **bad)
