"""Toy parts registered from outside the package (tests/toy_parts.py), on the CPU with the
kernel double: a mixer with state of its own, a layer that runs twice, a layer that reads
another layer's cache."""

import pytest
import torch

import beholdd
import toy_parts
from beholdd.engine import Engine
from kernel_emulation import TorchKernels


@pytest.fixture(autouse=True)
def toys():
    toy_parts.register()
    yield
    toy_parts.unregister()


def cpu_engine(folder):
    return Engine(folder, dtype="float32", max_tokens=1024, device="cpu", kernels=TorchKernels())


@pytest.mark.parametrize("architecture", ["ToyHybridForCausalLM", "ToyTwiceForCausalLM", "ToySharedCacheForCausalLM",
                                          "ToyParallelForCausalLM", "ToyWindowedForCausalLM", "ToyOwnForCausalLM"])
def test_toy_architectures_step_like_their_plain_forms(tmp_path, architecture):
    folder = beholdd.write_random_model(str(tmp_path), toy_parts.config_dict(architecture), seed=3, dtype="float32")
    engine = toy_parts.check_architecture(architecture, folder, cpu_engine, 1e-4)
    needs = engine.model.entry_needs
    if architecture == "ToyHybridForCausalLM":
        kinds = sorted({need.kind for need in needs.values()})
        assert kinds == ["kv", "state"] and len(engine.cache.groups) == 2
        state = [g for g in engine.cache.groups if g.need.kind == "state"][0].state
        assert state.shape == (2, engine.cache.max_slots, 48)
        # the toy mixer scans a step of several tokens on the host: its decode steps may be captured, longer ones not
        assert engine.model.graph_safe and engine.model.graph_safe_rows == 1
    elif architecture == "ToyTwiceForCausalLM":
        assert sorted(needs) == [0, 1, 2, 3, 4] and engine.model.run_writes == [True] * 5
    elif architecture == "ToyWindowedForCausalLM":
        # two groups of storage, one per need; a sequence of 150 tokens keeps only the pages that its window touches there
        windows = sorted(group.need.window for group in engine.cache.groups)
        assert windows == [0, toy_parts.WINDOW] and [len(group.entries) for group in engine.cache.groups] == [2, 2]
        import schedules
        from beholdd.engine import StepEntry
        slot = engine.alloc_slot()
        engine.step([StepEntry(slot, schedules.random_requests(101, [150], seed=1)[0], [])])
        windowed = [group for group in engine.cache.groups if group.need.window][0]
        full = [group for group in engine.cache.groups if not group.need.window][0]
        assert [page >= 0 for page in windowed.pages_of[slot]] == [False, True, True] and all(page >= 0 for page in full.pages_of[slot])
        engine.free_slot(slot)
        engine.cache.check_invariants()
    elif architecture == "ToyParallelForCausalLM":
        # a norm and a block of another make in the odd layers: their own tensors are in the model folder, and the model
        # may still be captured, for steps of any number of tokens per sequence
        kinds = [type(block).__name__ for block in engine.model.blocks]
        assert kinds == ["PreNormBlock", "ToyParallelBlock"] * 2
        names = {spec.name for spec in engine.model.tensor_specs()}
        assert "model.layers.1.input_layernorm.bias" in names and "model.layers.1.post_attention_layernorm.weight" not in names
        assert engine.model.graph_safe and engine.model.graph_safe_rows > 1000
    elif architecture == "ToyOwnForCausalLM":
        # a configuration class of its own, tensors under names of its own, a routed feed-forward whose
        # experts are all in use, a rotation of part of each head
        assert not isinstance(engine.config, beholdd.Qwen3Config)
        names = {spec.name for spec in engine.model.tensor_specs()}
        assert "symbols.weight" in names and "blocks.0.routed.experts.2.down_proj.weight" in names
        assert not any(name.startswith("model.") for name in names)
        import schedules
        from beholdd.engine import StepEntry
        tokens = schedules.random_requests(90, [120], seed=4)[0]
        slot = engine.alloc_slot()
        seen = {}
        engine.step([StepEntry(slot, tokens, [])], extras=seen)
        engine.free_slot(slot)
        _, weights = toy_parts.load_plain_weights(folder)
        _, routing = toy_parts.plain_own_logits(toy_parts.OWN, weights, tokens)
        routed = [block.feed_forward for block in engine.model.blocks[::2]]
        for part, want in zip(routed, routing):
            assert part.last_routing.tolist() == want.tolist()
        # what the parts leave in the step's extras comes out of the step function: one routing row per token and layer
        assert sorted(seen["routing"]) == ["blocks.0.routed.router.weight", "blocks.2.routed.router.weight"][:len(routed)]
        assert [seen["routing"][name].tolist() for name in sorted(seen["routing"])] == [want.tolist() for want in routing]
        assert sorted(set(routing[0].tolist())) == [0, 1, 2]
    else:
        assert sorted(needs) == [0, 2] and engine.model.run_writes == [True, False, True, False]


def test_state_is_zero_when_a_slot_is_used_again(tmp_path):
    folder = beholdd.write_random_model(str(tmp_path), toy_parts.config_dict("ToyHybridForCausalLM"), seed=3,
                                        dtype="float32")
    engine = cpu_engine(folder)
    import schedules
    request = schedules.random_requests(101, [20], seed=1)
    first = schedules.whole(engine, request)[0]
    again = schedules.whole(engine, request)[0]           # the same slot, whose state the first run left non-zero
    assert torch.equal(torch.from_numpy(first), torch.from_numpy(again))


def test_a_failed_step_puts_the_state_back(tmp_path):
    """A step that fails after the state mixer has advanced its state leaves the sequence as it was: the
    retry gives bit for bit what a cache that never saw the failure gives (the rule of the key/value pages,
    crates/beholdd-model/src/qwen3moe/forward.rs:2937-2998, kept for state of fixed size)."""
    import numpy as np
    import schedules
    from beholdd.engine import StepEntry

    folder = beholdd.write_random_model(str(tmp_path), toy_parts.config_dict("ToyHybridForCausalLM"), seed=3,
                                        dtype="float32")
    tokens = schedules.random_requests(101, [30], seed=2)[0]
    for cut, rest in ((20, tokens[20:]), (29, tokens[29:])):      # a step of several tokens, and a step of one
        engine = cpu_engine(folder)
        slot, other = engine.alloc_slot(), engine.alloc_slot()
        engine.step([StepEntry(slot, tokens[:cut], []), StepEntry(other, tokens[:5], [])])
        state = [g for g in engine.cache.groups if g.need.kind == "state"][0].state
        before = state.clone()
        real, calls = engine.kernels.swiglu, {"n": 0}

        def failing(*a, **k):
            calls["n"] += 1
            if calls["n"] == 4:          # the last layer's feed-forward: both state layers have run
                raise RuntimeError("injected failure")
            return real(*a, **k)

        engine.kernels.swiglu = failing
        with pytest.raises(RuntimeError, match="injected"):
            engine.step([StepEntry(slot, rest, [len(rest) - 1])])
        engine.kernels.swiglu = real
        assert torch.equal(state, before) and engine.cache.length(slot) == cut
        retried = engine.step([StepEntry(slot, rest, [len(rest) - 1])]).numpy()
        assert not torch.equal(state[:, slot], before[:, slot]) and torch.equal(state[:, other], before[:, other])
        fresh = cpu_engine(folder)          # the same steps, none of which fails
        s2, o2 = fresh.alloc_slot(), fresh.alloc_slot()
        fresh.step([StepEntry(s2, tokens[:cut], []), StepEntry(o2, tokens[:5], [])])
        assert np.array_equal(retried, fresh.step([StepEntry(s2, rest, [len(rest) - 1])]).numpy())


def test_registering_twice_is_refused():
    with pytest.raises(ValueError, match="already registered"):
        beholdd.register_architecture("Qwen3ForCausalLM", beholdd.Qwen3Config, lambda c: None)
    with pytest.raises(ValueError, match="already registered"):
        beholdd.parts.MIXERS.register("gqa_attention", lambda *a: None)
    with pytest.raises(KeyError, match="gqa_attention"):
        beholdd.parts.MIXERS.get("no_such_mixer")


def test_a_block_joins_a_norm_to_its_neighbours_only_when_all_three_offer_it():
    """The block hands a norm to the part before it, and that part's result to the part after it, only if
    the producer prepares norms, the consumer takes prepared input and the norm can describe itself."""
    from beholdd.parts.block import PreNormBlock

    calls = []

    class Norm:
        def __init__(self, name, describes=True):
            self.name = name
            if describes:
                self.request = lambda: ("request", name)

        def forward(self, ctx, hidden):
            calls.append(("norm", self.name))
            return ("normed", self.name)

    class Part:
        def __init__(self, name, prepares, takes):
            self.name = name
            if prepares:
                self.prepares_next_norm = True
            if takes:
                self.takes_prepared_input = True

        def forward(self, ctx, x, hidden, cache=None, then_norm=None):
            calls.append((self.name, x, then_norm))
            return ("prepared by", self.name) if then_norm is not None else None

    class OldPart:          # the interface without the optional argument
        def __init__(self, name):
            self.name = name

        def forward(self, ctx, x, hidden, cache=None):
            calls.append((self.name, x, None))

    # everything offers it: one norm call (the first), the rest rides
    first = PreNormBlock(Norm("n1"), Part("mixer", True, True), Norm("n2"), Part("ff", True, True))
    second = PreNormBlock(Norm("n3"), Part("mixer2", True, True), Norm("n4"), Part("ff2", True, True))
    carried = first.forward(None, None, None, None, second)
    assert carried == ("prepared by", "ff")
    assert calls == [("norm", "n1"), ("mixer", ("normed", "n1"), ("request", "n2")),
                     ("ff", ("prepared by", "mixer"), ("request", "n3"))]
    calls.clear()
    assert second.forward(None, None, None, carried, None) is None
    assert calls == [("mixer2", ("prepared by", "ff"), ("request", "n4")), ("ff2", ("prepared by", "mixer2"), None)]

    # a norm that cannot describe itself, an old-style part, consumers that do not take prepared input
    calls.clear()
    plain = PreNormBlock(Norm("n1"), Part("mixer", True, True), Norm("n2", describes=False), OldPart("ff"))
    picky = PreNormBlock(Norm("n3"), Part("mixer2", True, False), Norm("n4"), Part("ff2", True, False))
    last = PreNormBlock(Norm("n5"), Part("mixer3", True, False), Norm("n6"), Part("ff3", False, True))
    assert plain.forward(None, None, None, None, picky) is None
    assert picky.forward(None, None, None, None, last) is None
    assert calls == [("norm", "n1"), ("mixer", ("normed", "n1"), None), ("norm", "n2"), ("ff", ("normed", "n2"), None),
                     ("norm", "n3"), ("mixer2", ("normed", "n3"), None), ("norm", "n4"), ("ff2", ("normed", "n4"), None)]
