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


@pytest.mark.parametrize("architecture", ["ToyHybridForCausalLM", "ToyTwiceForCausalLM", "ToySharedCacheForCausalLM"])
def test_toy_architectures_step_like_their_plain_forms(tmp_path, architecture):
    folder = beholdd.write_random_model(str(tmp_path), toy_parts.config_dict(architecture), seed=3, dtype="float32")
    engine = toy_parts.check_architecture(architecture, folder, cpu_engine, 1e-4)
    needs = engine.model.entry_needs
    if architecture == "ToyHybridForCausalLM":
        kinds = sorted({need.kind for need in needs.values()})
        assert kinds == ["kv", "state"] and len(engine.cache.groups) == 2
        state = [g for g in engine.cache.groups if g.need.kind == "state"][0].state
        assert state.shape == (2, engine.cache.max_slots, 48)
    elif architecture == "ToyTwiceForCausalLM":
        assert sorted(needs) == [0, 1, 2, 3, 4] and engine.model.run_writes == [True] * 5
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


def test_registering_twice_is_refused():
    with pytest.raises(ValueError, match="already registered"):
        beholdd.register_architecture("Qwen3ForCausalLM", beholdd.Qwen3Config, lambda c: None)
    with pytest.raises(ValueError, match="already registered"):
        beholdd.parts.MIXERS.register("gqa_attention", lambda *a: None)
    with pytest.raises(KeyError, match="gqa_attention"):
        beholdd.parts.MIXERS.get("no_such_mixer")
