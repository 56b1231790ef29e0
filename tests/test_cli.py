"""The command lines' argument handling (no GPU needed): every flag once, values that are not flags,
unknown arguments refused; `--plan-only` prints the byte accounting and allocates nothing."""

import io
import json
import os

import pytest

import beholdd
from beholdd import cli
from beholdd.engine import replay


def run(argv):
    out = io.StringIO()
    code = cli.main(argv, out=out)
    return code, out.getvalue()


def test_usage_and_unknown_commands(capsys):
    assert run([])[0] == 2
    code, text = run(["help"])
    assert code == 0 and "beholdd generate" in text
    assert run(["serve"])[0] == 2 and "unknown command" in capsys.readouterr().err
    code, text = run(["architectures"])
    assert code == 0 and "Qwen3ForCausalLM" in text


@pytest.mark.parametrize("argv,message", [
    (["generate"], "--model DIR is required"),
    (["generate", "--model", "x", "--model", "y"], "--model may be given once"),
    (["generate", "--model", "x", "--max-new-tokens"], "needs a value"),
    (["generate", "--model", "x", "--max-new-tokens", "--seed"], "needs a value"),
    (["generate", "--model", "x", "--bogus", "1"], "unexpected argument"),
    (["generate", "--model", "x", "stray"], "unexpected argument"),
    (["generate", "--model", "x"], "at least one non-empty prompt"),
    (["generate", "--model", "x", "--prompt-ids", "1,b"], "comma-separated list"),
    (["generate", "--model", "x", "--prompt-ids", "1,-2"], "not negative"),
    (["generate", "--model", "x", "--prompt-ids", "1", "--max-new-tokens", "many"], "not a valid int"),
    (["generate", "--model", "x", "--prompt-ids", "1", "--plan-only", "--plan-only"], "may be given once"),
    (["random-model", "--out", "x"], "needs --config FILE and --out DIR"),
])
def test_argument_errors(capsys, argv, message):
    assert run(argv)[0] == 2
    assert message in capsys.readouterr().err


def test_existing_outputs_are_never_overwritten(tmp_path, capsys, model_dirs):
    taken = tmp_path / "logits.bin"
    taken.write_bytes(b"x")
    code, _ = run(["generate", "--model", model_dirs("A"), "--prompt-ids", "1,2", "--logits-out", str(taken)])
    assert code == 2 and "never overwritten" in capsys.readouterr().err


def test_plan_only_accounts_for_bytes_without_a_gpu(model_dirs):
    code, text = run(["generate", "--model", model_dirs("B"), "--prompt-ids", "1,2,3", "--prompt-ids", "4,5",
                      "--max-new-tokens", "100", "--dtype", "bfloat16", "--plan-only"])
    assert code == 0
    # tiny B: 397,152 parameters in bfloat16; two requests of up to 103 and 102 tokens -> 2 pages each
    assert "weights: 794304 bytes" in text
    assert "cache: 4 pages of 64 tokens" in text
    # keys and values of 3 layers: 3 * 2 * 4 pages * 2 heads * 64 * 32 * 2 bytes
    assert f"{3 * 2 * 4 * 2 * 64 * 32 * 2} bytes" in text


def test_random_model_command_writes_a_loadable_folder(tmp_path, tiny_configs):
    config = tmp_path / "c.json"
    config.write_text(json.dumps(tiny_configs["A"]))
    code, text = run(["random-model", "--config", str(config), "--out", str(tmp_path / "m"), "--seed", "4"])
    assert code == 0 and sorted(os.listdir(tmp_path / "m")) == ["config.json", "model.safetensors"]
    model = beholdd.load_model(str(tmp_path / "m"), "float32", "cpu")
    assert len(model.blocks) == 2


@pytest.mark.parametrize("argv,message", [
    ([], "missing"),
    (["--model", "m", "--dtype", "float16", "--out", "o", "--max-tokens", "64"], "--dtype must be"),
    (["--model", "m", "--dtype", "float32", "--out", "o", "--max-tokens", "0"], "must be positive"),
    (["--model", "m", "--dtype", "float32", "--out", "o", "--max-tokens", "x"], "must be an integer"),
    (["--model", "m", "--model", "n", "--dtype", "float32", "--out", "o", "--max-tokens", "64"], "may be given once"),
    (["--model", "m", "--dtype", "float32", "--out", "o", "--max-tokens", "64", "--steps", "3"], "unexpected argument"),
])
def test_trace_run_arguments(capsys, argv, message):
    assert replay.main(argv, stdin=io.StringIO("")) == 2
    assert message in capsys.readouterr().err


def test_trace_replay_on_the_kernel_double(model_dirs, tmp_path):
    """The replayer's own logic (request ids to slots, files, ends) with the engine on the CPU double."""
    import numpy as np
    import plain_qwen3 as plain
    from beholdd.engine import Engine
    from kernel_emulation import TorchKernels

    folder = model_dirs("A", "float32")
    cfg, weights = plain.load_plain(folder)
    engine = Engine(folder, dtype="float32", max_tokens=128, device="cpu", kernels=TorchKernels())
    player = replay.Replayer(engine, str(tmp_path / "out"))
    a, b = [5, 17, 3, 9], [7, 8]
    player.run_step({"step": 0, "entries": [{"id": "a", "tokens": a[:3], "want": [0, 2]}, {"id": "b", "tokens": b[:1], "want": []}], "end": []})
    player.run_step({"step": 1, "entries": [{"id": "a", "tokens": a[3:], "want": [0]}, {"id": "b", "tokens": b[1:], "want": [0]}], "end": ["b"]})
    player.run_step({"step": 2, "entries": [], "end": ["a"]})
    assert sorted(os.listdir(tmp_path / "out")) == ["0.f32", "1.f32"]
    wa, wb = plain.forward_logits(cfg, weights, a), plain.forward_logits(cfg, weights, b)
    got0 = np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(-1, cfg.vocab)
    got1 = np.fromfile(tmp_path / "out" / "1.f32", dtype="<f4").reshape(-1, cfg.vocab)
    assert np.allclose(got0, wa[[0, 2]], atol=1e-4) and np.allclose(got1, np.stack([wa[3], wb[1]]), atol=1e-4)
    assert engine.cache.live_slots() == [] and player.slot_of == {}
    with pytest.raises(replay.TraceError, match="never started"):
        player.run_step({"step": 3, "entries": [], "end": ["zzz"]})
    with pytest.raises(Exception):
        player.run_step({"step": 4, "entries": [{"id": "c", "tokens": [999], "want": [0]}], "end": []})
    assert engine.cache.live_slots() == [] and "c" not in player.slot_of      # a refused start leaves no slot behind
