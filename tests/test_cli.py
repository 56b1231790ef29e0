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


def test_plan_only_holds_weights_and_cache_against_the_budget(model_dirs):
    common = ["generate", "--model", model_dirs("B", "float32"), "--prompt-ids", "1,2,3", "--max-new-tokens", "10",
              "--dtype", "bfloat16", "--plan-only", "--memory-budget-bytes"]
    # stored in 32-bit: stays so in a bfloat16 engine; one page of cache for 3 layers
    code, text = run(common + [str(10 ** 9)])
    import re
    items = {m.group(1): int(m.group(2)) for m in (re.match(r"^(\S[^:]*): (\d+) bytes", line) for line in text.splitlines()) if m}
    assert items["weights"] == 397_152 * 4 and items["cache"] == 3 * 2 * 1 * 2 * 64 * 32 * 2
    # the plan goes beyond weights and cache: the largest step's working memory, the captured decode steps, the sampler
    assert any(label.startswith("working memory of a step of 64 rows") and value > 0 for label, value in items.items())
    assert any(label.startswith("captured decode steps") and value > 0 for label, value in items.items())
    total = items.pop("total")
    assert total == sum(items.values()) and total > items["weights"] + items["cache"]
    code, text = run(common + [str(total)])
    assert code == 0 and f"total: {total} bytes (budget {total}: fits)" in text
    code, text = run(common + [str(total - 1)])
    assert code == 1 and "does not fit" in text
    # fewer rows a step, less working memory
    code, less = run(common + [str(total), "--max-rows-per-step", "16"])
    assert code == 0 and "working memory of a step of 16 rows" in less


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
    player = replay.Replayer(engine, str(tmp_path / "out"), str(tmp_path / "capture.bhdlogit"))
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
    # step numbers: integers that are not negative, each once; nothing is written for a refused one
    for bad, message in (("../../x", "non-negative integer"), (-1, "non-negative integer"), (1.5, "non-negative integer"),
                         (True, "non-negative integer"), (1, "occurs twice")):
        with pytest.raises(replay.TraceError, match=message):
            player.run_step({"step": bad, "entries": [{"id": "d", "tokens": [1], "want": [0]}], "end": ["d"]})
    assert engine.cache.live_slots() == []
    # malformed entries are refused with a reason before any request is started
    for entries, message in (([{"tokens": [1]}], "'id' and 'tokens'"), ([{"id": "e"}], "'id' and 'tokens'"), (["e"], "'id' and 'tokens'"),
                             ([{"id": "e", "tokens": 3}], "are lists"), ([{"id": "e", "tokens": [1], "want": 0}], "are lists"),
                             ([{"id": ["e"], "tokens": [1]}], "a string or an integer"),
                             ([{"id": "e", "tokens": [1]}, {"id": "e", "tokens": [2]}], "occurs twice"), ("e", "are lists")):
        with pytest.raises(replay.TraceError, match=message):
            player.run_step({"step": 6, "entries": entries, "end": []})
        assert engine.cache.live_slots() == [] and player.slot_of == {}
    # an end that cannot be is refused before anything runs: the step's own requests are not started either
    for end, message in ((["nobody"], "never started"), (["f", "f"], "ends twice"), ([["f"]], "strings or integers"), ([True], "strings or integers")):
        with pytest.raises(replay.TraceError, match=message):
            player.run_step({"step": 7, "entries": [{"id": "f", "tokens": [1, 2], "want": [1]}], "end": end})
        assert engine.cache.live_slots() == [] and player.slot_of == {} and not os.path.exists(tmp_path / "out" / "7.f32")
    # an id that is used again after its request ended is another request in the capture
    player.run_step({"step": 5, "entries": [{"id": "a", "tokens": b, "want": [1]}], "end": ["a"]})
    player.close()
    assert sorted(os.listdir(tmp_path / "out")) == ["0.f32", "1.f32", "5.f32"]
    from beholdd.engine.artifact import read_position_capture
    capture = read_position_capture(str(tmp_path / "capture.bhdlogit"))
    assert capture.requests == {"a": a, "b": b, "a#1": b}
    assert capture.rows == [("a", 0, 0), ("a", 2, 0), ("a", 3, 1), ("b", 1, 1), ("a#1", 1, 5)]
    assert np.array_equal(capture.logits[:2], got0) and np.array_equal(capture.logits[2:4], got1)
    assert np.allclose(capture.logits[4], wb[1], atol=1e-4) and capture.notes == {}
    # without a capture path the replay writes the bare rows only
    bare = replay.Replayer(engine, str(tmp_path / "bare"))
    bare.run_step({"step": 0, "entries": [{"id": "a", "tokens": a, "want": [3]}], "end": ["a"]})
    bare.close()
    assert os.listdir(tmp_path / "bare") == ["0.f32"] and engine.cache.live_slots() == []


def test_position_capture_round_trip_and_refusals(tmp_path):
    import numpy as np
    from beholdd.engine.artifact import ArtifactError, PositionCaptureWriter, read_position_capture

    path = str(tmp_path / "c.bin")
    rows = np.arange(15, dtype=np.float32).reshape(3, 5)
    writer = PositionCaptureWriter(path, 5, {"dtype": "float32"})
    assert writer.feed("long name é", [1, 2]) == 0 and writer.feed("long name é", [3]) == 2
    writer.feed("x", [4])
    writer.add(0, [("long name é", 1), ("x", 0)], rows[:2])
    with pytest.raises(ArtifactError, match="no position 3"):
        writer.add(1, [("long name é", 3)], rows[2:])
    with pytest.raises(ArtifactError, match="not finite"):
        writer.add(1, [("long name é", 2)], np.full((1, 5), np.inf, np.float32))
    writer.add(7, [("long name é", 2)], rows[2:])
    assert not os.path.exists(path)             # nothing under the final name until the capture is complete
    writer.close()
    capture = read_position_capture(path)
    assert capture.requests == {"long name é": [1, 2, 3], "x": [4]} and capture.notes == {"dtype": "float32"}
    assert capture.rows == [("long name é", 1, 0), ("x", 0, 0), ("long name é", 2, 7)]
    assert np.array_equal(capture.logits, rows)
    with pytest.raises(ArtifactError, match="never overwritten"):
        PositionCaptureWriter(path, 5)
    data = open(path, "rb").read()
    for broken, message in ((data[:-1], "bad footer"), (data[:40] + b"\x09" + data[41:], "do not agree|not a version"),
                            (data[:64] + b"\x00\x00\x80\x7f" + data[68:], "not finite"),
                            (data[:8] + b"\x01" + data[9:], "not a version-2")):
        bad = tmp_path / "bad.bin"
        bad.write_bytes(broken)
        with pytest.raises(ArtifactError, match=message):
            read_position_capture(str(bad))


def test_compare_command(tmp_path, capsys):
    import numpy as np
    from beholdd.engine.artifact import PositionCaptureWriter, write_logits_artifact

    rng = np.random.default_rng(0)
    base = {("a", i): rng.normal(size=9).astype(np.float32) for i in range(4)}
    base.update({("b", i): rng.normal(size=9).astype(np.float32) for i in range(2)})

    def make(name, order, noise=0.0, tokens_b=(6, 0)):
        writer = PositionCaptureWriter(str(tmp_path / name), 9)
        writer.feed("a", [1, 2, 3, 4])
        writer.feed("b", list(tokens_b))
        for step, places in enumerate(order):
            writer.add(step, places, np.stack([base[p] + np.float32(noise) for p in places]))
        writer.close()
        return str(tmp_path / name)

    whole = make("whole", [[("a", 0), ("a", 3)], [("b", 1)]])
    again = make("again", [[("a", 0), ("a", 3)], [("b", 1)]])
    batched = make("batched", [[("b", 1), ("a", 3)], [("a", 0)]], noise=1e-6)
    fewer = make("fewer", [[("a", 0), ("a", 3)]])
    other = make("other", [[("a", 0), ("a", 3)], [("b", 1)]], tokens_b=(6, 1))
    code, text = run(["compare", whole, again])
    assert code == 0 and "Exact logit comparison: PASS" in text and "SHA-256" in text
    code, text = run(["compare", whole, batched, "--tolerance", "1e-5"])
    assert code == 0 and "within 1e-05: PASS" in text
    for candidate, tolerance, message in ((batched, "0", "same schedule"), (batched, "1e-9", "logits differ by"),
                                          (fewer, "1e-3", "different positions"), (other, "1e-3", "tokens of request 'b'"),
                                          (str(tmp_path / "missing"), "0", "No such file")):
        code, text = run(["compare", whole, candidate, "--tolerance", tolerance])
        assert code == 1 and text.startswith("FAIL:") and message in text, text
    # equal descriptors and rows, one differing byte: the offset and both sums are reported
    data = bytearray(open(whole, "rb").read())
    data[70] ^= 1
    (tmp_path / "flipped").write_bytes(bytes(data))
    code, text = run(["compare", whole, str(tmp_path / "flipped")])
    assert code == 1 and "differ at offset 70" in text and text.count("SHA-256") == 2
    # captures of one request's generated steps compare the same way
    logits = rng.normal(size=(2, 9)).astype(np.float32)
    tokens = [int(row.argmax()) for row in logits]
    for name in ("g1", "g2"):
        write_logits_artifact(str(tmp_path / name), [1, 2], tokens, logits)
    assert run(["compare", str(tmp_path / "g1"), str(tmp_path / "g2")])[0] == 0
    assert run(["compare", str(tmp_path / "g1"), whole])[0] == 1
    assert run(["compare", whole])[0] == 2



def test_refused_values_and_missing_files_are_one_line_not_a_traceback(tmp_path, capsys, model_dirs):
    base = ["generate", "--model", model_dirs("A"), "--plan-only"]
    for extra, message in ((["--prompt-ids-file", str(tmp_path / "absent")], "No such file"),
                           (["--prompt-ids", "1,2", "--dtype", "float16"], "engine dtype must be bfloat16 or float32"),
                           (["--prompt-ids", "1,2", "--max-tokens", "-1"], "max_tokens")):
        code, _ = run(base + extra)
        error = capsys.readouterr().err
        assert code == 1 and error.startswith("error: ") and message in error and "Traceback" not in error, error
    code, _ = run(["generate", "--model", str(tmp_path / "no_model"), "--prompt-ids", "1", "--plan-only"])
    assert code == 1 and "no such file" in capsys.readouterr().err
    import torch
    if not torch.cuda.is_available():
        argv = ["--model", model_dirs("A"), "--dtype", "float32", "--out", str(tmp_path / "out"), "--max-tokens", "64"]
        assert replay.main(argv, stdin=io.StringIO("")) == 1
        assert capsys.readouterr().err.startswith("trace_run: no GPU is visible")
