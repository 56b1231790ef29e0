"""Decode and prefill throughput of the Qwen3-8B shape with random bfloat16 weights on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C] [--shape 8b|14b|32b]

A step is one decode step of the batch: every live sequence's next token through the whole
model, logits of each and a greedy choice.  The sequences' caches are filled with random keys
and values to just under the context length, so the timed steps read a full-length cache and
end exactly at the context length.  Prints one JSON line.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0            # MI355X HBM3E
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

QWEN3_8B = {
    "architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "num_hidden_layers": 36, "hidden_size": 4096,
    "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128, "intermediate_size": 12288,
    "vocab_size": 151936, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 40960,
    "tie_word_embeddings": False,
}


# The other shapes of the family, for measurements beside the default one (--shape).
QWEN3_14B = dict(QWEN3_8B, num_hidden_layers=40, hidden_size=5120, num_attention_heads=40, intermediate_size=17408)
QWEN3_32B = dict(QWEN3_8B, num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, intermediate_size=25600)
SHAPES = {"8b": ("Qwen3-8B shape", QWEN3_8B), "14b": ("Qwen3-14B shape", QWEN3_14B), "32b": ("Qwen3-32B shape", QWEN3_32B)}


def parse():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=32)
    parser.add_argument("--warmup", type=int, default=4)
    parser.add_argument("--shape", default="8b", choices=sorted(SHAPES), help="layer sizes; the default is the benchmark's")
    parser.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has")
    parser.add_argument("--batch", type=int, default=8)
    parser.add_argument("--context", type=int, default=8192)
    parser.add_argument("--prefill-tokens", type=int, default=2048)
    parser.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    parser.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 decode points")
    parser.add_argument("--workload", action="store_true",
                        help="instead of the step timings, generate through the engine's own loop for the batch the shape's "
                             "benchmark configuration names (8b: 8 prompts of 256 to 1,024 tokens up to the context; 14b: 16 "
                             "prompts of 64 to 4,096 tokens, 256 greedy tokens each; 32b: 32 prompts of 128 to 8,192 tokens, "
                             "128 tokens each at temperature 1) and print its tokens per second")
    parser.add_argument("--hbm-ceiling", action="store_true",
                        help="measure what a plain streaming read and a copy of 8 GB reach on this GPU, print it and exit")
    parser.add_argument("--sampling", action="store_true",
                        help="time the selection kernel on 1, 8 and 64 rows of 151,936 logits (greedy, at a temperature, with "
                             "top-k, with top-p on rows of three spreads, with both), print the microseconds and exit")
    return parser.parse_args()


def fill_cache(engine, slots, length, torch):
    """Give each slot `length` tokens of random keys and values without running the model."""
    requests = [(slot, length) for slot in slots]
    engine.cache.reserve(requests)
    engine.cache.commit(requests)


def randomise_cache(engine, torch):
    generator = torch.Generator(device=engine.device).manual_seed(1)
    for group in engine.cache.groups:
        if group.k is not None:
            for tensor in (group.k, group.v):
                for layer in range(tensor.shape[0]):
                    tensor[layer].normal_(0.0, 1.0, generator=generator)


def decode_run(engine, batch, context, steps, warmup, torch):
    """Time `steps` decode steps of `batch` sequences that end at `context` tokens."""
    from beholdd.engine import StepEntry, decode_ahead
    from beholdd.sampling import SamplingParams

    start = context - steps - warmup - 1
    slots = [engine.alloc_slot() for _ in range(batch)]
    fill_cache(engine, slots, start, torch)
    greedy = [SamplingParams()] * batch
    tokens = [(7 * i + 3) % engine.model.vocab for i in range(batch)]

    # The generation loop's own way of stepping (engine/generation.py: decode_ahead): the next step is started
    # with the tokens still on the device, then the host reads the tokens chosen before it.
    requests = list(range(batch))
    logits = engine.step([StepEntry(slot, [token], [0]) for slot, token in zip(slots, tokens)])
    chosen = engine.select_async(logits, greedy, requests, [0] * batch)

    def one(step):
        nonlocal chosen
        ahead = decode_ahead(engine, slots, chosen, greedy, requests, [step + 1] * batch)
        chosen.result()
        chosen = ahead

    for step in range(warmup):
        one(step)
    chosen.result()
    torch.cuda.synchronize()
    begin = time.perf_counter()
    for step in range(steps):
        one(warmup + step)
    chosen.result()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - begin
    lengths = [engine.cache.length(slot) for slot in slots]
    for slot in slots:
        engine.free_slot(slot)
    mean_length = sum(lengths) / batch - steps / 2.0
    return elapsed / steps, mean_length


def prefill_run(engine, n_tokens, torch, repeats=3, prompts=1, host=False):
    """Seconds of one step that brings `prompts` prompts of `n_tokens` tokens each (the best of `repeats`); with
    `host` also the seconds until the step function returns, the device still busy."""
    from beholdd.engine import StepEntry
    tokens = [(31 * i + 5) % engine.model.vocab for i in range(n_tokens)]
    times, returned = [], []
    for _ in range(repeats + 1):          # the first run warms up and is dropped
        slots = [engine.alloc_slot() for _ in range(prompts)]
        torch.cuda.synchronize()
        begin = time.perf_counter()
        engine.step([StepEntry(slot, tokens, [n_tokens - 1]) for slot in slots])
        returned.append(time.perf_counter() - begin)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - begin)
        for slot in slots:
            engine.free_slot(slot)
    return (min(times[1:]), min(returned[1:])) if host else min(times[1:])


# Batches of the benchmark configurations: (prompts, shortest, longest, new tokens, temperature, context).
WORKLOADS = {"8b": (8, 256, 1024, 256, 0.0, 8192), "14b": (16, 64, 4096, 256, 0.0, 8192),
             "32b": (32, 128, 8192, 128, 1.0, 16384)}


def workload_run(engine, shape, torch):
    """Unequal prompts through `Engine.generate` (prompts in one step, then a token each, sequences that end
    give their slots back): what a user of the library gets, host loop and sampling included."""
    import random
    count, shortest, longest, new_tokens, temperature, _ = WORKLOADS[shape]
    rng = random.Random(0)
    lengths = [rng.randint(shortest, longest) for _ in range(count)]
    prompts = [[rng.randrange(engine.model.vocab) for _ in range(n)] for n in lengths]
    engine.generate(prompts, max_new_tokens=4)          # warms up: the graph of this batch size and page-table width is captured
    torch.cuda.synchronize()
    begin = time.perf_counter()
    results = engine.generate(prompts, max_new_tokens=new_tokens, temperature=temperature, seed=1)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - begin
    generated = sum(len(r.token_ids) for r in results)
    return {"prompts": count, "prompt_tokens": sum(lengths), "generated_tokens": generated,
            "seconds": round(elapsed, 3), "generated_tok_per_s": round(generated / elapsed, 1),
            "all_tok_per_s": round((generated + sum(lengths)) / elapsed, 1), "temperature": temperature}


def hbm_ceiling(torch):
    """What kernels that only stream memory reach here: torch's sum over 8 GB (read) and copy of 8 GB (read +
    write), and the library's own yardstick kernel, which reads 8 GB the way its weight and cache streams do
    (256 and 512 workgroups, with and without the streaming hint).  Not part of the product path; a yardstick
    for the roofline fractions."""
    from beholdd.kernels import HipKernels

    x = torch.empty(2 << 30, dtype=torch.float32, device="cuda:0").normal_()
    y = torch.empty_like(x)
    kernels = HipKernels("cuda:0")
    out = {}
    runs = [("hbm_read_GBs", lambda: x.sum(), x.numel() * 4), ("hbm_copy_GBs", lambda: y.copy_(x), 2 * x.numel() * 4)]
    for workgroups in (256, 512):
        for hint in (True, False):
            name = f"stream_read_{workgroups}wg_{'streaming' if hint else 'plain'}_GBs"
            runs.append((name, lambda w=workgroups, h=hint: kernels.stream_read(x, w, h), x.numel() * 4))
    for name, run, moved in runs:
        run()
        torch.cuda.synchronize()
        begin = time.perf_counter()
        for _ in range(10):
            run()
        torch.cuda.synchronize()
        out[name] = round(moved * 10 / (time.perf_counter() - begin) / 1e9, 1)
    return out


def sampling_times(torch):
    """Microseconds of one selection over rows of the benchmark's vocabulary, each mode replayed ten times from a
    captured graph so that the launches' host cost stays out."""
    from beholdd.kernels import HipKernels

    kernels, vocab, out = HipKernels("cuda:0"), QWEN3_8B["vocab_size"], {}
    for rows in (1, 8, 64):
        logits = torch.randn(rows, vocab, device="cuda:0") * 3
        tokens = torch.empty(rows, dtype=torch.int32, device="cuda:0")
        bad = torch.empty_like(tokens)
        temperature, uniform = torch.full((rows,), 0.8, device="cuda:0"), torch.rand(rows, device="cuda:0")
        top_k = torch.full((rows,), 50, dtype=torch.int32, device="cuda:0")
        top_p = torch.full((rows,), 0.9, device="cuda:0")
        # (top-p's share of these rows is a thousand tokens or so; of the "peaked" rows, three times the spread, under a
        # hundred, as of a trained model's mostly; of the "wide" rows, a sixth of the spread, most of the vocabulary)
        usual, peaked, wide = logits, logits * 3, logits / 6
        modes = {"greedy": {}, "temperature": dict(temperature=temperature, uniform=uniform),
                 "top_k": dict(temperature=temperature, uniform=uniform, top_k=top_k),
                 "top_p": dict(temperature=temperature, uniform=uniform, top_p=top_p),
                 "top_p_peaked": dict(temperature=temperature, uniform=uniform, top_p=top_p),
                 "top_p_wide": dict(temperature=temperature, uniform=uniform, top_p=top_p),
                 "top_k_top_p": dict(temperature=temperature, uniform=uniform, top_k=top_k, top_p=top_p)}
        for name, arguments in modes.items():
            logits = peaked if name.endswith("peaked") else wide if name.endswith("wide") else usual
            kernels.sample(logits, tokens, bad, **arguments)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(10):
                    kernels.sample(logits, tokens, bad, **arguments)
            graph.replay()
            torch.cuda.synchronize()
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            begin.record()
            graph.replay()
            end.record()
            torch.cuda.synchronize()
            out[f"rows_{rows}_{name}_us"] = round(begin.elapsed_time(end) * 100, 1)
    return out


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU library")
        return 2
    import torch
    if args.hbm_ceiling:
        print(json.dumps(hbm_ceiling(torch)))
        return 0
    if args.sampling:
        print(json.dumps(sampling_times(torch)))
        return 0

    from beholdd.engine import Engine, random_model_on_device

    shape_name, shape = SHAPES[args.shape]
    config = dict(shape, num_hidden_layers=args.layers or shape["num_hidden_layers"])
    device = "cuda:0"
    dtype_tag = "bf16" if args.dtype == "bfloat16" else "fp32"
    element = 2 if args.dtype == "bfloat16" else 4
    model = random_model_on_device(config, seed=0, dtype=args.dtype, device=device)
    biggest = 1 if args.no_points else 64
    if args.workload:
        count, _, longest, new_tokens, _, context = WORKLOADS[args.shape]
        engine = Engine(model=model, dtype=args.dtype, max_tokens=count * (-(-(longest + new_tokens) // 64) * 64),
                        max_slots=count, device=device)
        line = {"metric": f"generation of the {shape_name} batch", "unit": "tok/s", "dtype": dtype_tag,
                "layers": config["num_hidden_layers"], "layers_of_full_model": shape["num_hidden_layers"], "context": context}
        line.update(workload_run(engine, args.shape, torch))
        line["value"] = line["generated_tok_per_s"]
        print(json.dumps(line))
        return 0
    max_tokens = max(args.batch, biggest) * (-(-args.context // 64) * 64)
    engine = Engine(model=model, dtype=args.dtype, max_tokens=max_tokens, max_slots=max(args.batch, biggest, 64),
                    device=device)
    randomise_cache(engine, torch)
    cfg = engine.config

    layer_params = (cfg.hidden * (cfg.q_width + 2 * cfg.kv_width) + cfg.q_width * cfg.hidden
                    + 3 * cfg.hidden * cfg.intermediate)
    weight_bytes = (cfg.n_layers * layer_params + cfg.vocab * cfg.hidden) * element
    kv_bytes_per_token = cfg.n_layers * 2 * cfg.kv_width * element

    seconds, mean_length = decode_run(engine, args.batch, args.context, args.steps, args.warmup, torch)
    step_bytes = weight_bytes + args.batch * mean_length * kv_bytes_per_token
    achieved = step_bytes / seconds / 1e9
    value = args.batch / seconds

    t = min(args.prefill_tokens, args.context)      # (a context shorter than the prompt: a prompt of the context's length)
    prefill_seconds = prefill_run(engine, t, torch)
    prefill_flops = (2.0 * cfg.n_layers * layer_params * t + cfg.n_layers * cfg.n_heads * 2.0 * t * t * cfg.head_dim
                     + 2.0 * cfg.vocab * cfg.hidden)
    # Other batch sizes and contexts: tokens a second, and beside each the fraction of the HBM peak that the
    # bytes of its step (all weights once, the live requests' caches) amount to.
    points, fractions = {}, {}
    if not args.no_points:
        for batch, context, name in ((1, args.context, "decode_b1"), (64, args.context, "decode_b64"),
                                     (1, 512, "decode_b1_ctx512"), (1, 2048, "decode_b1_ctx2048"),
                                     (8, 640, "decode_b8_ctx640"), (64, 640, "decode_b64_ctx640")):
            steps = max(4, args.steps // 2)
            s, length = decode_run(engine, batch, context, steps, 2, torch)
            points[name] = round(batch / s, 2)
            fractions[name] = round((weight_bytes + batch * length * kv_bytes_per_token) / s / 1e9 / PEAK_HBM_GBS, 4)
    # Prompts of other lengths: tokens a second and the fraction of the matrix-core peak; for the short ones, which
    # the host's launches bound, also the milliseconds until the step function returns.
    prefill_points = {}
    if not args.no_points:
        def flops(tokens, prompts=1):
            return prompts * (2.0 * cfg.n_layers * layer_params * tokens + cfg.n_layers * cfg.n_heads * 2.0 * tokens * tokens * cfg.head_dim
                              + 2.0 * cfg.vocab * cfg.hidden)
        for tokens in (16, 64, 128):
            seconds_all, seconds_host = prefill_run(engine, tokens, torch, host=True)
            prefill_points[f"tokens_{tokens}"] = {"ms": round(seconds_all * 1e3, 3), "host_ms": round(seconds_host * 1e3, 3),
                                                  "tok_per_s": round(tokens / seconds_all, 1)}
        for tokens, prompts in ((512, 1), (1024, 1), (4096, 1), (8192, 1), (2048, 4)):
            if tokens > args.context:
                continue
            seconds_all = prefill_run(engine, tokens, torch, repeats=2, prompts=prompts)
            name = f"tokens_{tokens}" if prompts == 1 else f"prompts_{prompts}x{tokens}"
            prefill_points[name] = {"ms": round(seconds_all * 1e3, 3), "tok_per_s": round(prompts * tokens / seconds_all, 1),
                                    "frac": round(flops(tokens, prompts) / seconds_all / PEAK_FLOPS[dtype_tag], 4)}
    generated = None
    if not args.no_points and args.shape == "8b":
        generated = workload_run(engine, args.shape, torch)     # the same batch through Engine.generate

    # what a kernel that does nothing but read reaches on this GPU (the library's yardstick kernel over 4 GB of the cache)
    cache_tensor = engine.cache.groups[0].k
    span = cache_tensor.view(-1)[: min(cache_tensor.numel(), 2 << 30)]
    yardstick = None
    if span.numel() * span.element_size() >= 256 << 20:      # (a cache of a few MB says nothing about streaming)
        engine.kernels.stream_read(span)
        torch.cuda.synchronize()
        begin = time.perf_counter()
        read = sum(engine.kernels.stream_read(span) for _ in range(4))
        torch.cuda.synchronize()
        yardstick = read / (time.perf_counter() - begin) / 1e9

    line = {
        "metric": f"decode tok/s @ batch {args.batch} ({shape_name}, context {args.context})", "value": round(value, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(seconds * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype_tag,
        "data": "synthetic: seeded random weights, random token ids, caches filled with random keys and values",
        "config": {
            "model": shape_name, "layers": cfg.n_layers, "layers_of_full_model": shape["num_hidden_layers"],
            "hidden_size": cfg.hidden, "num_attention_heads": cfg.n_heads, "num_key_value_heads": cfg.n_kv_heads,
            "head_dim": cfg.head_dim, "intermediate_size": cfg.intermediate, "vocab_size": cfg.vocab,
            "rope_theta": cfg.rope_theta, "rms_norm_eps": cfg.rms_eps, "tie_word_embeddings": cfg.tie_word_embeddings,
            "global_batch": args.batch, "seq_len": args.context, "prefill_tokens": t, "parallelism": "single GPU",
        },
        "prefill": {"value": round(t / prefill_seconds, 1), "tokens": t, "ms": round(prefill_seconds * 1e3, 3),
                    "frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS[dtype_tag], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4), "plain_read_GBs": round(yardstick, 1) if yardstick is not None else None},
        "points": points,
        "points_hbm_frac": fractions,
    }
    if prefill_points:
        line["prefill_points"] = prefill_points
    if generated is not None:
        line["generate"] = generated
    if not args.no_points and args.shape == "8b" and args.layers is None and args.dtype == "bfloat16":
        # the other two shapes of the family, full depth: decode at batch 8 and the prompt of 2,048 tokens
        del engine, model, cache_tensor, span
        line["shapes"] = {name: other_shape(name, args, torch) for name in ("14b", "32b")}
    print(json.dumps(line))
    return 0


def other_shape(name, args, torch):
    import gc

    from beholdd.engine import Engine, random_model_on_device
    gc.collect()
    torch.cuda.empty_cache()
    config = SHAPES[name][1]
    model = random_model_on_device(dict(config), seed=0, dtype="bfloat16", device="cuda:0")
    engine = Engine(model=model, dtype="bfloat16", max_tokens=8 * (-(-args.context // 64) * 64), max_slots=8, device="cuda:0")
    randomise_cache(engine, torch)
    cfg = engine.config
    layer_params = (cfg.hidden * (cfg.q_width + 2 * cfg.kv_width) + cfg.q_width * cfg.hidden + 3 * cfg.hidden * cfg.intermediate)
    weight_bytes = (cfg.n_layers * layer_params + cfg.vocab * cfg.hidden) * 2
    kv_bytes_per_token = cfg.n_layers * 2 * cfg.kv_width * 2
    steps = max(4, args.steps // 2)
    seconds, mean_length = decode_run(engine, 8, args.context, steps, 2, torch)
    t = min(args.prefill_tokens, args.context)
    prefill_seconds = prefill_run(engine, t, torch, repeats=2)
    prefill_flops = (2.0 * cfg.n_layers * layer_params * t + cfg.n_layers * cfg.n_heads * 2.0 * t * t * cfg.head_dim
                     + 2.0 * cfg.vocab * cfg.hidden)
    out = {"layers": cfg.n_layers, "decode_b8_tok_per_s": round(8 / seconds, 2), "decode_b8_ms": round(seconds * 1e3, 4),
           "decode_b8_hbm_frac": round((weight_bytes + 8 * mean_length * kv_bytes_per_token) / seconds / 1e9 / PEAK_HBM_GBS, 4),
           "prefill_tok_per_s": round(t / prefill_seconds, 1), "prefill_ms": round(prefill_seconds * 1e3, 3),
           "prefill_frac": round(prefill_flops / prefill_seconds / PEAK_FLOPS["bf16"], 4)}
    del engine, model
    gc.collect()
    torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    sys.exit(main())
