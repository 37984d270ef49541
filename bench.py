"""Decode and prefill throughput of the engine on one MI355X.

Default run: the layer sizes of SmolLM2-135M (the preset ``smollm2-135m``),
random bfloat16 weights, 8 requests with 2,048-token uniform-random prompts
decoding inside a 4,096-token context.  A step is one decode step of the whole
batch through the engine's own loop: metadata, captured program, greedy pick,
tokens back on the host.  Prints ONE JSON line: beside the headline, batches 1 and 64, the prompt step, the same
model at contexts of 8k and 32k, the layer sizes of SmolLM2-1.7B and Llama-3-8B with 8 and with all of their layers,
and continuous batching of 64 requests at the 1.7B sizes.  Before anything is timed, the tokens of the timed way of
running are compared with those of kernels launched one by one (`checked`).
"""
import argparse
import json
import sys
import tempfile
import time

HBM_GBPS = 8000.0            # MI355X published peak, GB/s
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}
REFERENCE_B1_TOKS = 203.9    # the reference's own graph-replay decode, batch 1, FP32, RTX 4060 Laptop


def sizes_of(config):
    c = config
    return (c.num_hidden_layers, c.hidden_size, c.head_dim, c.num_attention_heads, c.num_key_value_heads,
            c.intermediate_size, c.vocab_size)


def measure(model, args, batches, prompt, context, steps, warmup, repeats):
    """Decode steps of every batch size in `batches` after whole prompts of `prompt` tokens, and the prompt steps
    themselves.  Every batch is timed `repeats` times, `steps` decode steps each between synchronisations; the
    median repeat counts.  Returns {batch: {...}}, the prompt step's median seconds and its flops."""
    import statistics
    import numpy as np
    import torch
    from runtime.engine import ModelRunner, StepEntry
    from runtime.sampling import Sampler
    c = model.config
    L, H, D, nh, nkv, I, V = sizes_of(c)
    itemsize = 2 if args.dtype == "bfloat16" else 4
    sampler = Sampler()
    rng = np.random.default_rng(0)
    runner = ModelRunner(model, n_pages=-(-max(batches) * context // args.page_size), page_size=args.page_size,
                         max_requests=max(batches), execution=args.execution)
    # bytes a decode step has to read: every weight it uses once, and the cache of the live requests
    layer_params = H * (nh + 2 * nkv) * D + nh * D * H + 3 * H * I + 2 * H
    weight_bytes = (L * layer_params + V * H + H) * itemsize     # (a tied head reads the embedding matrix; the gather reads rows)
    kv_bytes_per_token = L * 2 * nkv * D * itemsize
    prefill_flops = 2 * prompt * L * (layer_params - 2 * H) + L * nh * 4 * D * prompt * (prompt + 1) / 2 + 2 * V * H
    prefill_times = []

    def timed_prefill(key, tokens):
        runner.create(key)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = runner.step([StepEntry(key, tokens, [len(tokens) - 1])])
        first = sampler.pick(logits, [(0.0, 0, 0)])[0]
        torch.cuda.synchronize()
        prefill_times.append(time.perf_counter() - t0)
        return first

    out = {}
    for batch in batches:
        keys = [f"b{batch}-{i}" for i in range(batch)]
        # token ids as they come from a tokenizer: an array
        last = [timed_prefill(key, rng.integers(0, V, size=prompt, dtype=np.int32)) for key in keys]
        params = [(0.0, 0, 0)] * batch
        unread = None

        def one():
            nonlocal last, unread
            if args.overlap:
                # the step takes its tokens from the device, where the last pick left them; the host reads
                # the tokens of the step before while this one runs
                logits = runner.step([StepEntry(k, [0], [0], pending=True) for k in keys] if unread is not None else
                                     [StepEntry(k, [t], [0]) for k, t in zip(keys, last)])
                picked = runner.pick(sampler, logits, params)
                if unread is not None:
                    last = unread.tokens()
                unread = picked
            else:
                logits = runner.step([StepEntry(k, [t], [0]) for k, t in zip(keys, last)])
                last = sampler.pick(logits, params)

        for _ in range(warmup):
            one()
        timings, event_ms = [], []
        for _ in range(repeats):
            torch.cuda.synchronize()
            ctx0 = runner.length(keys[0])
            begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            t0 = time.perf_counter()
            begin.record()
            for _ in range(steps):
                one()
            end.record()
            torch.cuda.synchronize()      # (overlapped: the tokens of the last step are read by the next repeat's first)
            timings.append((time.perf_counter() - t0, ctx0 + steps / 2))
            event_ms.append(begin.elapsed_time(end) / steps)   # the same steps by the GPU's own events
        if unread is not None:
            last, unread = unread.tokens(), None
        for key in keys:
            runner.release(key)
        elapsed, ctx_mid = sorted(timings)[len(timings) // 2]
        step_bytes = weight_bytes + batch * ctx_mid * kv_bytes_per_token
        out[batch] = {"ms_per_step": elapsed / steps * 1e3, "tokens_per_s": batch * steps / elapsed,
                      "gbps": step_bytes / (elapsed / steps) / 1e9, "ms_all": [round(t / steps * 1e3, 4) for t, _ in timings],
                      "event_ms": round(statistics.median(event_ms), 4)}
    # the prompt step: the median of all timed ones but the very first (which pays one-time set-up)
    pf = statistics.median(prefill_times[1:] if len(prefill_times) > 1 else prefill_times)
    del runner
    return out, pf, prefill_flops


def library_matmul_tflops():
    """TFLOP/s of the vendor library's bf16 product of two 8192 x 8192 matrices, the median of five: what the matrix
    cores give a large product on this GPU, beside the published peak."""
    import statistics
    import torch
    n = 8192
    a = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
    b = torch.randn(n, n, device="cuda", dtype=torch.bfloat16)
    c = torch.empty(n, n, device="cuda", dtype=torch.bfloat16)
    torch.mm(a, b, out=c)
    times = []
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        torch.mm(a, b, out=c)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return 2 * n ** 3 / statistics.median(times) / 1e12


def copy_bandwidth():
    """GB/s of a plain device-to-device copy of 1 GiB (bytes read plus bytes written), the median of five: what
    this GPU's memory gives a kernel that does nothing else, beside the published peak."""
    import statistics
    import torch
    n = 1 << 30
    a = torch.empty(n, dtype=torch.uint8, device="cuda"); b = torch.empty_like(a)
    a.zero_(); b.copy_(a)
    times = []
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        b.copy_(a)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return 2 * n / statistics.median(times) / 1e9


def read_bandwidth():
    """GB/s of a kernel that reads 2 GiB once and does nothing else (the library's own stream_read), the median of
    five: what decode steps, which read weights and cache and write next to nothing, could get from this GPU."""
    import statistics
    import torch
    from runtime import measure
    n = 2 << 30
    a = torch.empty(n, dtype=torch.uint8, device="cuda")
    a.zero_()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    measure.stream_read(a, sink)
    times = []
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        measure.stream_read(a, sink)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return n / statistics.median(times) / 1e9


def self_check(model, args, prompt, steps=16):
    """Before anything is timed: the tokens of the timed way of running (captured programs, steps overlapped, tokens
    taken from the device) against those of the plain way (kernels launched one by one, every step waiting for its
    tokens), for `--batch` requests after whole prompts, greedy (the reference asserts the same of its modes before it
    times them, benchmarks/expansion.py:118-122).  The two ways round differently in places (a captured program sizes
    its attention launches by the context's power of two), so where the plain way's two best logits lie closer than
    a hundredth of the row's spread the runs may part there; that request is compared no further.  Any other
    difference raises."""
    import numpy as np
    import torch
    from runtime.engine import ModelRunner, StepEntry
    from runtime.sampling import Sampler
    V = model.config.vocab_size
    batch = args.batch
    prompts = [np.random.default_rng(100 + i).integers(0, V, size=prompt, dtype=np.int32) for i in range(batch)]
    params = [(0.0, 0, 0)] * batch
    pages = -(-batch * (prompt + steps + 2) // args.page_size) + batch
    keys = [f"check-{i}" for i in range(batch)]

    def run(execution, overlap):
        runner = ModelRunner(model, n_pages=pages, page_size=args.page_size, max_requests=batch, execution=execution)
        sampler = Sampler()
        tokens, margins = [], []
        last = []
        for key, ids in zip(keys, prompts):
            runner.create(key)
            last.append(sampler.pick(runner.step([StepEntry(key, ids, [len(ids) - 1])]), [(0.0, 0, 0)])[0])
        tokens.append(list(last))
        unread = None
        for _ in range(steps):
            if overlap:
                logits = runner.step([StepEntry(k, [0], [0], pending=True) for k in keys] if unread is not None else
                                     [StepEntry(k, [t], [0]) for k, t in zip(keys, last)])
                picked = runner.pick(sampler, logits, params)
                if unread is not None:
                    tokens.append(unread.tokens())
                unread = picked
            else:
                logits = runner.step([StepEntry(k, [t], [0]) for k, t in zip(keys, last)])
                top = torch.topk(logits, 2, dim=-1).values
                spread = (top[:, 0] - logits.median(dim=-1).values).clamp_min(1e-30)
                margins.append(((top[:, 0] - top[:, 1]) / spread).cpu().tolist())
                last = sampler.pick(logits, params)
                tokens.append(list(last))
        if unread is not None:
            tokens.append(unread.tokens())
        for key in keys:
            runner.release(key)
        return tokens, margins

    plain, margins = run("eager", False)
    timed, _ = run(args.execution, bool(args.overlap))
    same = ties = 0
    for r in range(batch):
        for step in range(steps + 1):
            if plain[step][r] == timed[step][r]:
                same += 1
                continue
            if step >= 1 and margins[step - 1][r] < 0.01:
                ties += 1
                break
            raise SystemExit(f"self-check failed: request {r} step {step}: token {timed[step][r]} in the timed way of running, "
                             f"{plain[step][r]} kernel by kernel")
    return {"requests": batch, "prompt_len": prompt, "steps": steps, "tokens_equal": same, "parted_at_near_ties": ties}


def summary(r, prompt, pf, flops, peak):
    return {**{f"decode_b{b}": round(r[b]["tokens_per_s"], 1) for b in r},
            **{f"decode_b{b}_ms": round(r[b]["ms_per_step"], 4) for b in r},
            **{f"decode_b{b}_hbm_frac": round(r[b]["gbps"] / HBM_GBPS, 5) for b in r},
            "prefill_tokens_per_s": round(prompt / pf, 1), "prefill_ms": round(pf * 1e3, 3),
            "prefill_frac": round(flops / pf / peak, 5)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--repeats", type=int, default=3, help="timed repeats of --steps decode steps; the median counts")
    ap.add_argument("--model", default="smollm2-135m")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration (reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--points", default="1,64", help="other batch sizes to time (comma separated, empty for none)")
    ap.add_argument("--sizes", default="smollm2-1.7b:8:4096,llama-3-8b:8:8192,smollm2-1.7b:24:4096,llama-3-8b:32:8192",
                    help="further layer sizes: preset:layers:context, comma separated (empty for none), with fewer layers than "
                         "the configuration or all of them (both numbers are reported); batches 1, 8 and 64 and a prompt step each")
    ap.add_argument("--contexts", default="7936:8192,32000:32768",
                    help="longer contexts of the main model: prompt:context, comma separated (empty for none); batches 8 and "
                         "64 and a prompt step each")
    ap.add_argument("--serving", default="smollm2-1.7b",
                    help="decode workload: the preset (all of its layers) that also runs the serving workload, reported under "
                         "`serving` (empty for none)")
    ap.add_argument("--execution", default="graph", choices=["graph", "eager"])
    ap.add_argument("--overlap", type=int, default=1, choices=[0, 1],
                    help="1: picked tokens stay on the device and a step is launched before the tokens of the one "
                         "before are read, as the scheduler's overlapped ticks do; 0: every step waits for its tokens")
    ap.add_argument("--workload", default="decode", choices=["decode", "serving"],
                    help="decode: fixed batches after whole prompts, timed per step (the default; its line also holds longer "
                         "contexts, further layer sizes and one serving run); serving: only --requests requests with prompts of "
                         "128..--prompt tokens and --new-tokens each through the scheduler, at --model's sizes")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--token-budget", type=int, default=2112, help="serving: rows a step (a whole prompt beside 64 decoded tokens)")
    ap.add_argument("--prefill-chunk", type=int, default=2048)
    ap.add_argument("--check", type=int, default=1, choices=[0, 1], help="compare the timed way of running with the plain one first")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only; --gpus {args.gpus} is not run")
        return 2

    import torch
    from runtime.config import preset
    from runtime.engine import load_model, random_model, write_random_model

    raw = preset(args.model)
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    longer = [tuple(int(x) for x in item.split(":")) for item in args.contexts.split(",") if item] if args.workload == "decode" else []
    raw["max_position_embeddings"] = max([raw["max_position_embeddings"], args.context] + [context for _, context in longer])
    folder = tempfile.mkdtemp(prefix="bench-model-")
    write_random_model(folder, raw, seed=0, dtype="bfloat16")
    model = load_model(folder, dtype=args.dtype)
    c = model.config
    if args.workload == "serving":
        print(json.dumps(serving(args, model, args.model, full_layers)))
        return 0
    checked = self_check(model, args, args.prompt) if args.check else None
    batches = [args.batch] + [int(b) for b in args.points.split(",") if b]
    repeats = max(1, args.repeats)

    def steps_for(context, prompt):
        return max(1, min(args.steps, (context - prompt - args.warmup - 1) // repeats))

    steps = steps_for(args.context, args.prompt)
    results, pf, pf_flops = measure(model, args, batches, args.prompt, args.context, steps, args.warmup, repeats)
    L, H, D, nh, nkv, I, V = sizes_of(c)
    main_r = results[args.batch]
    peak = PEAK_TFLOPS["bf16" if args.dtype == "bfloat16" else "fp32"] * 1e12
    copy_gbps = copy_bandwidth()
    read_gbps = read_bandwidth()
    matmul_tflops = library_matmul_tflops()
    points = {f"decode_b{b}": round(results[b]["tokens_per_s"], 1) for b in batches if b != args.batch}
    line = {
        "metric": f"decode tokens/s, {args.model} layer sizes, batch {args.batch}, {args.prompt}-token prompts in a {args.context} context",
        "value": round(main_r["tokens_per_s"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(main_r["ms_per_step"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": args.model, "global_batch": args.batch, "seq_len": args.context, "prompt_len": args.prompt,
                   "parallelism": "single-gpu", "layers": L, "layers_of_configuration": full_layers, "hidden": H,
                   "heads": nh, "kv_heads": nkv, "head_dim": D, "intermediate": I, "vocab": V,
                   "rope_theta": c.rope_theta, "rms_norm_eps": c.rms_norm_eps, "tied_head": c.tie_word_embeddings,
                   "page_size": args.page_size, "execution": args.execution + (", steps overlapped" if args.overlap else "")},
        "prefill": {"value": round(args.prompt / pf, 1), "tokens": args.prompt, "ms": round(pf * 1e3, 3),
                    "frac": round(pf_flops / pf / peak, 5), "peak_tflops": peak / 1e12,
                    "measured_library_matmul_tflops": round(matmul_tflops, 1)},
        "roofline": {"bound": "hbm", "achieved": round(main_r["gbps"], 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(main_r["gbps"] / HBM_GBPS, 5), "measured_copy": round(copy_gbps, 1), "measured_read": round(read_gbps, 1)},
        "points": points,
        "points_roofline_frac": {f"decode_b{b}": round(results[b]["gbps"] / HBM_GBPS, 5) for b in batches if b != args.batch},
        "checked": checked is not None,
        "method": {"repeats": repeats, "statistic": "median", "ms_per_step_of_repeats": main_r["ms_all"], "clock": "host, synchronised",
                   "ms_per_step_by_gpu_events": main_r["event_ms"], "self_check": checked},
        "reference_b1_tokens_per_s": REFERENCE_B1_TOKS,
    }
    # the same model at longer contexts: 8 and 64 requests after whole prompts, and the prompt step
    contexts = {}
    for prompt, context in longer:
        torch.cuda.empty_cache()
        n = steps_for(context, prompt)
        r, pf2, flops2 = measure(model, args, [8, 64], prompt, context, n, args.warmup, repeats)
        contexts[str(context)] = {"prompt_len": prompt, "steps": n, **summary(r, prompt, pf2, flops2, peak)}
    if contexts:
        line["contexts"] = contexts
    # further layer sizes, with some or all of their layers (both numbers named): random weights drawn on the device,
    # batches 1, 8 and 64 after 2,048-token prompts, and the prompt step; the serving workload runs on the model that
    # has all the layers of its configuration
    del model
    sizes = {}
    for item in [x for x in args.sizes.split(",") if x]:
        name, layers, context = item.split(":")
        layers, context = int(layers), int(context)
        raw = preset(name)
        of_configuration = raw["num_hidden_layers"]
        raw["num_hidden_layers"] = min(layers, of_configuration)
        raw["max_position_embeddings"] = max(raw["max_position_embeddings"], context, args.prompt + args.new_tokens)
        torch.cuda.empty_cache()
        other = random_model(raw, seed=0, dtype=args.dtype)
        n = steps_for(context, args.prompt)
        r, pf2, flops2 = measure(other, args, [1, 8, 64], args.prompt, context, n, args.warmup, repeats)
        sizes[f"{name}:{raw['num_hidden_layers']}"] = {"layers": raw["num_hidden_layers"], "layers_of_configuration": of_configuration,
                                                     "context": context, "prompt_len": args.prompt, "steps": n,
                                                     **summary(r, args.prompt, pf2, flops2, peak)}
        if name == args.serving and raw["num_hidden_layers"] == of_configuration and "serving" not in line:
            torch.cuda.empty_cache()
            run = serving(args, other, name, of_configuration)
            line["serving"] = {"metric": run["metric"], "value": run["value"], "unit": run["unit"], "ticks": run["steps"],
                               "layers": of_configuration, **run["serving"], "programs": run["programs"]}
        del other
    if sizes:
        line["sizes"] = sizes
    print(json.dumps(line))
    return 0


def serving(args, model, name, full_layers):
    """Continuous batching: every request is submitted at once, the scheduler admits, cuts prompts into
    portions under the token budget, decodes and frees.  Returns the line of the run: generated tokens a second."""
    import numpy as np
    import torch
    from runtime.engine import ModelRunner
    from runtime.engine.scheduler import Engine, Request
    c = model.config
    rng = np.random.default_rng(0)
    lengths = rng.integers(128, args.prompt + 1, size=args.requests).tolist()
    pages = sum(-(-(n + args.new_tokens) // args.page_size) for n in lengths) + 8
    runner = ModelRunner(model, n_pages=pages, page_size=args.page_size, max_requests=args.requests, execution=args.execution)
    engine = Engine(runner, max_active=args.requests, token_budget=args.token_budget, prefill_chunk=args.prefill_chunk,
                    overlap=bool(args.overlap),
                    policy="decode_first")
    # warm-up: a short run of the same shape of work compiles nothing new but fills the workspace
    for i in range(2):
        engine.submit(Request(f"warm{i}", rng.integers(0, c.vocab_size, size=args.prefill_chunk + 3).tolist(), 4))
    engine.run()
    for i, n in enumerate(lengths):
        engine.submit(Request(f"r{i}", rng.integers(0, c.vocab_size, size=n).tolist(), args.new_tokens))
    torch.cuda.synchronize()
    ticks0 = len(engine.trace)
    before = dict(runner.counters)
    t0 = time.perf_counter()
    done = engine.run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    reqs = [r for r in done if r.key.startswith("r")]
    generated = sum(len(r.generated) for r in reqs)
    assert all(r.status == "finished" and len(r.generated) == args.new_tokens for r in reqs)
    ticks = len(engine.trace) - ticks0
    ttft = sorted(r.first_token_at - t0 for r in reqs)
    report = runner.report()
    return {
        "metric": f"generated tokens/s, {name} layer sizes, {args.requests} requests at once, prompts of 128..{args.prompt} "
                  f"tokens, {args.new_tokens} new tokens each, continuous batching",
        "value": round(generated / elapsed, 1), "unit": "tokens/s", "n_gpus": 1, "steps": ticks, "warmup": 0,
        "ms_per_step": round(elapsed / ticks * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": name, "global_batch": args.requests, "seq_len": args.prompt + args.new_tokens,
                   "parallelism": "single-gpu", "layers": c.num_hidden_layers, "layers_of_configuration": full_layers,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": c.head_dim, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "token_budget": args.token_budget, "prefill_chunk": args.prefill_chunk, "page_size": args.page_size,
                   "execution": args.execution + (", steps overlapped" if args.overlap else "")},
        "serving": {"seconds": round(elapsed, 3), "prompt_tokens": int(sum(lengths)), "generated_tokens": generated,
                    "all_tokens_per_s": round((sum(lengths) + generated) / elapsed, 1),
                    "ttft_median_ms": round(ttft[len(ttft) // 2] * 1e3, 1), "ttft_last_ms": round(ttft[-1] * 1e3, 1)},
        # captured programs of the timed run: how many steps replayed one, how many were recorded or run kernel by kernel, evicted
        "programs": {k: report[k] - before.get(k, 0) for k in ("steps", "replays", "captures", "eager_steps", "evictions")},
    }


if __name__ == "__main__":
    sys.exit(main())
