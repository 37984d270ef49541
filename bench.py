"""Decode and prefill throughput of the engine on one MI355X.

Default run: the layer sizes of SmolLM2-135M (the preset ``smollm2-135m``),
random bfloat16 weights, 8 requests with 2,048-token uniform-random prompts
decoding inside a 4,096-token context.  A step is one decode step of the whole
batch through the engine's own loop: metadata, captured program, greedy pick,
tokens back on the host.  Prints ONE JSON line.
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
    from runtime.kernels import ops
    n = 2 << 30
    a = torch.empty(n, dtype=torch.uint8, device="cuda")
    a.zero_()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    ops.stream_read(a, sink)
    times = []
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ops.stream_read(a, sink)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
    return n / statistics.median(times) / 1e9


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
    ap.add_argument("--sizes", default="smollm2-1.7b:8:4096,llama-3-8b:8:8192",
                    help="further layer sizes, measured with fewer layers than their configurations have: "
                         "preset:layers:context, comma separated (empty for none); batches 1, 8 and 64 and a prompt step each")
    ap.add_argument("--contexts", default="7936:8192,32000:32768",
                    help="longer contexts of the main model: prompt:context, comma separated (empty for none); batches 8 and "
                         "64 and a prompt step each")
    ap.add_argument("--execution", default="graph", choices=["graph", "eager"])
    ap.add_argument("--overlap", type=int, default=1, choices=[0, 1],
                    help="1: picked tokens stay on the device and a step is launched before the tokens of the one "
                         "before are read, as the scheduler's overlapped ticks do; 0: every step waits for its tokens")
    ap.add_argument("--workload", default="decode", choices=["decode", "serving", "floor", "attention", "attention_forms", "decode_attention_shapes"],
                    help="decode: fixed batch after whole prompts (the default, timed per step); serving: --requests "
                         "requests with prompts of 128..--prompt tokens and --new-tokens each through the scheduler; "
                         "floor: a captured chain of kernels that do nothing (what a launch costs); attention: the attention kernel "
                         "alone over whole prompts of --attention-rows rows at the family's head shapes; attention_forms: every form "
                         "of that kernel at a grid of head shapes and --attention-rows, beside the form the engine picks; "
                         "decode_attention_shapes: every launch shape of the decode attention kernel at a grid of requests and "
                         "contexts, beside the one the engine picks")
    ap.add_argument("--attention-rows", default="2048,7936", help="attention workload: prompt lengths (comma separated)")
    ap.add_argument("--requests", type=int, default=64)
    ap.add_argument("--new-tokens", type=int, default=256)
    ap.add_argument("--token-budget", type=int, default=2112, help="serving: rows a step (a whole prompt beside 64 decoded tokens)")
    ap.add_argument("--prefill-chunk", type=int, default=2048)
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only; --gpus {args.gpus} is not run")
        return 2

    import torch
    from runtime.config import preset
    from runtime.engine import load_model, random_model, write_random_model

    if args.workload == "floor":
        return launch_floor(args)
    if args.workload == "attention_forms":
        return attention_forms(args)
    if args.workload == "decode_attention_shapes":
        return decode_attention_shapes(args)
    if args.workload == "attention":
        return prompt_attention(args)
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
        return serving(args, model, full_layers)
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
        "method": {"repeats": repeats, "statistic": "median", "ms_per_step_of_repeats": main_r["ms_all"], "clock": "host, synchronised",
                   "ms_per_step_by_gpu_events": main_r["event_ms"]},
        "reference_b1_tokens_per_s": REFERENCE_B1_TOKS,
    }
    # the same model at longer contexts: 8 and 64 requests after whole prompts, and the prompt step
    contexts = {}
    for prompt, context in longer:
        torch.cuda.empty_cache()
        n = steps_for(context, prompt)
        r, pf2, flops2 = measure(model, args, [8, 64], prompt, context, n, args.warmup, repeats)
        contexts[str(context)] = {"prompt_len": prompt, "steps": n,
                                  **{f"decode_b{b}": round(r[b]["tokens_per_s"], 1) for b in r},
                                  **{f"decode_b{b}_ms": round(r[b]["ms_per_step"], 4) for b in r},
                                  **{f"decode_b{b}_hbm_frac": round(r[b]["gbps"] / HBM_GBPS, 5) for b in r},
                                  "prefill_tokens_per_s": round(prompt / pf2, 1), "prefill_ms": round(pf2 * 1e3, 3),
                                  "prefill_frac": round(flops2 / pf2 / peak, 5)}
    if contexts:
        line["contexts"] = contexts
    # further layer sizes, with fewer layers than their configurations have (both numbers named): random weights drawn
    # on the device, batches 1, 8 and 64 after 2,048-token prompts, and the prompt step
    del model
    sizes = {}
    for item in [x for x in args.sizes.split(",") if x]:
        name, layers, context = item.split(":")
        layers, context = int(layers), int(context)
        raw = preset(name)
        of_configuration = raw["num_hidden_layers"]
        raw["num_hidden_layers"] = min(layers, of_configuration)
        raw["max_position_embeddings"] = max(raw["max_position_embeddings"], context)
        torch.cuda.empty_cache()
        other = random_model(raw, seed=0, dtype=args.dtype)
        n = steps_for(context, args.prompt)
        r, pf2, flops2 = measure(other, args, [1, 8, 64], args.prompt, context, n, args.warmup, repeats)
        sizes[name] = {"layers": raw["num_hidden_layers"], "layers_of_configuration": of_configuration, "context": context,
                       "prompt_len": args.prompt, "steps": n,
                       **{f"decode_b{b}": round(r[b]["tokens_per_s"], 1) for b in r},
                       **{f"decode_b{b}_ms": round(r[b]["ms_per_step"], 4) for b in r},
                       **{f"decode_b{b}_hbm_frac": round(r[b]["gbps"] / HBM_GBPS, 5) for b in r},
                       "prefill_tokens_per_s": round(args.prompt / pf2, 1), "prefill_ms": round(pf2 * 1e3, 3),
                       "prefill_frac": round(flops2 / pf2 / peak, 5)}
        del other
    if sizes:
        line["sizes"] = sizes
    print(json.dumps(line))
    return 0


def launch_floor(args):
    """Microseconds a kernel of a captured chain costs when it computes nothing: 1,000 launches of an empty kernel
    (one block, and one block a compute unit) in one graph, replayed; the median of 20 replays.  A decode step of
    L layers is 5 L + 4 kernels, so this times that count is the part of a step that no kernel work can remove.
    Beside it, what the other way to order a step's parts costs: a meeting of all blocks inside one kernel (counters
    in memory, 200 meetings, the median of 5 runs), alone and with 8 x 576 floats passed from all blocks to all."""
    import statistics
    import torch
    from runtime.config import preset
    from runtime.kernels import ops
    chain = 1000
    out = {}
    for name, blocks in (("one_block", 1), ("block_per_cu", torch.cuda.get_device_properties(0).multi_processor_count)):
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            ops.idle(blocks)
            stream.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                for _ in range(chain):
                    ops.idle(blocks)
        times = []
        for _ in range(20 + 3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            graph.replay()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        out[name] = round(statistics.median(times[3:]) / chain * 1e6, 3)
    # a meeting of all blocks inside one kernel, which a step fused into fewer kernels would need instead of a launch
    meeting = {}
    for name, blocks, exchange in (("128_blocks", 128, 0), ("256_blocks", 256, 0), ("256_blocks_passing_18_kb", 256, 8 * 576)):
        rounds, times = 200, []
        for _ in range(5 + 1):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            words = ops.grid_meet(blocks, rounds, exchange)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            if int(words[-1]) or int(words[0]) != rounds * (blocks // 32):
                raise SystemExit(f"grid_meet: {blocks} blocks did not all meet ({int(words[0])} arrivals, flag {int(words[-1])})")
        meeting[name] = round(statistics.median(times[1:]) / rounds * 1e6, 2)
    out["meeting_inside_a_kernel"] = meeting
    layers = preset(args.model)["num_hidden_layers"]
    kernels = 5 * layers + 4
    print(json.dumps({"metric": "microseconds a kernel that does nothing costs in a captured chain", "value": out["one_block"],
                      "unit": "us", "higher_is_better": False, "n_gpus": 1, "chain": chain, "replays": 20, "us_per_kernel": out,
                      "kernels_of_a_decode_step": kernels, "model": args.model,
                      "floor_ms_of_a_decode_step": round(kernels * out["one_block"] / 1e3, 4)}))
    return 0


def _time_attention(heads, kv_heads, D, T, P, form, calls=20):
    """Microseconds of one call of the prompt attention kernel in `form` (kind, n, halves): causal attention of T rows
    over their own T keys in a paged cache; `calls` calls in one captured graph, the median of five replays."""
    import statistics
    import numpy as np
    import torch
    from runtime.engine.context import fill_tasks
    from runtime.kernels import ops
    dev = torch.device("cuda:0")
    kind, n, halves = form
    pages = -(-T // P)
    q = torch.randn(T, heads * D, device=dev).bfloat16()
    K = torch.randn(pages, kv_heads, P, D, device=dev).bfloat16()
    V = torch.randn(pages, kv_heads, D, P, device=dev).bfloat16()
    tables = torch.arange(pages, dtype=torch.int32, device=dev).reshape(1, pages)
    seg = torch.zeros(T, dtype=torch.int32, device=dev)
    pos = torch.arange(T, dtype=torch.int32, device=dev)
    o = torch.empty(T, heads * D, device=dev, dtype=torch.bfloat16)
    rows_per_tile = (16 if kind == "tiles" else 64) * n // min(heads // kv_heads, 16)
    host = np.full((-(-T // rows_per_tile), 4), -1, dtype=np.int32)
    fill_tasks(host, [T], rows_per_tile, [0])
    tasks = torch.from_numpy(host).to(dev)

    def run():
        ops.attention_mfma(q, heads * D, K, V, tables, seg, pos, o, heads, kv_heads, D, P, None, D ** -0.5, tasks,
                           block_tiles={"tiles": False, "block": True, "square": 32}[kind], item_tiles=n, key_groups=halves)
    stream, graph = torch.cuda.Stream(), torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        run(); stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(calls):
                run()
    times = []
    for _ in range(6):
        torch.cuda.synchronize(); t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize(); times.append((time.perf_counter() - t0) / calls)
    return statistics.median(times[1:]) * 1e6


def _form_chooser():
    from runtime.engine import ModelRunner
    chooser = ModelRunner.__new__(ModelRunner)          # only its tiling rule is used
    chooser.square_tiles = chooser.block_tiles = chooser.square_halves = None
    chooser.item_tiles = 2
    return chooser


def _form_name(form):
    kind, n, halves = form
    return f"{kind} x{n}" + (", two halves" if halves == 2 else "")


def prompt_attention(args):
    """The attention kernel alone on whole prompts: causal attention of T rows over their own T keys in a paged cache, at
    the head shapes of the three family members, in the form the engine chooses for that size.  Twenty calls in one
    captured graph, the median of five replays; flops are those of the causal half, 4 T (T + 1) / 2 x head size x heads."""
    from runtime.config import preset
    P = args.page_size
    out = {}
    chooser = _form_chooser()
    for name in ("smollm2-135m", "smollm2-1.7b", "llama-3-8b"):
        raw = preset(name)
        heads, kv_heads = raw["num_attention_heads"], raw["num_key_value_heads"]
        D = raw.get("head_dim") or raw["hidden_size"] // heads
        for T in [int(t) for t in args.attention_rows.split(",") if t]:
            form = chooser.prompt_attention_form(T, 1, T, heads, kv_heads, D, P)
            us = _time_attention(heads, kv_heads, D, T, P, form)
            flops = 4 * T * (T + 1) / 2 * D * heads
            out[f"{name}_{T}"] = {"heads": heads, "kv_heads": kv_heads, "head_dim": D, "rows": T, "form": _form_name(form),
                                  "us": round(us, 1), "pflops": round(flops / us / 1e9, 3),
                                  "frac_of_bf16_peak": round(flops / us / 1e6 / PEAK_TFLOPS["bf16"], 4)}
    print(json.dumps({"metric": "prompt attention alone, PFLOP/s of the causal half (bf16, paged cache, page size %d)" % P,
                      "unit": "PFLOP/s", "n_gpus": 1, "value": out["smollm2-1.7b_%s" % args.attention_rows.split(",")[0]]["pflops"],
                      "higher_is_better": True, "shapes": out}))
    return 0


def attention_forms(args):
    """Every form of the prompt attention kernel at a grid of head shapes (heads/key heads x head size, the family's and
    others) and prompt lengths, beside the form the engine's rule picks: one line a point on stderr, then one JSON line
    with the worst and the mean loss of the rule against the best form of each point."""
    P = args.page_size
    chooser = _form_chooser()
    forms = [("tiles", 1, 1), ("tiles", 2, 1), ("block", 1, 1), ("block", 2, 1), ("square", 1, 1), ("square", 2, 1),
             ("square", 3, 1), ("square", 4, 1), ("square", 1, 2), ("square", 2, 2)]

    def takes(form, D, T):
        kind, n, halves = form
        if kind == "tiles":
            return T <= 4096 and (n == 1 or D <= 64)      # (far from the best beyond that, and slow to measure)
        return kind == "block" or D <= 64 or not (n == 4 or (n == 2 and halves == 2))
    shapes = [(9, 3, 64), (32, 32, 64), (32, 8, 128), (16, 4, 64), (12, 12, 128), (8, 8, 64), (24, 8, 96), (64, 8, 128)]
    points, losses = {}, []
    for heads, kv_heads, D in shapes:
        for T in [int(t) for t in args.attention_rows.split(",") if t]:
            us = {form: _time_attention(heads, kv_heads, D, T, P, form, calls=8) for form in forms if takes(form, D, T)}
            pick = tuple(chooser.prompt_attention_form(T, 1, T, heads, kv_heads, D, P))
            best = min(us, key=us.get)
            loss = us[pick] / us[best] - 1
            losses.append(loss)
            points[f"{heads}/{kv_heads}x{D}_{T}"] = {"pick": _form_name(pick), "pick_us": round(us[pick], 1), "best": _form_name(best),
                                                    "best_us": round(us[best], 1), "loss": round(loss, 3)}
            print(f"{heads:2d}/{kv_heads:2d} x {D:3d}  {T:5d} rows  pick {_form_name(pick):22s} {us[pick]:7.1f} us   best {_form_name(best):22s} "
                  f"{us[best]:7.1f} us   " + "  ".join(f"{_form_name(f)}: {v:.0f}" for f, v in us.items()), file=sys.stderr, flush=True)
    print(json.dumps({"metric": "loss of the rule that picks the prompt attention form against the best form of each point",
                      "unit": "fraction", "n_gpus": 1, "value": round(max(losses), 3), "higher_is_better": False,
                      "mean": round(sum(losses) / len(losses), 4), "points": points}))
    return 0


def decode_attention_shapes(args):
    """The decode attention kernel alone (one row a request, bf16, paged cache with scattered pages) at the family's head
    shapes over a grid of requests and contexts: every launch shape (wavefronts a block x blocks along the keys, with the
    merge kernel when the keys are split) beside the one `ModelRunner._rows_launch` picks.  Keys and values of up to
    eight layers take turns, so that nothing is read from a cache twice in a row.  One line a point on stderr, then one
    JSON line with the worst and the mean loss of the rule."""
    import math
    import torch
    from runtime.config import preset
    from runtime.engine import ModelRunner
    from runtime.kernels import ops
    dev, P = torch.device("cuda:0"), args.page_size
    points, losses = {}, []
    for name in ("smollm2-135m", "smollm2-1.7b", "llama-3-8b"):
        raw = preset(name)
        heads, kv = raw["num_attention_heads"], raw["num_key_value_heads"]
        D = raw.get("head_dim") or raw["hidden_size"] // heads
        group = heads // kv
        per_chunk = min(group, 16)
        for C in (512, 2048, 8192, 32768):
            for B in (1, 4, 8, 16, 32, 64, 128):
                if B * C * kv * D * 4 > 6 << 30:
                    continue
                pages_per = -(-C // P)
                n_pages = B * pages_per
                copies = int(max(1, min(8, (600 << 20) // (n_pages * kv * P * D * 4))))
                ks = [torch.randn(n_pages, kv, P, D, device=dev).bfloat16() for _ in range(copies)]
                vs = [torch.randn(n_pages, kv, D, P, device=dev).bfloat16() for _ in range(copies)]
                tables = torch.randperm(n_pages, device=dev).int().view(B, pages_per)
                q = torch.randn(B, heads * D, device=dev).bfloat16()
                seg = torch.arange(B, device=dev, dtype=torch.int32)
                pos = torch.full((B,), C - 1, device=dev, dtype=torch.int32)
                out = torch.empty(B, heads * D, device=dev).bfloat16()
                blocks = B * kv * -(-group // per_chunk)
                pick = tuple(ModelRunner._rows_launch(blocks, C, per_chunk, D))
                shapes = {(w, n) for w in (4, 8) for n in (1, 2, 4, 8, 16, 32) if (n == 1 or n * 32 <= C) and blocks * n <= 16384} | {pick}
                us = {}
                for waves, splits in sorted(shapes):
                    ws = (torch.empty(B * heads * splits * D, device=dev), torch.empty(B * heads * splits * 2, device=dev))

                    def run(i):
                        ops.attention_mfma(q, heads * D, ks[i], vs[i], tables, seg, pos, out, heads, kv, D, P, None, 1 / math.sqrt(D),
                                           None, splits, ws, waves)
                    calls = max(copies, 4)
                    for i in range(copies):
                        run(i)
                    torch.cuda.synchronize()
                    graph = torch.cuda.CUDAGraph()
                    with torch.cuda.graph(graph):
                        for i in range(calls):
                            run(i % copies)
                    graph.replay()
                    torch.cuda.synchronize()
                    times = []
                    for _ in range(3):
                        t0 = time.perf_counter()
                        graph.replay()
                        torch.cuda.synchronize()
                        times.append((time.perf_counter() - t0) / calls * 1e6)
                    us[(waves, splits)] = sorted(times)[1]
                best = min(us, key=us.get)
                loss = us[pick] / us[best] - 1
                losses.append(loss)
                label = lambda shape: f"{shape[0]} waves x {shape[1]}"
                points[f"{name}_{B}x{C}"] = {"pick": label(pick), "pick_us": round(us[pick], 1), "best": label(best),
                                             "best_us": round(us[best], 1), "loss": round(loss, 3)}
                print(f"{name:13s} {B:3d} rows x {C:5d} keys  pick {label(pick):13s} {us[pick]:7.1f} us   best {label(best):13s} {us[best]:7.1f} us   "
                      + "  ".join(f"{w}x{n}: {v:.1f}" for (w, n), v in sorted(us.items())), file=sys.stderr, flush=True)
    print(json.dumps({"metric": "loss of the rule that picks the decode attention launch shape against the best shape of each point",
                      "unit": "fraction", "n_gpus": 1, "value": round(max(losses), 3), "higher_is_better": False,
                      "mean": round(sum(losses) / len(losses), 4), "points": points}))
    return 0


def serving(args, model, full_layers):
    """Continuous batching: every request is submitted at once, the scheduler admits, cuts prompts into
    portions under the token budget, decodes and frees.  One JSON line: generated tokens a second."""
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
    t0 = time.perf_counter()
    done = engine.run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    reqs = [r for r in done if r.key.startswith("r")]
    generated = sum(len(r.generated) for r in reqs)
    assert all(r.status == "finished" and len(r.generated) == args.new_tokens for r in reqs)
    ticks = len(engine.trace) - ticks0
    ttft = sorted(r.first_token_at - t0 for r in reqs)
    line = {
        "metric": f"generated tokens/s, {args.model} layer sizes, {args.requests} requests at once, prompts of 128..{args.prompt} "
                  f"tokens, {args.new_tokens} new tokens each, continuous batching",
        "value": round(generated / elapsed, 1), "unit": "tokens/s", "n_gpus": 1, "steps": ticks, "warmup": 0,
        "ms_per_step": round(elapsed / ticks * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": args.model, "global_batch": args.requests, "seq_len": args.prompt + args.new_tokens,
                   "parallelism": "single-gpu", "layers": c.num_hidden_layers, "layers_of_configuration": full_layers,
                   "hidden": c.hidden_size, "heads": c.num_attention_heads, "kv_heads": c.num_key_value_heads,
                   "head_dim": c.head_dim, "intermediate": c.intermediate_size, "vocab": c.vocab_size,
                   "token_budget": args.token_budget, "prefill_chunk": args.prefill_chunk, "page_size": args.page_size,
                   "execution": args.execution + (", steps overlapped" if args.overlap else "")},
        "serving": {"seconds": round(elapsed, 3), "prompt_tokens": int(sum(lengths)), "generated_tokens": generated,
                    "all_tokens_per_s": round((sum(lengths) + generated) / elapsed, 1),
                    "ttft_median_ms": round(ttft[len(ttft) // 2] * 1e3, 1), "ttft_last_ms": round(ttft[-1] * 1e3, 1)},
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
