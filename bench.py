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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--model", default="smollm2-135m")
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration (reported)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--points", default="1,64", help="other batch sizes to time (comma separated, empty for none)")
    ap.add_argument("--execution", default="graph", choices=["graph", "eager"])
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only; --gpus {args.gpus} is not run")
        return 2

    import numpy as np
    import torch
    from runtime.config import preset
    from runtime.engine import ModelRunner, StepEntry, load_model, write_random_model
    from runtime.sampling import Sampler

    raw = preset(args.model)
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
    raw["max_position_embeddings"] = max(raw["max_position_embeddings"], args.context)
    folder = tempfile.mkdtemp(prefix="bench-model-")
    write_random_model(folder, raw, seed=0, dtype="bfloat16")
    model = load_model(folder, dtype=args.dtype)
    c = model.config
    itemsize = 2 if args.dtype == "bfloat16" else 4
    sampler = Sampler()
    rng = np.random.default_rng(0)
    batches = [args.batch] + [int(b) for b in args.points.split(",") if b]
    need_tokens = max(batches) * args.context
    runner = ModelRunner(model, n_pages=-(-need_tokens // args.page_size), page_size=args.page_size,
                         max_requests=max(batches), execution=args.execution)

    # bytes a decode step has to read: every weight it uses once, and the cache of the live requests
    L, H, D, nh, nkv, I, V = (c.num_hidden_layers, c.hidden_size, c.head_dim, c.num_attention_heads,
                              c.num_key_value_heads, c.intermediate_size, c.vocab_size)
    layer_params = H * (nh + 2 * nkv) * D + nh * D * H + 3 * H * I + 2 * H
    weight_bytes = (L * layer_params + V * H * (1 if c.tie_word_embeddings else 1) + H) * itemsize
    kv_bytes_per_token = L * 2 * nkv * D * itemsize

    def prefill_flops(T):
        gemm = 2 * T * L * (layer_params - 2 * H)
        attn = L * nh * 4 * D * T * (T + 1) / 2
        head = 2 * V * H  # one wanted row
        return gemm + attn + head

    def timed_prefill(key, tokens):
        runner.create(key)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = runner.step([StepEntry(key, tokens, [len(tokens) - 1])])
        first = sampler.pick(logits, [(0.0, 0, 0)])[0]
        torch.cuda.synchronize()
        return first, time.perf_counter() - t0

    def decode_run(batch, steps, warmup):
        keys = [f"b{batch}-{i}" for i in range(batch)]
        last, prefill_times = [], []
        for key in keys:
            tokens = rng.integers(0, V, size=args.prompt).tolist()
            first, dt = timed_prefill(key, tokens)
            last.append(first)
            prefill_times.append(dt)
        params = [(0.0, 0, 0)] * batch

        def one():
            nonlocal last
            logits = runner.step([StepEntry(k, [t], [0]) for k, t in zip(keys, last)])
            last = sampler.pick(logits, params)

        for _ in range(warmup):
            one()
        torch.cuda.synchronize()
        ctx0 = runner.length(keys[0])
        t0 = time.perf_counter()
        for _ in range(steps):
            one()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        ctx_mid = ctx0 + steps / 2
        for key in keys:
            runner.release(key)
        return elapsed, ctx_mid, prefill_times

    steps = min(args.steps, args.context - args.prompt - args.warmup - 1)
    results = {}
    for batch in batches:
        elapsed, ctx_mid, prefill_times = decode_run(batch, steps, args.warmup)
        results[batch] = (elapsed, ctx_mid, prefill_times)
    elapsed, ctx_mid, prefill_times = results[args.batch]
    ms_per_step = elapsed / steps * 1e3
    value = args.batch * steps / elapsed
    step_bytes = weight_bytes + args.batch * ctx_mid * kv_bytes_per_token
    achieved = step_bytes / (elapsed / steps) / 1e9
    # prefill: the best of the timed prompt steps after the first (the first pays one-time set-up)
    pf = min(prefill_times[1:]) if len(prefill_times) > 1 else prefill_times[0]
    peak = PEAK_TFLOPS["bf16" if args.dtype == "bfloat16" else "fp32"] * 1e12
    points = {f"decode_b{b}": round(b * steps / results[b][0], 1) for b in batches if b != args.batch}
    line = {
        "metric": f"decode tokens/s, {args.model} layer sizes, batch {args.batch}, {args.prompt}-token prompts in a {args.context} context",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": args.model, "global_batch": args.batch, "seq_len": args.context, "prompt_len": args.prompt,
                   "parallelism": "single-gpu", "layers": L, "layers_of_configuration": full_layers, "hidden": H,
                   "heads": nh, "kv_heads": nkv, "head_dim": D, "intermediate": I, "vocab": V,
                   "rope_theta": c.rope_theta, "rms_norm_eps": c.rms_norm_eps, "tied_head": c.tie_word_embeddings,
                   "page_size": args.page_size, "execution": args.execution},
        "prefill": {"value": round(args.prompt / pf, 1), "tokens": args.prompt, "ms": round(pf * 1e3, 3),
                    "frac": round(prefill_flops(args.prompt) / pf / peak, 5)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 5)},
        "points": points,
        "reference_b1_tokens_per_s": REFERENCE_B1_TOKS,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
