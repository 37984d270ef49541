"""Run token-id workloads or a local Llama checkpoint on the MI355X.

Options keep the names and meanings of the reference's command line
(runtime/__main__.py:13-26); `--device cpu` does not exist here (there is no CPU
path), `--dtype float16` is not built, `--execution buffered` is what `eager`
already is (stable buffers, explicit kernels), and `--execution` defaults to
`graph` (the reference's default, eager, is the slow path in both).  Added: `--model` (a named
configuration with seeded random weights when no checkpoint is given),
`--seed`, `--temperature`, `--max-active`.
"""
import argparse
import json
import sys
import tempfile
from pathlib import Path


def main(argv=None):
    parser = argparse.ArgumentParser(prog="python -m runtime", description=__doc__)
    parser.add_argument("--device", choices=["hip", "cuda"], default="hip", help="the MI355X (both names mean it)")
    parser.add_argument("--dtype", choices=["float32", "bfloat16"], default="bfloat16")
    parser.add_argument("--execution", choices=["eager", "buffered", "graph"], default="graph",
                        help="graph: every step as a captured program (the default here: it is the fast path); "
                             "eager or buffered: kernels launched one by one")
    parser.add_argument("--checkpoint", type=Path, help="folder with config.json and *.safetensors")
    parser.add_argument("--model", default="tiny-a", help="named configuration for random weights (no --checkpoint)")
    parser.add_argument("--seed", type=int, default=0, help="seed of random weights and of sampling")
    parser.add_argument("--prompt", default="The capital of France is")
    parser.add_argument("--tokens", default="1,2,3", help="prompt as token IDs")
    parser.add_argument("--max-new-tokens", type=int, default=16)
    parser.add_argument("--temperature", type=float, default=0.0, help="0 = greedy")
    parser.add_argument("--requests", type=Path, help="JSON list: key,prompt (IDs),max_new_tokens,arrival_s")
    parser.add_argument("--policy", choices=["serial", "chunked", "decode_first"], default="decode_first")
    parser.add_argument("--pages", type=int, default=128, help="cache pages; 0: as many as fit into the free GPU memory")
    parser.add_argument("--page-size", type=int, default=16)
    parser.add_argument("--token-budget", type=int, default=32)
    parser.add_argument("--prefill-chunk", type=int, default=8)
    parser.add_argument("--max-active", type=int, default=8)
    parser.add_argument("--overlap", action="store_true",
                        help="launch each step before the tokens of the step before are read (same tokens, less idle GPU)")
    parser.add_argument("--plugin", action="append", default=[], metavar="MODULE",
                        help="import this module first: it may register parts or an architecture of its own (may be given more than once)")
    parser.add_argument("--report", action="store_true",
                        help="add the step function's counters and memory (steps, programs captured and replayed, "
                             "bytes of workspace, scratch, staging and cache) to the output")
    args = parser.parse_args(argv)

    from .config import read_config_json
    from .engine.loading import import_plugins
    from .engine.scheduler import Engine, Request
    import_plugins(args.plugin)

    tokenizer, raw = None, {}
    execution = "graph" if args.execution == "graph" else "eager"
    common = dict(dtype=args.dtype, pages=args.pages, page_size=args.page_size, execution=execution,
                  policy=args.policy, token_budget=args.token_budget, prefill_chunk=args.prefill_chunk,
                  max_active=args.max_active, overlap=args.overlap)
    if args.checkpoint:
        raw = read_config_json(args.checkpoint)
        engine = Engine.from_folder(args.checkpoint, **common)
        tokenizer_file = args.checkpoint / "tokenizer.json"
        if tokenizer_file.exists():
            from tokenizers import Tokenizer
            tokenizer = Tokenizer.from_file(str(tokenizer_file))
            prompt = tokenizer.encode(args.prompt).ids
        else:
            prompt = [int(t) for t in args.tokens.split(",")]
    else:
        folder = tempfile.mkdtemp(prefix="runtime-random-")
        engine = Engine.from_preset(args.model, seed=args.seed, folder=folder, **common)
        raw = read_config_json(folder)
        prompt = [int(t) for t in args.tokens.split(",")]
    if args.requests:
        workload = json.loads(args.requests.read_text())
    else:
        workload = [dict(key="request-0", prompt=prompt, max_new_tokens=args.max_new_tokens)]
    for index, item in enumerate(workload):
        # what the file says wins over the defaults: the checkpoint's end-of-sequence id, the command line's sampling
        engine.submit(Request(**{"eos_token_id": raw.get("eos_token_id"), "temperature": args.temperature,
                                 "seed": args.seed + index, **item}))

    def outcome(r):
        waited = None if r.first_token_at is None else 1e3 * (r.first_token_at - r.submitted_at)
        return dict(key=r.key, status=r.status, generated=r.generated,
                    text=None if tokenizer is None else tokenizer.decode(r.generated), ttft_ms=waited)

    # the reference's report (runtime/__main__.py:43-50): one object, the requests in the order they were submitted
    report = dict(device="hip", dtype=args.dtype, execution=execution,
                  weights=f"random-{args.model}" if not args.checkpoint else "pretrained-local",
                  requests=[outcome(r) for r in engine.run()])
    if args.report:
        report["runner"] = engine.runner.report()
    print(json.dumps(report, indent=2))
    return 0


if __name__ == "__main__":
    sys.exit(main())
