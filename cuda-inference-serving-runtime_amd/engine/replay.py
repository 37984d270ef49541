"""Trace replay: feeds given token ids through a model step by step and writes
logits.  It samples nothing and has no forward pass, cache or loader of its
own: it drives load_model, ModelRunner.step and the cache manager, the ones that
generation uses.

Input, one JSON object per line on standard input:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
A step may also say "fork": [["a", "b"]]: before its entries run, request b starts as a copy of what a holds
(pages shared, the partly filled last page copied at b's or a's next write; the reference's fork,
runtime/cache.py:64-76, exercised by tests/test_execution.py:55-64).
For a step in which something is wanted, ``<out>/<step>.f32`` receives the
logits at the wanted places as little-endian float32 [wanted, vocab], in the
order of the entries and of ``want``.  After every step ``done <step>`` is
printed and flushed.  (The reference's nearest relatives are its fixed step
schedules in tests/test_model.py:24-25 and tests/test_execution.py:25-30.)
"""
import argparse
import json
import sys
from pathlib import Path

import torch

from .loading import import_plugins, load_model
from .runner import ModelRunner, StepEntry

PAGE_SIZE = 16          # divides 64, so a request rounded up to 64 tokens never holds more than its share
MAX_LIVE = 4


def replay(model_dir, dtype, out_dir, max_tokens, lines, page_size=PAGE_SIZE, echo=print, execution="eager"):
    """`execution`: "eager" launches every step's kernels one by one; "graph" runs every step as a captured program
    (the way serving decodes), padded to its bucket of rows, segments and wanted rows."""
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    model = load_model(model_dir, dtype=dtype)
    pages = max(1, -(-int(max_tokens) // page_size))
    runner = ModelRunner(model, n_pages=pages, page_size=page_size, max_requests=4 * MAX_LIVE, execution=execution)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        for source, target in record.get("fork", []):
            runner.fork(source, target)
        entries = []
        for item in record.get("entries", []):
            if item["id"] not in runner.cache:
                runner.create(item["id"])
            entries.append(StepEntry(item["id"], item["tokens"], item.get("want", [])))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0]:
                data = logits.to(torch.float32).cpu().numpy().astype("<f4", copy=False)
                data.tofile(out_dir / f"{record['step']}.f32")
        for request in record.get("end", []):
            if request in runner.cache:
                runner.release(request)
        torch.cuda.synchronize()
        echo(f"done {record['step']}")
    return runner


def main(argv=None):
    parser = argparse.ArgumentParser(prog="trace_run", description="Replay a token trace and write logits.")
    parser.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    parser.add_argument("--dtype", choices=["bfloat16", "float32"], required=True)
    parser.add_argument("--out", required=True, help="folder for <step>.f32 files")
    parser.add_argument("--max-tokens", type=int, required=True,
                        help="most tokens live requests hold at any time (each rounded up to 64)")
    parser.add_argument("--page-size", type=int, default=PAGE_SIZE, help="tokens a cache page (a power of two that divides 64)")
    parser.add_argument("--execution", choices=["eager", "graph"], default="eager",
                        help="eager: kernels launched one by one; graph: every step as a captured program")
    parser.add_argument("--plugin", action="append", default=[], metavar="MODULE",
                        help="import this module first: it may register parts or an architecture of its own (may be given more than once)")
    args = parser.parse_args(argv)
    import_plugins(args.plugin)

    def echo(text):
        print(text, flush=True)

    if args.page_size <= 0 or 64 % args.page_size:
        parser.error("--page-size must divide 64")
    replay(args.model, args.dtype, args.out, args.max_tokens, sys.stdin, page_size=args.page_size, echo=echo, execution=args.execution)
    return 0
