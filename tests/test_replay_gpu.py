"""Trace replay against the plain implementation, in float32 and bfloat16: each
request whole; most of it in one step and the last 32 tokens one by one; in
portions of changing size down to two tokens; mixed, up to four live requests
with so few pages that they are used again; long decoding; the first tokens."""
import os
import subprocess
import sys


import numpy as np
import pytest

from conftest import ROOT, TINY, random_tokens
from trace_tools import Trace

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
EXECUTIONS = ["eager", "graph"]     # kernels launched one by one; every step as a captured program


def run(folder, dtype, trace, out_dir, max_tokens=None, page_size=None, execution="eager"):
    from runtime.engine.replay import replay, PAGE_SIZE
    done = []
    runner = replay(folder, dtype, out_dir, max_tokens or trace.peak, trace.lines(), page_size=page_size or PAGE_SIZE,
                    echo=done.append, execution=execution)
    assert done == [f"done {i}" for i in range(len(trace.steps))]
    runner.cache.check()
    return runner


@pytest.mark.parametrize("execution", EXECUTIONS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_whole_requests_alone(folders, tmp_path, name, dtype, execution):
    V = TINY[name]["vocab_size"]
    seqs = {f"r{i}": random_tokens(10 * i + 1, n, V) for i, n in enumerate([1, 5, 64, 65, 150])}
    trace = Trace()
    for rid, toks in seqs.items():
        trace.add([(rid, toks, list(range(len(toks))))], end=[rid])
    runner = run(folders[name], dtype, trace, tmp_path, execution=execution)
    trace.check(folders[name], tmp_path, dtype, V, seqs)
    assert all(free == g.pool.n_pages for free, g in zip(runner.cache.free_pages(), runner.cache.groups))


@pytest.mark.parametrize("execution", EXECUTIONS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_prefix_then_last_32_one_by_one(folders, tmp_path, name, dtype, execution):
    V = TINY[name]["vocab_size"]
    toks = random_tokens(77, 131, V)
    trace = Trace()
    trace.add([("p", toks[:-32], list(range(len(toks) - 32)))])
    for t in toks[-32:]:
        trace.add([("p", [t], [0])])
    run(folders[name], dtype, trace, tmp_path, execution=execution)
    trace.check(folders[name], tmp_path, dtype, V, {"p": toks})


@pytest.mark.parametrize("execution", EXECUTIONS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_portions_of_changing_size(folders, tmp_path, name, dtype, execution):
    V = TINY[name]["vocab_size"]
    toks = random_tokens(5, 140, V)
    trace, at = Trace(), 0
    sizes = [7, 2, 13, 3, 2, 16, 17, 2, 31, 5, 2, 33, 2]   # crosses page edges at every offset
    for i, n in enumerate(sizes):
        n = min(n, len(toks) - at)
        if n <= 0:
            break
        want = list(range(n)) if i % 3 else [0, n - 1]     # sometimes every place, sometimes the ends
        trace.add([("q", toks[at:at + n], want)])
        at += n
    trace.add([("q", toks[at:], list(range(len(toks) - at)))], end=["q"])
    run(folders[name], dtype, trace, tmp_path, execution=execution)
    trace.check(folders[name], tmp_path, dtype, V, {"q": toks})


def mixed_trace(V, seed):
    """Up to four live requests: portions of some beside single decoded tokens of
    others; requests end and new ones start on the pages they gave back; one
    request sits out some steps."""
    rng = np.random.default_rng(seed)
    lengths = [70, 33, 120, 9, 64, 97, 40, 130]
    seqs = {f"m{i}": random_tokens(seed * 100 + i, n, V) for i, n in enumerate(lengths)}
    waiting = list(seqs)
    live, fed = [], {}
    trace = Trace()
    step = 0
    while waiting or live:
        while waiting and len(live) < 4:
            rid = waiting.pop(0); live.append(rid); fed[rid] = 0
        entries, ending = [], []
        for rid in list(live):
            remaining = len(seqs[rid]) - fed[rid]
            if rid == live[0] and step % 5 == 3 and len(live) > 1:
                continue                                  # left out of this step, goes on later
            if remaining > 12:                            # still in its prompt: a portion of changing size
                n = int(rng.choice([2, 3, 7, 16, 21, 40]))
                n = min(n, remaining - 8)
                if n < 2:
                    n = remaining - 8 if remaining - 8 >= 1 else 1
                want = [n - 1] if rng.random() < 0.5 else list(range(n))
            else:                                         # decoding: one token
                n, want = 1, [0]
            entries.append((rid, seqs[rid][fed[rid]:fed[rid] + n], want))
            fed[rid] += n
            if fed[rid] == len(seqs[rid]):
                ending.append(rid); live.remove(rid)
        if entries:
            trace.add(entries, end=ending)
        step += 1
    return trace, seqs


@pytest.mark.parametrize("execution", EXECUTIONS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_mixed_requests_reuse_pages(folders, tmp_path, name, dtype, execution):
    V = TINY[name]["vocab_size"]
    trace, seqs = mixed_trace(V, seed=3)
    assert any(len(s["entries"]) == 4 for s in trace.steps)
    assert any(len(e["tokens"]) > 1 for s in trace.steps for e in s["entries"] if len(s["entries"]) > 1)
    runner = run(folders[name], dtype, trace, tmp_path, execution=execution)   # pool = exactly the peak of rounded-up tokens
    pool = runner.cache.groups[0].pool
    assert pool.n_pages * 16 == trace.peak
    assert sum(-(-len(s) // 16) for s in seqs.values()) > pool.n_pages, "the trace must need more pages than exist"
    assert pool.peak > pool.n_pages // 2
    trace.check(folders[name], tmp_path, dtype, V, seqs)


@pytest.mark.parametrize("execution", EXECUTIONS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name, page_size", [("a", 16), ("b", 8), ("c", 16)])
def test_fork_in_the_middle_of_a_page_then_both_go_on(folders, tmp_path, name, page_size, dtype, execution):
    """A request is forked where its last page is partly filled (37 tokens); source and copy go on with different
    tokens, in portions and token by token, beside a third request, in a pool so small that the pages the first
    fork gave back are taken again; then the copy is forked once more, right after a decoded token.  Whoever
    writes into the shared page first gets a copy of it; the other must still read what was there."""
    V = TINY[name]["vocab_size"]
    stem = random_tokens(21, 37, V)
    seqs = {"a": stem + random_tokens(22, 60, V), "b": stem + random_tokens(23, 45, V), "c": random_tokens(24, 50, V)}
    seqs["d"] = seqs["b"][:37 + 20] + random_tokens(25, 30, V)
    trace = Trace()
    trace.add([("a", stem, [36])])
    # the copy writes first (a portion that crosses the page's edge), the source sits this step out
    trace.add([("b", seqs["b"][37:37 + 13], list(range(13))), ("c", seqs["c"][:9], [8])], fork=[("a", "b")])
    trace.add([("a", seqs["a"][37:39], [0, 1]), ("b", seqs["b"][50:51], [0]), ("c", seqs["c"][9:30], [20])])
    at = {"a": 39, "b": 51, "c": 30}
    for _ in range(6):
        trace.add([(k, seqs[k][at[k]:at[k] + 1], [0]) for k in "abc"])
        for k in at:
            at[k] += 1
    assert at["b"] == 57
    # a second fork, from the copy, right after a decoded token; its source ends in the same step
    trace.add([("d", seqs["d"][57:57 + 11], list(range(11))), ("a", seqs["a"][at["a"]:at["a"] + 17], [16])], fork=[("b", "d")])
    at["a"] += 17
    trace.add([("b", seqs["b"][57:], list(range(len(seqs["b"]) - 57))), ("d", seqs["d"][68:70], [1])], end=["b"])
    trace.add([("a", seqs["a"][at["a"]:], [len(seqs["a"]) - at["a"] - 1]), ("c", seqs["c"][at["c"]:], [len(seqs["c"]) - at["c"] - 1]),
               ("d", seqs["d"][70:], list(range(len(seqs["d"]) - 70)))], end=["a", "c", "d"])
    assert all(trace.fed[k] == seqs[k] for k in seqs)
    runner = run(folders[name], dtype, trace, tmp_path, page_size=page_size, execution=execution)
    pool = runner.cache.groups[0].pool
    assert pool.peak < sum(-(-len(s) // page_size) for s in seqs.values()), "the forks shared no page"
    assert all(free == g.pool.n_pages for free, g in zip(runner.cache.free_pages(), runner.cache.groups))
    trace.check(folders[name], tmp_path, dtype, V, seqs)


@pytest.mark.parametrize("execution", EXECUTIONS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_tiny_b_with_pages_of_eight_tokens(folders, tmp_path, dtype, execution):
    """The second tiny configuration as it is specified: pages of 8 tokens.  Prompts of 1, 9, 33 and 64 tokens cut
    into portions of 7 beside decoded tokens of the others, then 12 more tokens each."""
    name = "b"
    V = TINY[name]["vocab_size"]
    seqs = {f"r{i}": random_tokens(40 + i, n + 12, V) for i, n in enumerate([1, 9, 33, 64])}
    prompt = {k: len(v) - 12 for k, v in seqs.items()}
    trace, at = Trace(), {k: 0 for k in seqs}
    while any(at[k] < len(seqs[k]) for k in seqs):
        entries, ending = [], []
        for k in seqs:
            if at[k] >= len(seqs[k]):
                continue
            n = min(7, prompt[k] - at[k]) if at[k] < prompt[k] else 1
            entries.append((k, seqs[k][at[k]:at[k] + n], [n - 1]))
            at[k] += n
            if at[k] == len(seqs[k]):
                ending.append(k)
        trace.add(entries, end=ending)
    run(folders[name], dtype, trace, tmp_path, page_size=8, execution=execution)
    trace.check(folders[name], tmp_path, dtype, V, seqs)


@pytest.mark.parametrize("execution", EXECUTIONS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_and_first_tokens(folders, tmp_path, dtype, execution):
    name = "a"
    V = TINY[name]["vocab_size"]
    toks = random_tokens(9, 300, V)
    trace = Trace()
    for t in toks:                       # position 0 alone, then 299 single-token steps
        trace.add([("d", [t], [0])])
    run(folders[name], dtype, trace, tmp_path, execution=execution)
    got = trace.check(folders[name], tmp_path, dtype, V, {"d": toks})
    assert [p for p, _ in got["d"]][:3] == [0, 1, 2]


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_do_not_depend_on_the_cut_or_the_company(folders, tmp_path, dtype):
    """The same request whole, cut, and beside other requests: float32 agrees to
    rounding between the runs themselves, not only with the plain implementation."""
    name = "c"
    V = TINY[name]["vocab_size"]
    a, b = random_tokens(1, 90, V), random_tokens(2, 50, V)
    whole = Trace(); whole.add([("a", a, list(range(90)))])
    cut = Trace()
    cut.add([("b", b[:20], []), ("a", a[:37], list(range(37)))])
    cut.add([("a", a[37:39], [0, 1]), ("b", b[20:], [])], end=["b"])
    for t in range(39, 90):
        cut.add([("a", [a[t]], [0])])
    run(folders[name], dtype, whole, tmp_path / "whole")
    run(folders[name], dtype, cut, tmp_path / "cut", page_size=8)
    x = np.fromfile(tmp_path / "whole" / "0.f32", "<f4").reshape(90, V)
    y = np.concatenate([np.fromfile(tmp_path / "cut" / f"{s}.f32", "<f4").reshape(-1, V) for s in sorted(cut.expect)])
    if dtype == "float32":
        assert np.abs(x - y).max() / np.abs(x).max() < 2e-5
    else:   # the two runs round at different places (other kernels for portions and single tokens);
        # the bound is the one that holds against the plain implementation
        from conftest import BF16_RMSE
        assert np.linalg.norm(x - y) / np.linalg.norm(x) < BF16_RMSE


def test_out_of_pages_and_bad_input_fail_loudly(folders, tmp_path):
    from runtime.cache import OutOfPages
    V = TINY["a"]["vocab_size"]
    trace = Trace(); trace.add([("x", random_tokens(1, 70, V), [69])])
    with pytest.raises(OutOfPages):
        run(folders["a"], "float32", trace, tmp_path, max_tokens=64)
    bad = Trace(); bad.add([("x", [V], [0])])
    with pytest.raises(ValueError, match="vocabulary"):
        run(folders["a"], "float32", bad, tmp_path)
    over = Trace(); over.add([("x", [1] * (TINY["a"]["max_position_embeddings"] + 1), [0])])
    with pytest.raises(ValueError, match="context limit"):
        run(folders["a"], "float32", over, tmp_path, max_tokens=1024)


@pytest.mark.parametrize("dtype,execution", [("float32", None), ("bfloat16", None), ("bfloat16", "graph")])
def test_trace_run_program(folders, tmp_path, dtype, execution):
    """The program itself, as a user runs it: reads steps from its input, writes
    <step>.f32 and prints `done <step>` after every step."""
    name = "b"
    V = TINY[name]["vocab_size"]
    toks, other = random_tokens(4, 80, V), random_tokens(6, 30, V)
    trace = Trace()
    trace.add([("u", toks[:50], [49]), ("v", other[:10], [])])
    trace.add([("u", toks[50:52], [0, 1]), ("v", other[10:], [19])], end=["v"])
    for t in toks[52:]:
        trace.add([("u", [t], [0])])
    out = tmp_path / "out"
    env = dict(os.environ, PYTHONPATH="")
    proc = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(folders[name]), "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(trace.peak)] + (["--execution", execution] if execution else []),
                          input="\n".join(trace.lines()) + "\n",
                          capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:len(trace.steps)] == [f"done {i}" for i in range(len(trace.steps))]
    trace.check(folders[name], out, dtype, V, {"u": toks, "v": other})
