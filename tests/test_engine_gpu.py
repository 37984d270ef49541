"""Generation through the entry points: greedy tokens equal the plain
implementation's, every policy and execution mode gives the same tokens,
sampling does not depend on the batch, the command line works."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama as P
from conftest import ROOT, TINY, assert_close, plain_logits, random_tokens

pytestmark = pytest.mark.gpu


def plain_greedy_margin(cfg, w, prompt, steps):
    """Greedy tokens, the gap between the two best logits at every step and those two tokens."""
    tokens, out, gaps, top2 = list(prompt), [], [], []
    for _ in range(steps):
        logits = P.forward(cfg, w, tokens)[-1]
        order = np.argsort(logits)[-2:]
        gaps.append(float(logits[order[1]] - logits[order[0]]))
        top2.append({int(order[0]), int(order[1])})
        out.append(int(np.argmax(logits)))
        tokens.append(out[-1])
    return out, gaps, top2


@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation_matches_plain(folders, name, dtype, execution):
    from runtime.engine.scheduler import Engine
    cfg, w = P.read_folder(folders[name])
    V = TINY[name]["vocab_size"]
    prompts = [random_tokens(20 + i, n, V) for i, n in enumerate([5, 11, 17])]
    want = [plain_greedy_margin(cfg, w, p, 8) for p in prompts]
    engine = Engine.from_folder(folders[name], dtype=dtype, pages=32, page_size=16, token_budget=16, prefill_chunk=7,
                                execution=execution)
    got = engine.generate(prompts, max_new_tokens=8)
    for g, (tokens, gaps, top2) in zip(got, want):
        if dtype == "float32" or min(gaps) > 0.05:
            assert g == tokens
        else:   # a near tie may flip in bfloat16: equal up to the first place whose two best logits are that close
            first_tie = next(i for i, gap in enumerate(gaps) if gap < 0.05)
            assert g[:first_tie] == tokens[:first_tie]
            assert g[first_tie] in top2[first_tie], "a flipped near tie picks the runner-up, nothing else"
    engine.runner.cache.check()
    assert engine.runner.cache.free_pages() == [32]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_policies_and_execution_modes_agree(folders, dtype):
    # reference tests/test_engine.py:12-21 and tests/test_execution.py:42-53
    from runtime.engine.scheduler import Engine, Request
    V = TINY["c"]["vocab_size"]
    prompts = [random_tokens(40 + i, n, V) for i, n in enumerate([1, 7, 3, 40])]
    outputs = []
    for policy, execution, budget, chunk, overlap in [
            ("serial", "eager", 3, 2, False), ("chunked", "eager", 3, 2, False), ("decode_first", "eager", 3, 2, False),
            ("decode_first", "graph", 64, 64, False), ("chunked", "graph", 5, 3, False),
            ("chunked", "eager", 3, 2, True), ("decode_first", "graph", 64, 64, True), ("chunked", "graph", 5, 3, True)]:
        e = Engine.from_folder(folders["c"], dtype=dtype, pages=20, page_size=4, execution=execution, policy=policy,
                               token_budget=budget, prefill_chunk=chunk, overlap=overlap)
        for i, p in enumerate(prompts):
            e.submit(Request(str(i), p, 12))
        result = e.run()
        assert all(r.status == "finished" and len(r.generated) == 12 for r in result)
        assert all(t["processed_tokens"] <= budget for t in e.trace)
        e.runner.cache.check()
        assert e.runner.cache.free_pages() == [20] and not e.reserved
        outputs.append([r.generated for r in result])
        if execution == "graph":
            assert any(p["graph"] is not None for p in e.runner.programs.values()), "no decode step was captured"
    assert all(o == outputs[0] for o in outputs[1:])


def test_graph_replays_match_eager_logits(folders):
    """Captured decode programs replayed many times, with eager steps, changing
    batch sizes and request order in between: every replay equals the eager run."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    V = TINY["c"]["vocab_size"]
    model = load_model(folders["c"], dtype="bfloat16")
    runners = [ModelRunner(model, n_pages=40, page_size=8, execution=mode) for mode in ("eager", "graph")]
    seqs = {k: random_tokens(60 + i, 80, V) for i, k in enumerate("abc")}
    fed = {k: 0 for k in seqs}
    schedule = [("a", "b"), ("a",), ("a", "b", "c"), ("c", "a"), ("b",)] * 6   # reference tests/test_execution.py:25-30
    for r in runners:
        for k in seqs:
            r.create(k)
            r.step([StepEntry(k, seqs[k][:5], [])])
    for k in seqs:
        fed[k] = 5
    for keys in schedule:
        entries = [StepEntry(k, [seqs[k][fed[k]]], [0]) for k in keys]
        a, b = (r.step(entries).clone() for r in runners)
        torch.cuda.synchronize()
        assert torch.equal(a, b), f"replay differs from eager at {keys}"
        for k in keys:
            fed[k] += 1
    graph_runner = runners[1]
    decode_programs = [p for key, p in graph_runner.programs.items() if key[3] and p["graph"] is not None]
    assert len(decode_programs) >= 2 and all(p["runs"] >= 3 for p in decode_programs)


@pytest.mark.parametrize("name,dtype", [("c", "bfloat16"), ("a", "float32")])
def test_evicted_programs_are_built_again_and_stay_right(folders, name, dtype):
    """More step shapes than the runner keeps captured programs for: the oldest are dropped (their buffers go
    back) and, when their shape comes again, built, captured and replayed anew.  Every step, before and after, is
    compared with the plain model."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from conftest import plain_logits, assert_close
    V = TINY[name]["vocab_size"]
    model = load_model(folders[name], dtype=dtype)
    runner = ModelRunner(model, n_pages=80, page_size=8, max_requests=4, execution="graph", program_capacity=16)
    seqs = {k: random_tokens(700 + i, 200, V) for i, k in enumerate("uvw")}
    refs = {k: plain_logits(folders[name], seqs[k]) for k in seqs}
    fed = {}

    def restart():
        for k in seqs:
            if k in runner.cache:
                runner.release(k)
            runner.create(k)
            fed[k] = 0

    def feed(parts, wanted=True):
        entries, places = [], []
        for k, n in parts:
            want = ([0, n - 1] if n > 1 else [0]) if wanted else []
            entries.append(StepEntry(k, seqs[k][fed[k]:fed[k] + n], want))
            places += [(k, fed[k] + j) for j in want]
            fed[k] += n
        logits = runner.step(entries).float().cpu().numpy()
        assert logits.shape[0] == len(places)
        for row, (k, pos) in zip(logits, places):
            assert_close(row[None], refs[k][pos][None], dtype, f"request {k} position {pos}")

    first = [("u", 5), ("v", 1)]
    restart()
    feed([("u", 3)]); feed([("v", 2)])
    for _ in range(3):                      # built, captured, replayed
        feed(first)
    first_key = next(reversed(runner.programs))
    assert runner.programs[first_key]["graph"] is not None
    shapes = [[("u", n)] for n in (1, 2, 3, 5, 9, 17, 33)] + [[("u", n), ("v", m)] for n, m in ((1, 1), (2, 3), (9, 9), (17, 20))] \
        + [[("u", 1), ("v", 1), ("w", 1)], [("u", 2), ("v", 1), ("w", 7)], [("u", 30), ("v", 1), ("w", 40)]]
    seen = set()
    for wanted in (True, False):
        restart()
        for parts in shapes:
            for _ in range(2):              # the second run of a shape captures it
                if max(fed[k] + n for k, n in parts) > 190:
                    restart()
                feed(parts, wanted)
                seen.add(next(reversed(runner.programs)))
            assert len(runner.programs) <= runner.program_capacity
    assert len(seen) > runner.program_capacity, "not enough different shapes to push a program out"
    report = runner.report()
    assert report["evictions"] >= len(seen) - 16        # what the step function says of itself: every drop counted
    assert report["captures"] >= len(seen) and report["replays"] > 0 and report["programs"] <= 16
    assert first_key not in runner.programs, "the first program was never dropped"
    restart()
    feed([("u", 3)]); feed([("v", 2)])
    for _ in range(3):                      # the dropped shape again: built, captured and replayed anew
        feed(first)
    again = runner.programs[first_key]
    assert again["graph"] is not None and again["runs"] == 3
    runner.cache.check()


@pytest.mark.parametrize("name,dtype", [("d", "float32"), ("d", "bfloat16"), ("a", "bfloat16"), ("c", "bfloat16")])
def test_captured_prompt_and_mixed_steps_match_the_plain_model(folders, name, dtype):
    """In graph mode every step shape becomes a captured program: portions of prompts, alone and
    beside decoded tokens, padded to the program's sizes.  The same shapes come again and again
    with other requests, positions and pages; every replay is compared with the plain model."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from conftest import plain_logits, assert_close
    V = TINY[name]["vocab_size"]
    model = load_model(folders[name], dtype=dtype)
    runner = ModelRunner(model, n_pages=24, page_size=8, max_requests=4, execution="graph")
    for round_ in range(5):
        seqs = {k: random_tokens(300 + 10 * round_ + i, 45, V) for i, k in enumerate("xyz")}
        refs = {k: plain_logits(folders[name], seqs[k]) for k in seqs}
        for k in seqs:
            runner.create(k)
        fed = {k: 0 for k in seqs}

        def feed(*parts):
            entries, places = [], []
            for k, n in parts:
                entries.append(StepEntry(k, seqs[k][fed[k]:fed[k] + n], [0, n - 1] if n > 1 else [0]))
                places += [(k, fed[k]), (k, fed[k] + n - 1)] if n > 1 else [(k, fed[k])]
                fed[k] += n
            logits = runner.step(entries).float().cpu().numpy()
            assert logits.shape[0] == len(places)
            for row, (k, pos) in zip(logits, places):
                assert_close(row[None], refs[k][pos][None], dtype, f"round {round_} request {k} position {pos}")

        feed(("x", 19))                        # a portion alone
        feed(("y", 19))                        # the same shape, another request
        feed(("x", 1), ("y", 1), ("z", 11))    # decoded tokens beside a portion
        feed(("x", 1), ("y", 1), ("z", 11))
        feed(("z", 19))
        feed(("x", 1), ("y", 1), ("z", 1))
        feed(("x", 1), ("y", 1), ("z", 1))
        for k in seqs:
            runner.release(k)
    captured = [p for p in runner.programs.values() if p["graph"] is not None]
    assert len(captured) >= 3 and all(p["runs"] >= 3 for p in captured)
    assert any(not key[3] for key, p in runner.programs.items() if p["graph"] is not None), "no prompt step was captured"
    runner.cache.check()


@pytest.mark.parametrize("name,dtype", [("a", "bfloat16"), ("b", "bfloat16"), ("c", "bfloat16")])
@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("launch", [None, (4, 3)])
def test_decoded_tokens_of_mixed_steps_in_a_launch_of_their_own(folders, name, dtype, execution, launch):
    """From a certain context on, the one-token segments of a mixed step leave the tile list and are attended
    to by the decode kernel over a list of rows, their keys split over blocks; forced here from the first
    token, with the natural launch shape and with three splits (some of them empty at these lengths).  Under
    graphs the list is padded to the program's size with rows of no request."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.kernels import ops
    from conftest import plain_logits, assert_close
    V = TINY[name]["vocab_size"]
    model = load_model(folders[name], dtype=dtype)
    from conftest import tune_attention
    tune_attention(model, split_single_from=1, rows_launch=launch)
    runner = ModelRunner(model, n_pages=32, page_size=8, max_requests=4, execution=execution)
    seen = []
    attend = ops.attention_mfma
    def spy(*a, **kw):
        seen.append(kw.get("row_ids"))
        return attend(*a, **kw)
    ops_attention, ops.attention_mfma = ops.attention_mfma, spy
    try:
        for round_ in range(3):
            seqs = {k: random_tokens(700 + 10 * round_ + i, 50, V) for i, k in enumerate("wxyz")}
            refs = {k: plain_logits(folders[name], seqs[k]) for k in seqs}
            for k in seqs:
                runner.create(k)
            fed = {k: 0 for k in seqs}

            def feed(*parts):
                entries, places = [], []
                for k, n in parts:
                    entries.append(StepEntry(k, seqs[k][fed[k]:fed[k] + n], [0, n - 1] if n > 1 else [0]))
                    places += [(k, fed[k]), (k, fed[k] + n - 1)] if n > 1 else [(k, fed[k])]
                    fed[k] += n
                logits = runner.step(entries).float().cpu().numpy()
                for row, (k, pos) in zip(logits, places):
                    assert_close(row[None], refs[k][pos][None], dtype, f"round {round_} request {k} position {pos}")

            feed(("w", 21), ("x", 9))
            feed(("w", 1), ("y", 13))                          # one decoded token beside a portion
            feed(("y", 1), ("z", 17), ("w", 1), ("x", 1))      # three, the portion between them
            feed(("w", 1), ("x", 7), ("y", 1))
            feed(("x", 1), ("y", 1), ("z", 2), ("w", 1))       # a portion of two tokens
            feed(("w", 1), ("x", 1), ("y", 1), ("z", 1))       # decode only: the ordinary launch
            feed(("z", 1), ("x", 5))
            for k in seqs:
                runner.release(k)
    finally:
        ops.attention_mfma = ops_attention
    assert sum(r is not None for r in seen) >= (30 if execution == "eager" else 1), "the decoded tokens of mixed steps had no launch of their own"
    runner.cache.check()


@pytest.mark.parametrize("name", ["a", "b"])
@pytest.mark.parametrize("execution", ["eager", "graph"])
def test_steps_through_the_wide_product_match_the_plain_model(folders, name, execution, monkeypatch, no_gemv):
    """With large weights the products of steps of up to 64 rows run the kernel that keeps the activations in
    registers, with norm, rotary embedding and cache write as kernels of their own; forced here on the tiny
    models: decode steps, short portions, mixed steps, again and again (its workspace is shared by the steps)."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.kernels import ops
    from conftest import plain_logits, assert_close
    for limit in ("WIDE_MIN_BYTES", "WIDE_MIN_BYTES_FEW_ROWS", "WIDE_MIN_BYTES_MANY_ROWS"):
        monkeypatch.setattr(ops, limit, 0)
    V = TINY[name]["vocab_size"]
    model = load_model(folders[name], dtype="bfloat16")
    runner = ModelRunner(model, n_pages=24, page_size=8, max_requests=4, execution=execution)
    calls = []
    wide = ops._gemm_wide
    monkeypatch.setattr(ops, "_gemm_wide", lambda *a: (calls.append(a[5]), wide(*a))[1])   # a[5]: which entry point asked
    seqs = {k: random_tokens(500 + i, 60, V) for i, k in enumerate("xyz")}
    refs = {k: plain_logits(folders[name], seqs[k]) for k in seqs}
    for k in seqs:
        runner.create(k)
    fed = {k: 0 for k in seqs}

    def feed(*parts):
        entries, places = [], []
        for k, n in parts:
            entries.append(StepEntry(k, seqs[k][fed[k]:fed[k] + n], [0, n - 1] if n > 1 else [0]))
            places += [(k, fed[k]), (k, fed[k] + n - 1)] if n > 1 else [(k, fed[k])]
            fed[k] += n
        logits = runner.step(entries).float().cpu().numpy()
        for row, (k, pos) in zip(logits, places):
            assert_close(row[None], refs[k][pos][None], "bfloat16", f"request {k} position {pos}")

    feed(("x", 33))                              # three row tiles
    feed(("y", 17), ("z", 2))                    # two
    for _ in range(3):
        feed(("x", 1), ("y", 1), ("z", 1))       # decode steps
    feed(("x", 1), ("y", 9), ("z", 30))
    for _ in range(3):
        feed(("x", 1), ("y", 1), ("z", 1))
    assert {"gemm", "gemm_swiglu"} <= set(calls)
    runner.cache.check()


REAL_SIZES = {
    # two layers of the SmolLM2-1.7B sizes
    "1.7b": dict(num_hidden_layers=2, hidden_size=2048, num_attention_heads=32, num_key_value_heads=32, head_dim=64,
                 intermediate_size=8192, vocab_size=49152, rope_theta=130000.0, rms_norm_eps=1e-5,
                 tie_word_embeddings=True, max_position_embeddings=512),
    # one layer with Llama-3-8B's attention (grouped heads of 128) and width, a narrower feed-forward and vocabulary
    "8b": dict(num_hidden_layers=1, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=6144, vocab_size=16000, rope_theta=500000.0, rms_norm_eps=1e-5,
               tie_word_embeddings=False, max_position_embeddings=512),
}


@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("sizes", ["1.7b", "8b"])
def test_layers_of_real_sizes_match_the_plain_model(tmp_path_factory, sizes, execution, monkeypatch, no_gemv):
    """Layers of real sizes: the sizes at which products choose other kernels by themselves (the wide
    weight-streaming product for decode steps, with the fused projection finishing in it; the vendor's library
    for portions of more than 64 rows).  Whole prompts, portions, decode steps of several requests and mixed
    steps against the plain model.  Products that end a part are left to the norm that follows: the slices of
    the wide product with few rows, the library's result with many."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from runtime.kernels import ops
    from conftest import write_folder, plain_logits, assert_close
    left = []
    unfinished = ops.gemm_unfinished
    monkeypatch.setattr(ops, "gemm_unfinished", lambda *a, **kw: (left.append(unfinished(*a, **kw)), left[-1])[1])
    cfg = REAL_SIZES[sizes]
    folder = write_folder(tmp_path_factory.mktemp("real") / "m", cfg, 77, sharp=False)
    model = load_model(folder, dtype="bfloat16")
    w_gate_up = model.layers[0].ffn.w_gate_up
    assert ops.wide_ok(5, w_gate_up, True, after_norm=True) and ops.library_ok(90, w_gate_up)   # what this test is for
    runner = ModelRunner(model, n_pages=40, page_size=16, max_requests=8, execution=execution)
    for round_ in range(3):    # the same step shapes again with other requests: in graph mode eager, captured, replayed
        seqs = {k: random_tokens(900 + 10 * round_ + i, 100, cfg["vocab_size"]) for i, k in enumerate("abcde")}
        refs = {k: plain_logits(folder, seqs[k]) for k in seqs}
        for k in seqs:
            runner.create(k)
        fed = {k: 0 for k in seqs}

        def feed(*parts):
            entries, places = [], []
            for k, n in parts:
                entries.append(StepEntry(k, seqs[k][fed[k]:fed[k] + n], [0, n - 1] if n > 1 else [0]))
                places += [(k, fed[k]), (k, fed[k] + n - 1)] if n > 1 else [(k, fed[k])]
                fed[k] += n
            logits = runner.step(entries).float().cpu().numpy()
            for row, (k, pos) in zip(logits, places):
                assert_close(row[None], refs[k][pos][None], "bfloat16", f"round {round_} request {k} position {pos}")

        feed(("a", 90))                                   # more than 64 rows: the library's products
        feed(("b", 70), ("c", 3))
        feed(("c", 40), ("d", 20))                        # 60 rows: four row tiles of the wide product
        feed(("e", 7))
        for _ in range(3):
            feed(("a", 1), ("b", 1), ("c", 1), ("d", 1), ("e", 1))   # decode steps of five rows
        feed(("a", 1), ("b", 1), ("c", 30), ("d", 1), ("e", 50))     # mixed: 83 rows
        for _ in range(2):
            feed(("a", 1), ("b", 1), ("c", 1), ("d", 1), ("e", 1))
        for k in seqs:
            runner.release(k)
    if execution == "graph":
        replayed = [key for key, p in runner.programs.items() if p["graph"] is not None and p["runs"] >= 3]
        assert any(key[0] > 64 for key in replayed) and any(key[3] for key in replayed)
    if sizes == "1.7b":     # few rows: the wide product's slices; many rows: the library's bf16 product
        assert sum(u is not None and u[1] > 1 for u in left) >= 3, "no cut product was left to the norm that follows"
        assert sum(u is not None and u[1] == 0 for u in left) >= 3, "no library product was left to the norm that follows"
    runner.cache.check()


@pytest.mark.parametrize("name", ["a", "c"])
@pytest.mark.parametrize("item_tiles", [1, 2])
def test_long_portions_through_block_tiles_match_the_plain_model(folders, name, item_tiles):
    """With many heads and long portions the attention of a prompt step runs in blocks whose waves share keys
    through LDS; forced here on small models: a whole prompt, then a second portion beside another request."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from conftest import plain_logits, assert_close
    V = TINY[name]["vocab_size"]
    model = load_model(folders[name], dtype="bfloat16")
    from conftest import tune_attention
    tune_attention(model, block_tiles=item_tiles, square_tiles=0)
    runner = ModelRunner(model, n_pages=64, page_size=8, max_requests=4)
    seqs = {k: random_tokens(500 + i, 230, V) for i, k in enumerate("pq")}
    refs = {k: plain_logits(folders[name], seqs[k]) for k in seqs}
    for k in seqs:
        runner.create(k)
    got = runner.step([StepEntry("p", seqs["p"][:150], list(range(150)))]).float().cpu().numpy()
    assert_close(got, refs["p"][:150], "bfloat16", "first portion")
    got = runner.step([StepEntry("p", seqs["p"][150:], list(range(80))),
                       StepEntry("q", seqs["q"][:97], list(range(97)))]).float().cpu().numpy()
    assert_close(got[:80], refs["p"][150:], "bfloat16", "second portion on a cached prefix")
    assert_close(got[80:], refs["q"][:97], "bfloat16", "another request in the same step")


@pytest.mark.parametrize("name", ["a", "c"])
@pytest.mark.parametrize("square, halves", [(1, 1), (2, 1), (3, 1), (4, 1), (1, 2), (2, 2)])
def test_long_portions_through_square_tiles_match_the_plain_model(folders, name, square, halves):
    """Long portions of long contexts run on the 32 x 32 matrix instruction with waves of their own for the copies;
    forced here on small models: a whole prompt, then a second portion beside another request, then graph replays."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from conftest import plain_logits, assert_close
    V = TINY[name]["vocab_size"]
    model = load_model(folders[name], dtype="bfloat16")
    seqs = {k: random_tokens(600 + i, 230, V) for i, k in enumerate("pq")}
    refs = {k: plain_logits(folders[name], seqs[k]) for k in seqs}
    for execution in ("eager", "graph"):
        from conftest import tune_attention
        tune_attention(model, square_tiles=square, square_halves=halves)
        runner = ModelRunner(model, n_pages=64, page_size=8, max_requests=4, execution=execution)
        for k in seqs:
            runner.create(k)
        got = runner.step([StepEntry("p", seqs["p"][:150], list(range(150)))]).float().cpu().numpy()
        assert_close(got, refs["p"][:150], "bfloat16", f"{execution}: first portion")
        got = runner.step([StepEntry("p", seqs["p"][150:], list(range(80))),
                           StepEntry("q", seqs["q"][:97], list(range(97)))]).float().cpu().numpy()
        assert_close(got[:80], refs["p"][150:], "bfloat16", f"{execution}: second portion on a cached prefix")
        assert_close(got[80:], refs["q"][:97], "bfloat16", f"{execution}: another request in the same step")
        runner.cache.check()


def test_temperature_sampling_is_seeded_and_independent_of_the_batch(folders):
    from runtime.engine.scheduler import Engine, Request
    V = TINY["b"]["vocab_size"]
    prompts = [random_tokens(80 + i, n, V) for i, n in enumerate([1, 9, 33, 64])]

    def generate(which, **kw):
        e = Engine.from_folder(folders["b"], dtype="float32", pages=64, page_size=8, **kw)
        for i in which:
            e.submit(Request(str(i), prompts[i], 12, temperature=0.8, seed=100 + i))
        return {r.key: r.generated for r in e.run()}

    together = generate(range(4), token_budget=16, prefill_chunk=7)
    again = generate(range(4), token_budget=16, prefill_chunk=7)
    alone = {}
    for i in range(4):
        alone.update(generate([i], token_budget=64, prefill_chunk=64))
    assert together == again == alone
    greedy = generate(range(4), token_budget=16, prefill_chunk=7)
    e = Engine.from_folder(folders["b"], dtype="float32", pages=64, page_size=8)
    assert e.generate(prompts[:2], max_new_tokens=12) != [together["0"], together["1"]]   # sampling is not greedy here


@pytest.mark.parametrize("overlap,execution", [(False, "eager"), (True, "graph")])
def test_sampled_tokens_are_those_of_a_plain_sampler(folders, overlap, execution):
    """The tokens the engine samples (prompts of 1, 9, 33 and 64 tokens cut into portions of 7 beside decoding
    requests, 12 tokens each at temperature 0.8) against float64 softmax(plain logits / T) drawn by inverse CDF at
    uniform01(seed, index).  Each token is checked given the engine's own tokens before it; a draw that falls
    within 2e-5 of an edge of its interval (the engine's softmax is 32-bit; a token's interval is about 2e-3 wide
    with this vocabulary) may land on the neighbour and is only required to."""
    import plain_sampling
    from runtime.engine.scheduler import Engine, Request
    cfg, w = P.read_folder(folders["b"])
    V = TINY["b"]["vocab_size"]
    prompts = [random_tokens(80 + i, n, V) for i, n in enumerate([1, 9, 33, 64])]
    e = Engine.from_folder(folders["b"], dtype="float32", pages=64, page_size=8, token_budget=16, prefill_chunk=7,
                           execution=execution, overlap=overlap)
    for i, p in enumerate(prompts):
        e.submit(Request(str(i), p, 12, temperature=0.8, seed=100 + i))
    got = {r.key: r.generated for r in e.run()}
    exact = 0
    for i, p in enumerate(prompts):
        tokens = got[str(i)]
        assert len(tokens) == 12
        for n, token in enumerate(tokens):
            logits = P.forward(cfg, w, p + tokens[:n])[-1]
            want, room = plain_sampling.draw(logits, 0.8, 100 + i, n)
            if room > 2e-5:
                assert token == want, f"request {i} token {n}: {token} instead of {want}"
                exact += 1
            else:
                assert abs(token - want) <= 1, f"request {i} token {n}: {token} is no neighbour of {want}"
    assert exact >= 40, "too few draws away from the edges to say anything"
    assert any(t != g for i, p in enumerate(prompts) for t, g in zip(got[str(i)], P.greedy(cfg, w, p, 12))), "nothing was sampled"


@pytest.mark.parametrize("execution", ["eager", "graph"])
def test_overlapped_ticks_sample_and_stop_like_plain_ticks(folders, execution):
    """Steps launched before the tokens of the step before are read: the same sampled tokens, the same
    stop at an end-of-sequence token (found one step late, the extra token dropped), every page back."""
    from runtime.engine.scheduler import Engine, Request
    V = TINY["b"]["vocab_size"]
    prompts = [random_tokens(60 + i, n, V) for i, n in enumerate([1, 9, 33, 20, 5])]
    news = [12, 1, 7, 12, 2]

    def run(overlap, eos=None):
        e = Engine.from_folder(folders["b"], dtype="float32", pages=24, page_size=8, execution=execution,
                               token_budget=12, prefill_chunk=7, max_active=3, overlap=overlap)
        for i, (p, n) in enumerate(zip(prompts, news)):
            e.submit(Request(str(i), p, n, eos_token_id=eos, temperature=0.7 if i % 2 else 0.0, seed=5 + i))
        out = {r.key: r.generated for r in e.run()}
        e.runner.cache.check()
        assert e.runner.cache.free_pages() == [24] and not e.reserved and e.inflight is None
        return out

    plain = run(False)
    assert run(True) == plain
    assert [len(plain[str(i)]) for i in range(5)] == news
    eos = plain["0"][4]
    stopped = run(False, eos)
    assert len(stopped["0"]) <= 5 and stopped["0"][-1] == eos
    assert run(True, eos) == stopped


@pytest.mark.parametrize("execution", ["eager", "graph"])
def test_a_step_that_fails_leaves_its_requests_where_they_stood(folders, execution):
    """Slots are placed before a step runs, the tokens are counted only once it is launched: a step that fails on
    the way gives its pages back, and the same step, tried again, gives the right logits."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from conftest import plain_logits, assert_close
    V = TINY["a"]["vocab_size"]
    model = load_model(folders["a"], dtype="float32")
    r = ModelRunner(model, n_pages=12, page_size=8, execution=execution)
    a, b = random_tokens(31, 30, V), random_tokens(32, 12, V)
    r.create("a"); r.create("b")
    r.step([StepEntry("a", a[:5], []), StepEntry("b", b[:3], [])])
    free = r.cache.free_pages()
    real = model.forward

    def broken(ctx):
        raise RuntimeError("a kernel refused its shape")

    model.forward = broken
    try:
        with pytest.raises(RuntimeError, match="refused"):
            r.step([StepEntry("a", a[5:25], [19]), StepEntry("b", [b[3]], [0])])
    finally:
        model.forward = real
    assert (r.length("a"), r.length("b")) == (5, 3) and r.cache.free_pages() == free
    r.cache.check()
    out = r.step([StepEntry("a", a[5:25], [19]), StepEntry("b", [b[3]], [0])]).cpu().numpy()
    assert (r.length("a"), r.length("b")) == (25, 4)
    assert_close(out[:1], plain_logits(folders["a"], a)[24:25], "float32", "the portion, tried again")
    assert_close(out[1:], plain_logits(folders["a"], b)[3:4], "float32", "the decoded token, tried again")
    r.cache.check()


def test_fork_shares_a_prefix_and_copies_on_write(folders):
    # reference tests/test_execution.py:55-64
    from runtime.engine import load_model, ModelRunner, StepEntry
    from conftest import plain_logits, assert_close
    V = TINY["a"]["vocab_size"]
    model = load_model(folders["a"], dtype="float32")
    r = ModelRunner(model, n_pages=12, page_size=16)
    prefix = random_tokens(3, 21, V)
    r.create("src")
    r.step([StepEntry("src", prefix, [])])
    r.fork("src", "dst")
    assert r.cache.table(0, "src") == r.cache.table(0, "dst")
    tail_a, tail_b = random_tokens(4, 6, V), random_tokens(5, 6, V)
    out = r.step([StepEntry("src", tail_a, list(range(6))), StepEntry("dst", tail_b, list(range(6)))]).cpu().numpy()
    assert r.cache.table(0, "src")[0] == r.cache.table(0, "dst")[0]     # the full page stays shared
    assert r.cache.table(0, "src")[1] != r.cache.table(0, "dst")[1]     # the partly filled one was copied
    assert_close(out[:6], plain_logits(folders["a"], prefix + tail_a)[21:], "float32", "source after fork")
    assert_close(out[6:], plain_logits(folders["a"], prefix + tail_b)[21:], "float32", "fork")
    r.release("src"); r.release("dst"); r.cache.check()
    assert r.cache.free_pages() == [12]


@pytest.mark.parametrize("execution", ["eager", "graph"])
def test_decode_rows_handed_out_longest_first_give_the_same_logits(folders, execution):
    """From many blocks on, an unsplit decode launch lists its rows longest first (told here to do so always): the same
    logits bit for bit as in the rows' own order, for requests of very different lengths, also under captured programs
    with padding rows."""
    from runtime.engine import load_model, ModelRunner, StepEntry
    from conftest import tune_attention
    name = "a"
    V = TINY[name]["vocab_size"]
    seqs = {k: random_tokens(700 + i, n, V) for i, (k, n) in enumerate(zip("uvwxy", (90, 12, 47, 90, 9)))}
    outs = []
    for order_from in (1, 10 ** 9):
        model = load_model(folders[name], dtype="bfloat16")
        tune_attention(model, order_rows_from=order_from, rows_launch=(4, 1))
        runner = ModelRunner(model, n_pages=64, page_size=8, max_requests=8, execution=execution)
        for k, toks in seqs.items():
            runner.create(k)
            runner.step([StepEntry(k, toks[:-6], [])])
        got = []
        for t in range(6):
            live = [k for k in seqs if not (t >= 3 and k == "v")]                  # five rows (padded to eight), then four
            got.append(runner.step([StepEntry(k, [seqs[k][len(seqs[k]) - 6 + t]], [0]) for k in live]).float().cpu())
        outs.append(got)
        assert any("RowsLongestFirst" in a for a in runner.report()["step_arrays"])
    for with_order, without in zip(*outs):
        assert torch.equal(with_order, without)
    ref = {k: plain_logits(folders[name], seqs[k]) for k in seqs}
    first = outs[0][0].numpy()
    for row, k in enumerate(seqs):
        assert_close(first[row:row + 1], ref[k][len(seqs[k]) - 6:len(seqs[k]) - 5], "bfloat16", f"request {k}")


def test_command_line(folders, tmp_path):
    requests = [{"key": "x", "prompt": [1, 2, 3, 4, 5], "max_new_tokens": 4}, {"key": "y", "prompt": [9], "max_new_tokens": 3}]
    (tmp_path / "requests.json").write_text(json.dumps(requests))
    env = dict(os.environ, PYTHONPATH=str(ROOT))
    proc = subprocess.run([sys.executable, "-m", "runtime", "--checkpoint", str(folders["a"]), "--dtype", "float32",
                           "--requests", str(tmp_path / "requests.json"), "--policy", "chunked", "--pages", "16",
                           "--page-size", "8", "--token-budget", "6", "--prefill-chunk", "3"],
                          capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    result = json.loads(proc.stdout)
    cfg, w = P.read_folder(folders["a"])
    assert result["dtype"] == "float32" and result["weights"] == "pretrained-local"
    by_key = {r["key"]: r for r in result["requests"]}
    assert by_key["x"]["generated"] == P.greedy(cfg, w, [1, 2, 3, 4, 5], 4) and by_key["x"]["status"] == "finished"
    assert by_key["y"]["generated"] == P.greedy(cfg, w, [9], 3) and by_key["y"]["ttft_ms"] > 0
    proc = subprocess.run([sys.executable, "-m", "runtime", "--model", "tiny-b", "--tokens", "5,6,7", "--max-new-tokens", "3",
                           "--execution", "graph", "--overlap", "--pages", "0", "--report"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout)
    assert out["weights"] == "random-tiny-b" and len(out["requests"][0]["generated"]) == 3
    told = out["runner"]
    assert told["steps"] == told["eager_steps"] + told["replays"] >= 3 and told["programs"] >= 1
    assert told["workspace_bytes"] > 0 and told["cache"][0]["resident_pages"] == 0


def test_smoke_entry():
    sys.path.insert(0, str(ROOT))
    import __graft_entry__
    __graft_entry__.smoke()
