"""python -m runtime.measure <workload>: what single kernels and the machine cost, one JSON line each.

  floor                    a captured chain of kernels that do nothing (what a launch costs), and a meeting of all
                           blocks inside one kernel (what a barrier over the grid costs instead)
  attention                the prompt attention kernel alone at the family's head shapes, in the form the rule picks
  attention_forms          every form of that kernel at a grid of head shapes, beside the form the rule picks
  decode_attention_shapes  every launch shape of the decode attention kernel at a grid of requests and contexts,
                           beside the one the rule picks
  chain                    a captured chain of 150 dependent matrix-vector products of the 135M sizes' shapes, each
                           the leanest kernel there is (what a decode step of one request costs at the least); the
                           same chain with its kernels alternating on two streams and handing over through counters
                           in memory instead of the stream's order; and two independent chains on two streams
  reread                   GB/s of a kernel that reads the same buffer again and again, by the buffer's size (what
                           the L2 caches and the memory-side cache hold from kernel to kernel)
  hot_weights              decode steps with every layer sharing one layer's weights (the order of layers names one
                           layer for every place) against distinct layers: what weights that are already in a cache
                           are worth, the bound of anything that fetches weights ahead
  one_launch               a mock decode step as ONE launch: the blocks of each die meet inside the kernel through
                           that die's L2, a request a die (what a step fused into one kernel would cost at the least)
  stream_loads             decode steps with ordinary and with non-temporal loads of keys and values beside the rule's
                           choice, and the decode attention kernel alone over rows of mixed lengths, in row order and
                           longest first
"""
import argparse
import json
import sys
import time

PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}


def launch_floor(args):
    """Microseconds a kernel of a captured chain costs when it computes nothing: 1,000 launches of an empty kernel
    (one block, and one block a compute unit) in one graph, replayed; the median of 20 replays.  A decode step of
    L layers is 5 L + 4 kernels, so this times that count is the part of a step that no kernel work can remove.
    Beside it, what the other way to order a step's parts costs: a meeting of all blocks inside one kernel (counters
    in memory, 200 meetings, the median of 5 runs), alone and with 8 x 576 floats passed from all blocks to all."""
    import statistics
    import torch
    from runtime.config import preset
    from runtime import measure
    chain = 1000
    out = {}
    for name, blocks in (("one_block", 1), ("block_per_cu", torch.cuda.get_device_properties(0).multi_processor_count)):
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            measure.idle(blocks)
            stream.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                for _ in range(chain):
                    measure.idle(blocks)
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
            words = measure.grid_meet(blocks, rounds, exchange)
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
    from runtime.kernels.attention import fill_tasks
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
    from runtime.kernels.attention import prompt_form
    for name in ("smollm2-135m", "smollm2-1.7b", "llama-3-8b"):
        raw = preset(name)
        heads, kv_heads = raw["num_attention_heads"], raw["num_key_value_heads"]
        D = raw.get("head_dim") or raw["hidden_size"] // heads
        for T in [int(t) for t in args.attention_rows.split(",") if t]:
            form = prompt_form(T, 1, T, heads, kv_heads, D, P)
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
    from runtime.kernels.attention import prompt_form
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
            pick = tuple(prompt_form(T, 1, T, heads, kv_heads, D, P))
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
    merge kernel when the keys are split) beside the one `kernels.attention.rows_launch` picks.  Keys and values of up to
    eight layers take turns, so that nothing is read from a cache twice in a row.  One line a point on stderr, then one
    JSON line with the worst and the mean loss of the rule."""
    import math
    import torch
    from runtime.config import preset
    from runtime.kernels import ops
    from runtime.kernels.attention import rows_launch, rows_stream_loads
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
                pick = tuple(rows_launch(blocks, C, per_chunk, D))
                pick += (rows_stream_loads(blocks, C, pick[0], pick[1], D),)
                shapes = {(w, n, nt) for w in (4, 8) for n in (1, 2, 4, 8, 16, 32) for nt in (False, True)
                          if (n == 1 or n * 32 <= C) and blocks * n <= 16384} | {pick}
                us = {}
                for waves, splits, stream_loads in sorted(shapes):
                    ws = (torch.empty(B * heads * splits * D, device=dev), torch.empty(B * heads * splits * 2, device=dev))

                    def run(i):
                        ops.attention_mfma(q, heads * D, ks[i], vs[i], tables, seg, pos, out, heads, kv, D, P, None, 1 / math.sqrt(D),
                                           None, splits, ws, waves, stream_loads=stream_loads)
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
                    us[(waves, splits, stream_loads)] = sorted(times)[1]
                best = min(us, key=us.get)
                loss = us[pick] / us[best] - 1
                losses.append(loss)
                label = lambda shape: f"{shape[0]} waves x {shape[1]}" + (" nt" if shape[2] else "")
                points[f"{name}_{B}x{C}"] = {"pick": label(pick), "pick_us": round(us[pick], 1), "best": label(best),
                                             "best_us": round(us[best], 1), "loss": round(loss, 3)}
                print(f"{name:13s} {B:3d} rows x {C:5d} keys  pick {label(pick):13s} {us[pick]:7.1f} us   best {label(best):13s} {us[best]:7.1f} us   "
                      + "  ".join(f"{w}x{n}{'nt' if nt else ''}: {v:.1f}" for (w, n, nt), v in sorted(us.items())), file=sys.stderr, flush=True)
    print(json.dumps({"metric": "loss of the rule that picks the decode attention launch shape against the best shape of each point",
                      "unit": "fraction", "n_gpus": 1, "value": round(max(losses), 3), "higher_is_better": False,
                      "mean": round(sum(losses) / len(losses), 4), "points": points}))
    return 0


def chain(args):
    """See the module's text.  One line: microseconds a link."""
    import statistics
    import torch
    from runtime import measure
    dev = torch.device("cuda:0")
    layers = args.chain_layers
    shapes = [(512, 512), (512, 512), (512, 512), (1536, 512), (512, 1536)] * layers      # (N, K): five products a layer
    gen = torch.Generator(device=dev).manual_seed(0)
    weights = [(torch.rand(n, k, generator=gen, device=dev) * 2 - 1).mul_(1.7 / k ** 0.5).bfloat16() for n, k in shapes]
    links = len(shapes)

    def buffers():
        acts = torch.zeros(links + 1, 1536, device=dev)
        acts[0, :512] = torch.linspace(0.5, 1.0, 512, device=dev)
        return acts
    acts, acts2 = buffers(), buffers()
    counters = torch.zeros((links + 2) * 64, dtype=torch.int32, device=dev)
    err = counters[(links + 1) * 64:]

    def run(i, buf, wait):
        cnt = None
        if wait:
            cnt = (counters[i * 64:], 0 if i == 0 else shapes[i - 1][0] // 4, counters[(i + 1) * 64:], err)
        measure.chain_phase(weights[i], buf[i], buf[i + 1], cnt, wait)

    def capture(stream, body):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            body(); stream.synchronize()
            with torch.cuda.graph(graph, stream=stream):
                body()
        return graph

    def timed(step, reps=15):
        times = []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            step()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        return statistics.median(times) * 1e6

    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    plain = capture(s1, lambda: [run(i, acts, False) for i in range(links)])
    torch.cuda.synchronize()
    reference = acts[links, :512].clone()
    out = {"links": links, "weights_mb": round(sum(w.numel() * 2 for w in weights) / 2 ** 20, 1)}
    out["one_stream_us_a_link"] = round(timed(lambda: plain.replay()) / links, 3)
    # the same kernels with the hand-over through counters, still in one stream's order: what the hand-over itself costs
    in_order = capture(s1, lambda: (counters.zero_(), [run(i, acts, True) for i in range(links)]))
    out["one_stream_with_counters_us_a_link"] = round(timed(lambda: in_order.replay()) / links, 3)
    # even links on one stream, odd links on the other, nothing but the counters between them
    even = capture(s1, lambda: [run(i, acts, True) for i in range(0, links, 2)])
    odd = capture(s2, lambda: [run(i, acts, True) for i in range(1, links, 2)])

    def two_streams():
        with torch.cuda.stream(s1):
            counters.zero_()
            s2.wait_stream(s1)
            even.replay()
        with torch.cuda.stream(s2):
            odd.replay()
    acts[links].zero_()
    out["two_streams_with_counters_us_a_link"] = round(timed(two_streams) / links, 3)
    torch.cuda.synchronize()
    out["two_streams_same_result"] = bool(torch.equal(acts[links, :512], reference)) and int(err[0]) == 0
    # two independent chains, a stream each: what running two steps side by side costs
    other = capture(s2, lambda: [run(i, acts2, False) for i in range(links)])

    def side_by_side():
        with torch.cuda.stream(s1):
            plain.replay()
        with torch.cuda.stream(s2):
            other.replay()
    out["two_independent_chains_us_a_link_of_each"] = round(timed(side_by_side) / links, 3)
    print(json.dumps({"metric": "microseconds a link of a captured chain of dependent matrix-vector kernels", "unit": "us",
                      "value": out["one_stream_us_a_link"], "higher_is_better": False, "n_gpus": 1, **out}))
    return 0


def one_launch(args):
    """A decode step as one launch against the step of 154 launches: the mock of csrc/measure.hip (blocks of a die
    meet inside the kernel through that die's L2; every die runs the step of a request of its own) at the sizes of
    --model, with one die or all eight at work, 32 or 64 blocks a die, one row's keys a die or eight rows'.  What the
    mock leaves out (norms, rotary embedding, softmax, the merge of split attention) would only add to its times."""
    import statistics
    import torch
    from runtime import measure
    from runtime.config import preset
    dev = torch.device("cuda:0")
    raw = preset(args.model)
    H, I, L = raw["hidden_size"], raw["intermediate_size"], raw["num_hidden_layers"]
    D = raw.get("head_dim") or H // raw["num_attention_heads"]
    qkv = (raw["num_attention_heads"] + 2 * raw["num_key_value_heads"]) * D
    context = 2048
    row_words = context * raw["num_key_value_heads"] * D * 2 * 2 // 16           # keys and values of a layer, one row, 16-byte words
    weights = torch.full((L * ((qkv + H + 2 * I) * H + H * I),), 0.01, dtype=torch.bfloat16, device=dev)
    kv = torch.ones(8 * L * 8 * row_words * 4, dtype=torch.int32, device=dev)
    scratch = torch.zeros(8 * 16384, device=dev)
    words = torch.zeros(1024, dtype=torch.int32, device=dev)
    stream = torch.cuda.Stream()
    points = {}
    for blocks in (32, 64):
        for active in (1, 8):
            for rows in (1, 8):
                def body():
                    words.zero_()
                    measure.one_launch_step(weights, L, H, qkv, I, kv, rows * row_words, scratch, words, blocks=blocks, active=active)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.stream(stream):
                    body(); stream.synchronize()
                    if int(words[1023]):
                        raise SystemExit("a block gave up waiting at a meeting")
                    with torch.cuda.graph(graph, stream=stream):
                        body()
                    times = []
                    for _ in range(12):
                        stream.synchronize()
                        t0 = time.perf_counter()
                        graph.replay()
                        stream.synchronize()
                        times.append(time.perf_counter() - t0)
                    if int(words[1023]):
                        raise SystemExit("a block gave up waiting at a meeting")
                points[f"{blocks}_blocks_a_die_{active}_dies_{rows}_rows_each"] = round(statistics.median(times) * 1e3, 4)
    print(json.dumps({"metric": "milliseconds of a mock decode step run as one launch, blocks meeting inside their die", "unit": "ms",
                      "value": points["32_blocks_a_die_8_dies_1_rows_each"], "higher_is_better": False, "n_gpus": 1, "model": args.model,
                      "layers": L, "weights_mb_a_layer": round(((qkv + H + 2 * I) * H + H * I) * 2 / 2 ** 20, 2),
                      "keys_and_values_mb_a_layer_and_row": round(row_words * 16 / 2 ** 20, 2), "ms_a_step": points}))
    return 0


def reread(args):
    """GB/s of the read-only kernel over a buffer that it reads again and again (20 or more passes in one captured
    graph, the median of five replays), by the buffer's size."""
    import statistics
    import torch
    from runtime import measure
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    out = {}
    for mb in (8, 16, 32, 64, 128, 256, 512, 2048):
        a = torch.empty(mb << 20, dtype=torch.uint8, device="cuda")
        a.zero_()
        passes = max(4, 2048 // mb)
        graph = torch.cuda.CUDAGraph()
        measure.stream_read(a, sink, 1024); torch.cuda.synchronize()
        with torch.cuda.graph(graph):
            for _ in range(passes):
                measure.stream_read(a, sink, 1024)
        graph.replay(); torch.cuda.synchronize()
        times = []
        for _ in range(5):
            t0 = time.perf_counter(); graph.replay(); torch.cuda.synchronize(); times.append((time.perf_counter() - t0) / passes)
        out[f"{mb}_MB"] = {"us_a_pass": round(statistics.median(times) * 1e6, 1), "GB/s": round((mb << 20) / statistics.median(times) / 1e9)}
        del a, graph
    print(json.dumps({"metric": "GB/s of a read-only kernel over a buffer that is read again and again, by size", "unit": "GB/s",
                      "value": out["32_MB"]["GB/s"], "higher_is_better": True, "n_gpus": 1, "sizes": out}))
    return 0


def _decode_step_ms(runner, sampler, rng, vocab, batch, prompt, steps=64, repeats=4):
    """Seconds a decode step of `batch` requests takes after prompts of `prompt` random tokens: overlapped steps, as the
    benchmark times them; the median of the repeats but the first.  The requests are released again."""
    import statistics
    import numpy as np
    import torch
    from runtime.engine import StepEntry
    keys = [f"{batch}-{prompt}-{i}" for i in range(batch)]
    last = []
    for key in keys:
        runner.create(key)
        logits = runner.step([StepEntry(key, rng.integers(0, vocab, size=prompt, dtype=np.int32), [prompt - 1])])
        last.append(sampler.pick(logits, [(0.0, 0, 0)])[0])
    params, unread, times = [(0.0, 0, 0)] * batch, None, []
    for rep in range(repeats):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            entries = [StepEntry(k, [0], [0], pending=True) for k in keys] if unread is not None else [StepEntry(k, [t], [0]) for k, t in zip(keys, last)]
            unread = runner.pick(sampler, runner.step(entries), params)
        torch.cuda.synchronize()
        times.append((time.perf_counter() - t0) / steps)
    for key in keys:
        runner.release(key)
    return statistics.median(times[1:])


def hot_weights(args):
    """Decode steps (captured programs, steps overlapped, as the benchmark times them) of 1, 8 and 64 requests after
    2,048-token prompts: a model whose layers are distinct against the same model with one layer's weights at every
    place of the order (every place still keeps a cache of its own)."""
    import numpy as np
    import torch
    from runtime.config import preset
    from runtime.engine import ModelRunner, random_model
    from runtime.models import ScheduleEntry
    from runtime.sampling import Sampler
    out = {}
    for name, layers in (("smollm2-135m", 30), ("smollm2-1.7b", 8)):
        raw = preset(name)
        raw["num_hidden_layers"] = layers
        raw["max_position_embeddings"] = 4096
        for shared in (False, True):
            model = random_model(raw, seed=0)
            if shared:
                model.schedule = [ScheduleEntry(0) for _ in range(layers)]
            sampler, rng = Sampler(), np.random.default_rng(0)
            runner = ModelRunner(model, n_pages=64 * 4096 // 16, page_size=16, max_requests=64, execution="graph")
            result = {f"b{batch}_ms": round(_decode_step_ms(runner, sampler, rng, raw["vocab_size"], batch, 2048) * 1e3, 4) for batch in (1, 8, 64)}
            out[f"{name}_{layers}_layers_{'one_layers_weights_everywhere' if shared else 'distinct_layers'}"] = result
            del runner, model
            torch.cuda.empty_cache()
    print(json.dumps({"metric": "ms a decode step with distinct layers and with one layer's weights at every place", "unit": "ms",
                      "value": out["smollm2-135m_30_layers_distinct_layers"]["b8_ms"], "higher_is_better": False, "n_gpus": 1, "steps": out}))
    return 0


def stream_loads(args):
    """Non-temporal loads of keys and values in decode attention, and the order in which its rows are handed out.
    First whole decode steps (captured programs, overlapped) at the three sizes, with ordinary loads, with non-temporal
    ones and with what `kernels.attention.rows_stream_loads` picks; then the kernel alone over 64 rows of mixed lengths
    (228 to 2,304 keys, the serving workload's) at the 1.7B head shape, in row order and longest first, against 64 rows
    of their mean length.  One line a point on stderr, then one JSON line."""
    import math
    import numpy as np
    import torch
    from runtime.config import preset
    from runtime.engine import ModelRunner, random_model
    from runtime.kernels import attention, ops
    from runtime.sampling import Sampler
    rule = attention.rows_stream_loads
    steps = {}
    grid = [("smollm2-135m", 30, [(1984, [1, 8, 16, 64]), (7936, [8, 64])]),
            ("smollm2-1.7b", 8, [(1984, [1, 8, 32, 64]), (7936, [1, 8])]),
            ("llama-3-8b", 8, [(1984, [1, 8, 64]), (7936, [8, 64])])]
    try:
        for name, layers, points in grid:
            raw = preset(name)
            raw["num_hidden_layers"] = layers
            raw["max_position_embeddings"] = 8448
            model = random_model(raw, seed=0)
            sampler, rng = Sampler(), np.random.default_rng(0)
            runner = ModelRunner(model, n_pages=64 * 8448 // args.page_size, page_size=args.page_size, max_requests=64, execution="graph")
            for prompt, batches in points:
                for batch in batches:
                    ms = {}
                    for how, pick in (("ordinary", lambda *a: False), ("non_temporal", lambda *a: True), ("rule", rule)):
                        attention.rows_stream_loads = pick
                        runner.programs.clear()          # the choice is part of a captured program
                        ms[how] = round(_decode_step_ms(runner, sampler, rng, raw["vocab_size"], batch, prompt, steps=32) * 1e3, 4)
                    steps[f"{name}_{layers}_layers_{batch}x{prompt}"] = ms
                    print(f"{name:13s} {batch:3d} rows x {prompt:5d} keys  ordinary {ms['ordinary']:.4f} ms  non-temporal {ms['non_temporal']:.4f}"
                          f" ({100 * (ms['non_temporal'] / ms['ordinary'] - 1):+5.1f} %)  rule {ms['rule']:.4f}", file=sys.stderr, flush=True)
            del runner, model
            torch.cuda.empty_cache()
    finally:
        attention.rows_stream_loads = rule
    # the kernel alone: 64 rows, 32 key heads of 64 (the 1.7B sizes), pages scattered, three layers' keys and values in turn
    dev, P, heads, kv, D = torch.device("cuda:0"), args.page_size, 32, 32, 64
    gen = torch.Generator().manual_seed(0)
    mixed = [int(x) for x in torch.randint(228, 2305, (64,), generator=gen)]
    kernel = {}
    for label, lengths in (("mixed_228_to_2304", mixed), (f"all_{sum(mixed) // 64}", [sum(mixed) // 64] * 64)):
        pages_per = -(-max(lengths) // P)
        n_pages = 64 * pages_per
        ks = [torch.randn(n_pages, kv, P, D, device=dev).bfloat16() for _ in range(3)]
        vs = [torch.randn(n_pages, kv, D, P, device=dev).bfloat16() for _ in range(3)]
        tables = torch.randperm(n_pages, device=dev).int().view(64, pages_per)
        q = torch.randn(64, heads * D, device=dev).bfloat16()
        seg = torch.arange(64, device=dev, dtype=torch.int32)
        pos = torch.tensor([n - 1 for n in lengths], device=dev, dtype=torch.int32)
        out = torch.empty(64, heads * D, device=dev).bfloat16()
        longest_first = torch.argsort(-pos.long(), stable=True).int()
        for order_name, ids in (("row_order", None), ("longest_first", longest_first)):
            for nt in (False, True):
                def run(i):
                    ops.attention_mfma(q, heads * D, ks[i], vs[i], tables, seg, pos, out, heads, kv, D, P, None, 1 / math.sqrt(D),
                                       None, 1, None, 4, row_ids=ids, stream_loads=nt)
                for i in range(3):
                    run(i)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    for i in range(6):
                        run(i % 3)
                graph.replay()
                torch.cuda.synchronize()
                times = []
                for _ in range(5):
                    t0 = time.perf_counter()
                    graph.replay()
                    torch.cuda.synchronize()
                    times.append((time.perf_counter() - t0) / 6 * 1e6)
                kernel[f"{label}_{order_name}_{'non_temporal' if nt else 'ordinary'}"] = round(sorted(times)[2], 1)
        print(f"kernel alone, 64 rows {label}: " + "  ".join(f"{k[len(label) + 1:]} {v} us" for k, v in kernel.items() if k.startswith(label)),
              file=sys.stderr, flush=True)
    print(json.dumps({"metric": "ms a decode step of 8 requests at the 135M sizes with the rule's choice of loads for keys and values",
                      "unit": "ms", "value": steps["smollm2-135m_30_layers_8x1984"]["rule"], "higher_is_better": False, "n_gpus": 1,
                      "decode_steps_ms": steps, "kernel_alone_us": kernel}))
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m runtime.measure")
    ap.add_argument("workload", choices=["floor", "attention", "attention_forms", "decode_attention_shapes", "chain", "reread", "hot_weights", "one_launch", "stream_loads"])
    ap.add_argument("--chain-layers", type=int, default=30, help="chain: layers of five products each (30: 113 MB of weights; 240: 904 MB, "
                                                                 "more than the memory-side cache holds)")
    ap.add_argument("--model", default="smollm2-135m", help="floor: the preset whose decode step the floor is priced for")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--attention-rows", default="2048,7936", help="attention workloads: prompt lengths (comma separated)")
    args = ap.parse_args(argv)
    return {"floor": launch_floor, "attention": prompt_attention, "attention_forms": attention_forms,
            "decode_attention_shapes": decode_attention_shapes, "chain": chain, "reread": reread, "stream_loads": stream_loads,
            "hot_weights": hot_weights, "one_launch": one_launch}[args.workload](args)


if __name__ == "__main__":
    sys.exit(main())
