"""The scheduler's decisions on the CPU, above a stand-in for the step function
(a deterministic function of each request's token history) and the real cache
manager without device memory."""
import hashlib

import numpy as np
import pytest
import torch

from runtime.cache import CacheManager, KVNeed
from runtime.engine.scheduler import Engine, Request


class FakeModel:
    vocab_size = 50


class FakeRunner:
    """Same interface as ModelRunner, logits = hash of the request's history."""

    def __init__(self, pages=20, page_size=4, max_requests=8, max_context=64):
        self.model, self.page_size, self.max_requests, self.max_context = FakeModel(), page_size, max_requests, max_context
        self.cache = CacheManager({0: KVNeed(1, 8)}, pages, page_size, max_requests)
        self.history, self.calls = {}, []

    def create(self, key):
        self.cache.create(key); self.history[key] = []

    def release(self, key):
        self.cache.release(key); del self.history[key]

    def step(self, entries):
        self.cache.append_many([(e.request, len(e.tokens)) for e in entries])
        self.calls.append([(e.request, len(e.tokens), list(e.want)) for e in entries])
        rows = []
        for e in entries:
            for i, t in enumerate(e.tokens):
                self.history[e.request].append(int(t))
                if i in e.want:
                    digest = hashlib.sha256(str(self.history[e.request]).encode()).digest()
                    rows.append(np.frombuffer(digest * 2, dtype=np.uint8)[:50].astype(np.float32))
        return torch.from_numpy(np.stack(rows)) if rows else torch.empty(0, 50)


class ArgmaxSampler:
    def pick(self, logits, params):
        assert len(params) == logits.shape[0]
        return logits.argmax(-1).tolist()


class Later:
    def __init__(self, tokens):
        self._tokens = tokens

    def tokens(self):
        return self._tokens


class OverlapRunner(FakeRunner):
    """The stand-in with picked tokens kept 'on the device': a pending entry takes its token from there."""

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.device_tokens, self.wanted = {}, []

    def step(self, entries):
        from runtime.engine.runner import StepEntry
        real = []
        for e in entries:
            if e.pending:
                assert list(e.tokens) == [0] and e.request in self.device_tokens
                real.append(StepEntry(e.request, [self.device_tokens[e.request]], e.want))
            else:
                real.append(e)
        self.wanted = [e.request for e in entries for _ in e.want]
        return super().step(real)

    def pick(self, sampler, logits, params):
        tokens = sampler.pick(logits, params)
        self.device_tokens.update(zip(self.wanted, tokens))
        return Later(tokens)

    def release(self, key):
        super().release(key)
        self.device_tokens.pop(key, None)


def make_engine(runner=None, **kw):
    return Engine(runner or FakeRunner(), sampler=ArgmaxSampler(), **kw)


def test_policies_produce_identical_tokens_and_release():
    # reference tests/test_engine.py:12-21
    outputs = []
    for policy in ("serial", "chunked", "decode_first"):
        e = make_engine(policy=policy, token_budget=3, prefill_chunk=2)
        for i, length in enumerate([1, 7, 3]):
            e.submit(Request(str(i), list(range(length)), 5))
        result = e.run()
        outputs.append([r.generated for r in result])
        assert all(r.status == "finished" and len(r.generated) == 5 for r in result)
        assert not e.reserved
        e.runner.cache.check()
        assert e.runner.cache.free_pages() == [20]
        assert all(t["processed_tokens"] <= 3 for t in e.trace)
    assert outputs[0] == outputs[1] == outputs[2]


def test_steps_carry_prompt_portions_beside_decode_tokens():
    e = make_engine(policy="decode_first", token_budget=6, prefill_chunk=4)
    e.submit(Request("short", [1, 2], 4))
    e.submit(Request("long", list(range(11)), 2))
    e.run()
    calls = e.runner.calls
    assert calls[0] == [("short", 2, [1]), ("long", 4, [])]            # last prompt token wanted, mid-prompt not
    assert calls[1] == [("short", 1, [0]), ("long", 4, [])]            # decode first, one token, beside a portion
    assert calls[2] == [("short", 1, [0]), ("long", 3, [2])]
    assert all(sum(n for _, n, _ in c) <= 6 for c in calls)


def test_cancel_waiting_active_zero_output_and_budget():
    # reference tests/test_engine.py:23-31
    e = make_engine(token_budget=1)
    e.submit(Request("a", [1, 2, 3], 3)); e.submit(Request("b", [1], 3))
    e.cancel("b"); e.tick(); e.cancel("a")
    e.submit(Request("c", [1], 0)); e.run()
    assert e.requests["a"].status == "cancelled" and e.requests["b"].status == "cancelled"
    assert e.requests["c"].generated == [] and e.requests["c"].status == "finished"
    assert all(t["processed_tokens"] <= 1 for t in e.trace)
    e.cancel("a")  # idempotent
    e.runner.cache.check()
    assert e.runner.cache.free_pages() == [20]


def test_reject_oversized_and_fairness():
    # reference tests/test_engine.py:33-39
    e = make_engine(token_budget=1, prefill_chunk=1)
    with pytest.raises(ValueError):
        e.submit(Request("bad", [1] * 100, 1))            # beyond the context limit
    with pytest.raises(ValueError):
        make_engine(FakeRunner(pages=2)).submit(Request("big", [1] * 9, 1))  # 3 pages can never fit in 2
    for i in range(3):
        e.submit(Request(str(i), [1] * 4, 2))
    for _ in range(3):
        e.tick()
    assert all(r.cursor > 0 for r in e.active)
    e.run()


def test_submit_checks():
    e = make_engine()
    e.submit(Request("a", [1], 1))
    for bad in (Request("a", [1], 1), Request("x", [], 1), Request("x", [1], -1), Request("x", [99], 1),
                Request("x", [1], 1, arrival_s=-1), Request("x", [1], 1, cursor=1)):
        with pytest.raises(ValueError):
            e.submit(bad)
    with pytest.raises(ValueError):
        make_engine(policy="fifo")
    with pytest.raises(ValueError):
        make_engine(token_budget=0)


def test_when_pages_run_out_requests_wait_and_none_fails():
    # 6 pages of 4 tokens.  Each request reserves ceil((8 + 4 - 1) / 4) = 3 pages,
    # so two run at a time and the third waits until one finishes; no step ever
    # fails for lack of pages and every request completes.
    runner = FakeRunner(pages=6)
    e = make_engine(runner, policy="chunked", token_budget=16, prefill_chunk=8)
    for i in range(3):
        e.submit(Request(str(i), [i + 1] * 8, 4))
    e.tick()
    assert [r.key for r in e.active] == ["0", "1"] and [r.key for r in e.waiting] == ["2"]
    assert sum(e.reserved.values()) == 6
    peak = 0
    while e.tick():
        peak = max(peak, runner.cache.groups[0].pool.used)
        assert sum(e.reserved.values()) <= 6
    assert peak <= 6 and all(r.status == "finished" and len(r.generated) == 4 for r in e.requests.values())
    assert runner.cache.free_pages() == [6]


def test_pages_are_promised_group_by_group():
    """Two cache groups: one keeps every key (plenty of pages), one a window of 8 (few pages).  A request is
    promised all its pages in the first and what a window and a portion can touch in the second, and the
    scarcer group decides how many run together."""
    runner = FakeRunner(pages=40, max_context=512)
    window = KVNeed(1, 8, window=8)
    runner.cache = CacheManager({0: KVNeed(1, 8), 1: window}, {KVNeed(1, 8): 40, window: 9}, 4, 8)
    e = make_engine(runner, token_budget=8, prefill_chunk=4)
    assert e.ledger.need(30) == [8, 4]               # ceil(30/4); (8 + 4 - 1)//4 + 2
    assert e.ledger.need(5) == [2, 2]                # a short request never holds more than its tokens
    for i in range(3):
        e.submit(Request(str(i), [1] * 27, 4))       # 30 cached tokens each
    e.tick()
    assert [r.key for r in e.active] == ["0", "1"] and [r.key for r in e.waiting] == ["2"]   # 3 x 4 > 9 window pages
    assert e.reserved == {"0": 12, "1": 12}
    peak = [0, 0]
    while e.tick():
        peak = [max(p, g.pool.used) for p, g in zip(peak, runner.cache.groups)]
        runner.cache.check()
    assert peak[0] <= 16 and peak[1] <= 8
    assert all(r.status == "finished" and len(r.generated) == 4 for r in e.requests.values())
    assert runner.cache.free_pages() == [40, 9] and not e.reserved
    with pytest.raises(ValueError, match="can never run"):
        e.submit(Request("huge", [1] * 200, 1))      # 50 pages in the group that keeps everything


def test_a_small_request_passes_a_large_one_that_does_not_fit_yet():
    runner = FakeRunner(pages=6)
    e = make_engine(runner, token_budget=8, prefill_chunk=8)
    e.submit(Request("running", [1] * 8, 5))   # 3 pages
    e.tick()
    e.submit(Request("large", [2] * 13, 4))    # 4 pages: does not fit beside 3
    e.submit(Request("small", [3] * 4, 2))     # 2 pages: fits
    e.tick()
    assert {r.key for r in e.active} == {"running", "small"} and [r.key for r in e.waiting] == ["large"]
    e.run()
    assert e.requests["large"].status == "finished"


def test_eos_finishes_and_is_kept():
    e = make_engine()
    e.submit(Request("probe", [5, 6], 6))
    e.run()
    tokens = e.requests["probe"].generated
    e2 = make_engine()
    e2.submit(Request("probe", [5, 6], 6, eos_token_id=tokens[2]))
    e2.run()
    first = tokens.index(tokens[2])
    assert e2.requests["probe"].generated == tokens[:first + 1]
    e3 = make_engine()
    e3.submit(Request("probe", [5, 6], 6, eos_token_id=[tokens[1], 49]))
    e3.run()
    assert e3.requests["probe"].generated == tokens[:tokens.index(tokens[1]) + 1]


def test_sampling_parameters_reach_the_sampler():
    seen = []

    class Spy(ArgmaxSampler):
        def pick(self, logits, params):
            seen.append(list(params)); return super().pick(logits, params)

    e = Engine(FakeRunner(), sampler=Spy(), token_budget=8, prefill_chunk=8)
    e.submit(Request("a", [1, 2], 3, temperature=0.8, seed=7))
    e.run()
    assert seen == [[(0.8, 7, 0)], [(0.8, 7, 1)], [(0.8, 7, 2)]]   # counter = tokens generated so far


def test_serial_runs_one_request_at_a_time():
    e = make_engine(policy="serial", token_budget=8, prefill_chunk=8)
    for i in range(3):
        e.submit(Request(str(i), [1, 2, 3], 2))
    e.run()
    assert all(len({k for k, _, _ in call}) == 1 for call in e.runner.calls)
    assert e.max_active == 1


@pytest.mark.parametrize("policy", ["serial", "chunked", "decode_first"])
def test_overlapped_ticks_give_the_same_tokens(policy):
    lengths, news = [1, 7, 3, 9, 2], [5, 1, 8, 3, 6]
    plain = make_engine(policy=policy, token_budget=4, prefill_chunk=3)
    for i, (length, new) in enumerate(zip(lengths, news)):
        plain.submit(Request(str(i), list(range(length)), new))
    want = [r.generated for r in plain.run()]
    e = make_engine(OverlapRunner(), policy=policy, token_budget=4, prefill_chunk=3, overlap=True)
    for i, (length, new) in enumerate(zip(lengths, news)):
        e.submit(Request(str(i), list(range(length)), new))
    result = e.run()
    assert [r.generated for r in result] == want
    assert all(r.status == "finished" for r in result) and not e.reserved and e.inflight is None
    e.runner.cache.check()
    assert e.runner.cache.free_pages() == [20]
    assert all(t["processed_tokens"] <= 4 for t in e.trace)
    # a request is never stepped past its last token: the count is known before the token is read
    fed = {}
    for call in e.runner.calls:
        for key, n, _ in call:
            fed[key] = fed.get(key, 0) + n
    assert fed == {str(i): length + new - 1 for i, (length, new) in enumerate(zip(lengths, news))}


def test_overlapped_ticks_end_on_eos_one_step_late_and_drop_the_extra_token():
    probe = make_engine()
    probe.submit(Request("probe", [5, 6], 8))
    probe.submit(Request("other", [7], 8))
    probe.run()
    tokens = probe.requests["probe"].generated
    e = make_engine(OverlapRunner(), overlap=True)
    e.submit(Request("probe", [5, 6], 8, eos_token_id=tokens[2]))
    e.submit(Request("other", [7], 8))
    e.run()
    stop = tokens.index(tokens[2])
    assert e.requests["probe"].generated == tokens[:stop + 1]
    assert e.requests["other"].generated == probe.requests["other"].generated
    assert not e.reserved and e.inflight is None
    e.runner.cache.check()
    assert e.runner.cache.free_pages() == [20]
    # the token after the end was decoded (the step was already launched) and thrown away
    fed = sum(n for call in e.runner.calls for key, n, _ in call if key == "probe")
    assert fed == 2 + stop + 1


def test_overlapped_ticks_cancel_while_a_step_is_in_flight():
    e = make_engine(OverlapRunner(), overlap=True)
    e.submit(Request("a", [1, 2, 3], 6))
    e.submit(Request("b", [4], 6))
    e.tick(); e.tick()
    e.cancel("a")
    e.run()
    assert e.requests["a"].status == "cancelled" and e.requests["b"].status == "finished"
    assert len(e.requests["b"].generated) == 6 and not e.reserved
    e.runner.cache.check()
    assert e.runner.cache.free_pages() == [20]


@pytest.mark.parametrize("seed", range(12))
def test_random_workloads_finish_and_give_everything_back(seed):
    """Random pools, limits, policies and windows; requests arrive while others run, some are cancelled, some are too
    long for the context or the pool: every accepted request ends finished or cancelled, the engine comes to rest,
    no page and no promise is left behind."""
    import random
    rng = random.Random(seed)
    pages, page_size = rng.randint(6, 30), rng.choice([2, 4, 8])
    max_requests, overlap = rng.randint(2, 8), rng.random() < 0.5
    window = rng.choice([None, None, 8, 12])
    runner = (OverlapRunner if overlap else FakeRunner)(pages=pages, page_size=page_size, max_requests=max_requests,
                                                        max_context=rng.choice([32, 64, 96]))
    if window is not None:   # a second group of layers that look back over a window: pages of their own
        runner.cache = CacheManager({0: KVNeed(1, 8), 1: KVNeed(1, 8, window)}, pages, page_size, max_requests)
    engine = make_engine(runner, max_active=rng.randint(1, 8), token_budget=rng.randint(2, 40), prefill_chunk=rng.randint(1, 16),
                         policy=rng.choice(["serial", "chunked", "decode_first"]), overlap=overlap)
    arriving = [(f"r{i}", [rng.randrange(50) for _ in range(rng.randint(1, 40))], rng.randint(1, 12), rng.choice([None, None, 7, (3, 9)]))
                for i in range(rng.randint(1, 12))]
    accepted, ticks = [], 0
    while arriving or engine.waiting or engine.active or engine.inflight:
        ticks += 1
        assert ticks < 5000, "the engine does not come to rest"
        if arriving and rng.random() < 0.4:
            key, prompt, new, eos = arriving.pop()
            try:
                engine.submit(Request(key, prompt, new, eos))
                accepted.append(key)
            except ValueError:
                pass          # refused at the door: longer than the context, or than the pool could ever hold
        if accepted and rng.random() < 0.05:
            engine.cancel(rng.choice(accepted))
        engine.tick()
    runner.cache.check()
    assert not runner.cache.lengths and not engine.ledger.promised
    for key in accepted:
        request = engine.requests[key]
        assert str(request.status) in ("finished", "cancelled")
        if str(request.status) == "finished":
            assert 1 <= len(request.generated) <= request.max_new_tokens
