"""Continuous batching above the step function.

Same requests, limits and policies as the reference's Engine
(runtime/engine.py:13-122): admission by worst-case page reservation, a token
budget per tick, a bounded prompt portion per request per tick, at most one
decoded token per request per tick, rotation for fairness, `decode_first`
putting decoding requests ahead, `serial` running one request at a time.
Unlike the reference, whose tick runs one token per request per microstep, a
tick here is ONE step whose entries are prompt portions of several tokens
beside single decode tokens.

When pages run out: they cannot for an admitted request, because admission
reserves the pages of its whole prompt and output (runtime/engine.py:65-76).
A request that does not fit beside the running ones waits (later, smaller ones
may pass it); one that could never fit is refused at submit
(runtime/engine.py:46-47).  Nothing is preempted.

With `overlap`, a tick launches its step before the tokens of the step before
are read: picked tokens stay on the device, the next step takes them from
there, and the host prepares step N+1 while the GPU runs step N.  The tokens
are the same; a request that ends on an end-of-sequence token is found out one
step late, and the token it decoded meanwhile is dropped.
"""
import enum
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Optional

from .runner import StepEntry

POLICIES = ("serial", "chunked", "decode_first")


class Phase(str, enum.Enum):
    """Where a request stands.  A member compares equal to its name in lower case ("finished")."""
    WAITING = "waiting"        # submitted, holds nothing
    PREFILL = "prefill"        # admitted, its prompt is being cached
    DECODE = "decode"          # one token a step
    DRAINING = "draining"      # overlapped ticks: its last token is picked on the device and not read yet
    FINISHED = "finished"
    CANCELLED = "cancelled"

    def __str__(self):
        return self.value

    @property
    def over(self):
        return self in (Phase.FINISHED, Phase.CANCELLED)


@dataclass
class Request:
    """A request and its progress (the fields of the reference's Request, runtime/engine.py:13-26, and the
    sampling parameters)."""
    key: str
    prompt: list
    max_new_tokens: int = 16
    eos_token_id: Optional[int] = None     # one id, or a collection of them
    arrival_s: float = 0.0
    temperature: float = 0.0
    seed: int = 0
    generated: list = field(default_factory=list)
    cursor: int = 0          # prompt tokens cached so far
    launched: int = 0        # tokens picked for it so far, read by the host or not (overlapped ticks)
    status: Phase = Phase.WAITING
    submitted_at: float = 0.0
    first_token_at: Optional[float] = None
    token_times: list = field(default_factory=list)
    finished_at: Optional[float] = None

    @property
    def cached_tokens(self):
        """Tokens that will ever sit in the cache: the last generated token is never fed back."""
        return len(self.prompt) + max(0, self.max_new_tokens - 1)

    def ends_with(self, token):
        eos = self.eos_token_id
        if eos is None:
            return False
        return token in eos if isinstance(eos, (list, tuple, set, frozenset)) else token == eos

    def take(self, token, when):
        """Record a generated token; True if it is the request's last."""
        self.generated.append(int(token))
        self.token_times.append(when)
        if self.first_token_at is None:
            self.first_token_at = when
        return len(self.generated) >= self.max_new_tokens or self.ends_with(token)


class PageLedger:
    """Pages promised to admitted requests, group by group of the cache.

    A request is admitted only if every group can promise it the most pages it will ever hold there (all its
    tokens in a group that keeps every key; a window and a portion in a group that keeps a window), so a step of
    admitted requests cannot run out of pages.  The numbers come from the cache manager."""

    def __init__(self, cache, portion):
        self.cache, self.portion, self.promised = cache, portion, {}

    def need(self, tokens):
        return self.cache.most_pages_held(tokens, self.portion)

    def ever_fits(self, need):
        return all(n <= cap for n, cap in zip(need, self.cache.capacity()))

    def fits_now(self, need):
        taken = [sum(p[g] for p in self.promised.values()) for g in range(len(need))]
        return all(n <= cap - t for n, cap, t in zip(need, self.cache.capacity(), taken))

    def promise(self, key, need):
        self.promised[key] = list(need)

    def withdraw(self, key):
        return self.promised.pop(key, None) is not None


class Engine:
    def __init__(self, runner, max_active=8, token_budget=32, prefill_chunk=8, policy="chunked", sampler=None,
                 overlap=False):
        for name, value in (("max_active", max_active), ("token_budget", token_budget), ("prefill_chunk", prefill_chunk)):
            if value <= 0:
                raise ValueError(f"{name} must be positive, not {value}")
        if policy not in POLICIES:
            raise ValueError(f"policy {policy!r} is none of {POLICIES}")
        self.runner = runner
        self.max_active = 1 if policy == "serial" else min(max_active, runner.max_requests)
        self.token_budget, self.prefill_chunk, self.policy = token_budget, prefill_chunk, policy
        if sampler is None:
            from ..sampling import Sampler
            sampler = Sampler()
        self.sampler = sampler
        self.ledger = PageLedger(runner.cache, min(prefill_chunk, token_budget))
        self.waiting, self.active, self.requests = deque(), [], {}
        self.trace, self.start, self.rotation = [], time.perf_counter(), 0
        self.overlap, self.inflight = overlap, None

    @property
    def reserved(self):
        """{request key: pages promised to it, summed over the cache groups}."""
        return {key: sum(need) for key, need in self.ledger.promised.items()}

    # -- requests come and go -------------------------------------------------------------
    def _refusal(self, r):
        """Why `r` cannot be taken, or None (what the reference checks at submit, runtime/engine.py:38-50)."""
        if r.key in self.requests:
            return f"the key {r.key!r} is already in use"
        if r.status is not Phase.WAITING or r.cursor or r.launched or r.generated:
            return f"request {r.key!r} has run before: submit a fresh Request"
        if len(r.prompt) == 0:
            return f"request {r.key!r} has an empty prompt"
        if r.max_new_tokens < 0 or r.arrival_s < 0:
            return f"request {r.key!r}: max_new_tokens and arrival_s cannot be negative"
        vocab = self.runner.model.vocab_size
        stray = next((t for t in r.prompt if not 0 <= t < vocab), None)
        if stray is not None:
            return f"request {r.key!r}: token {stray} is outside the vocabulary of {vocab}"
        if r.cached_tokens > self.runner.max_context:
            return f"request {r.key!r} would cache {r.cached_tokens} tokens, the context limit is {self.runner.max_context}"
        need = self.ledger.need(r.cached_tokens)
        if not self.ledger.ever_fits(need):
            return f"request {r.key!r} needs {need} pages, the pools hold {self.runner.cache.capacity()}: it can never run"
        return None

    def submit(self, request):
        reason = self._refusal(request)
        if reason is not None:
            raise ValueError(reason)
        request.submitted_at = self.start + request.arrival_s
        self.requests[request.key] = request
        self.waiting.append(request)

    def _close(self, r, phase=Phase.FINISHED):
        """End a request: whatever it holds (cache pages, state slot, promised pages) goes back."""
        if self.ledger.withdraw(r.key):
            self.runner.release(r.key)
            self.active.remove(r)
        r.status, r.finished_at = phase, time.perf_counter()

    def cancel(self, key):
        r = self.requests[key]
        if r.status.over:
            return
        if r.status is Phase.WAITING:
            self.waiting.remove(r)
        self._close(r, Phase.CANCELLED)

    def _admit(self):
        """Take waiting requests in while there is room: the whole queue is looked at, so a request that does
        not fit now does not hold up a later one that does (runtime/engine.py:65-76)."""
        now = time.perf_counter()
        for r in tuple(self.waiting):
            if len(self.active) >= self.max_active:
                return
            if r.submitted_at > now:
                continue                      # not arrived yet
            need = self.ledger.need(r.cached_tokens)
            if not self.ledger.fits_now(need):
                continue
            self.waiting.remove(r)
            if r.max_new_tokens == 0:
                self._close(r)                # nothing to generate: it never touches the cache
                continue
            self.runner.create(r.key)
            self.ledger.promise(r.key, need)
            r.status = Phase.PREFILL
            self.active.append(r)

    # -- one tick = one step --------------------------------------------------------
    def plan(self):
        """[(request, n_tokens)] for the next step under the budget; advances the rotation.  The request that is
        served first moves on by one place every tick, so that a budget smaller than the batch starves nobody
        (the reference's rotating priority, runtime/engine.py:82-85); `decode_first` then lets every decoding
        request, in that order, stand before every prompt."""
        live = [r for r in self.active if r.status is not Phase.DRAINING]
        first = self.rotation % len(self.active) if self.active else 0
        turn = {id(r): (i - first) % len(self.active) for i, r in enumerate(self.active)}
        self.rotation = first + 1
        if self.policy == "decode_first":
            live.sort(key=lambda r: (r.status is not Phase.DECODE, turn[id(r)]))
        else:
            live.sort(key=lambda r: turn[id(r)])
        plan, left = [], self.token_budget
        for r in live:
            if left <= 0:
                break
            n = 1 if r.status is Phase.DECODE else min(self.prefill_chunk, len(r.prompt) - r.cursor, left)
            plan.append((r, n))
            left -= n
        return plan

    def _entries(self, plan):
        """The step's entries, and the requests whose logits are wanted (a token is picked for them)."""
        entries, picking = [], []
        for r, n in plan:
            if r.status is Phase.DECODE:
                on_device = r.launched > len(r.generated)     # its last token is picked but not read yet
                entries.append(StepEntry(r.key, [0] if on_device else [r.generated[-1]], [0], pending=on_device))
                picking.append(r)
            else:
                portion = r.prompt[r.cursor:r.cursor + n]
                last = r.cursor + n == len(r.prompt)
                entries.append(StepEntry(r.key, portion, [n - 1] if last else []))
                if last:
                    picking.append(r)
        return entries, picking

    @staticmethod
    def _fed(r, n):
        """Account for n tokens of `r` having been stepped; True if the step picks a token for it."""
        if r.status is Phase.PREFILL:
            r.cursor += n
            if r.cursor < len(r.prompt):
                return False
            r.status = Phase.DECODE
        return True

    def _record(self, began, plan):
        now = time.perf_counter()
        self.trace.append({"elapsed_s": now - self.start, "step_s": now - began,
                           "processed_tokens": sum(n for _, n in plan), "active": len(self.active),
                           "resident_pages": sum(g.pool.used for g in self.runner.cache.groups)})

    def tick(self):
        """Admit, run one step, hand out its tokens.  False when nothing is left to do."""
        self._admit()
        if not self.active and self.inflight is None:
            return bool(self.waiting)
        began = time.perf_counter()
        plan = self.plan()
        entries, picking = self._entries(plan)
        if self.overlap:
            self._step_ahead(plan, entries, picking)
        else:
            logits = self.runner.step(entries)
            tokens = dict(zip((r.key for r in picking),
                              self.sampler.pick(logits, [(r.temperature, r.seed, len(r.generated)) for r in picking])))
            when = time.perf_counter()
            for r, n in plan:
                if self._fed(r, n) and r.take(tokens[r.key], when):
                    self._close(r)
        self._record(began, plan)
        return bool(self.active or self.waiting or self.inflight)

    def _step_ahead(self, plan, entries, picking):
        """Overlapped ticks: launch this step, then read the tokens of the step before.  What is known without
        the token is settled at launch (the prompt cursor, the count of tokens); what needs the token (an
        end-of-sequence) one step late."""
        launched = None
        if entries:
            logits = self.runner.step(entries)
            if picking:
                picked = self.runner.pick(self.sampler, logits, [(r.temperature, r.seed, r.launched) for r in picking])
                launched = (picked, picking)
            for r, n in plan:
                if self._fed(r, n):
                    r.launched += 1
                    if r.launched >= r.max_new_tokens:
                        r.status = Phase.DRAINING     # nothing more to decode; it ends when this token is read
        previous, self.inflight = self.inflight, launched
        if previous is None:
            return
        picked, requests = previous
        tokens = picked.tokens()
        when = time.perf_counter()
        for r, token in zip(requests, tokens):
            if r.status.over:
                continue                  # ended by an earlier token, or cancelled: this one is dropped
            if r.take(token, when):
                self._close(r)

    def run(self):
        """Tick until every request is over.  While nothing is live and the next arrival lies in the future the
        loop sleeps, never longer than 10 ms at a time (the reference's idle wait, runtime/engine.py:117-122)."""
        busy = True
        while busy:
            busy = self.tick()
            if busy and not self.active and self.waiting:
                until_next = min(r.submitted_at for r in self.waiting) - time.perf_counter()
                time.sleep(max(0.0, min(until_next, 0.01)))
        return [self.requests[key] for key in self.requests]

    # -- conveniences ---------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder, dtype="bfloat16", pages=128, page_size=16, execution="graph", device="cuda:0", **limits):
        """An engine for the model in `folder` (config.json + safetensors).  Steps run as captured programs unless
        execution="eager" (kernels launched one by one).  pages None (or 0): as many as fit
        into four fifths of the GPU memory that is free once the weights are loaded, at most what the
        requests can address."""
        import torch
        from ..cache import pages_that_fit
        from .loading import load_model
        from .runner import ModelRunner
        model = load_model(folder, dtype=dtype, device=device)
        max_requests = max(8, limits.get("max_active", 8))
        if not pages:
            free, _ = torch.cuda.mem_get_info(torch.device(device))
            addressable = max_requests * -(-model.max_positions // page_size)
            # (the attention kernels address a site's keys with 32-bit byte offsets: fewer than 2^31 elements;
            # a model whose mixers keep no keys has nothing to size)
            widths = [need.kv_heads * need.head_dim for need in model.cache_needs().values() if need is not None]
            if widths:
                by_offsets = (2 ** 31 - 1) // (max(widths) * page_size)
                if by_offsets < addressable:
                    import sys
                    print(f"[runtime] the pool is limited to {by_offsets} pages a layer by the kernels' 32-bit offsets "
                          f"(the requests could address {addressable})", file=sys.stderr)
                    addressable = by_offsets
            pages = pages_that_fit(model.cache_needs(), page_size, 2 if dtype == "bfloat16" else 4, free, most=addressable)
        runner = ModelRunner(model, n_pages=pages, page_size=page_size, max_requests=max_requests, device=device,
                             execution=execution)
        return cls(runner, **limits)

    @classmethod
    def from_preset(cls, name, seed=0, folder=None, **kwargs):
        """An engine for a named configuration with seeded random weights."""
        import tempfile
        from .loading import write_random_model
        folder = folder or tempfile.mkdtemp(prefix=f"runtime-{name}-")
        write_random_model(folder, name, seed, dtype="bfloat16")
        return cls.from_folder(folder, **kwargs)

    def generate(self, prompts, max_new_tokens=16, temperature=0.0, seed=0, eos_token_id=None):
        """Generate for a list of prompts (lists of token ids); returns the lists of new tokens."""
        base = len(self.requests)
        keys = [f"generate-{base + i}" for i in range(len(prompts))]
        for i, (key, prompt) in enumerate(zip(keys, prompts)):
            self.submit(Request(key, list(prompt), max_new_tokens, eos_token_id, temperature=temperature, seed=seed + i))
        self.run()
        return [self.requests[key].generated for key in keys]
