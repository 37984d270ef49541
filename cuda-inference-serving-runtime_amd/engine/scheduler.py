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
import math
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Optional

from .runner import StepEntry

POLICIES = ("serial", "chunked", "decode_first")


@dataclass
class Request:
    key: str
    prompt: list
    max_new_tokens: int = 16
    eos_token_id: Optional[int] = None
    arrival_s: float = 0.0
    temperature: float = 0.0
    seed: int = 0
    generated: list = field(default_factory=list)
    cursor: int = 0
    launched: int = 0        # tokens picked for it so far, read by the host or not (overlapped ticks)
    status: str = "waiting"  # waiting, prefill, decode, draining (its last token is picked, not read), finished, cancelled
    submitted_at: float = 0.0
    first_token_at: Optional[float] = None
    token_times: list = field(default_factory=list)
    finished_at: Optional[float] = None


class Engine:
    def __init__(self, runner, max_active=8, token_budget=32, prefill_chunk=8, policy="chunked", sampler=None,
                 overlap=False):
        if min(max_active, token_budget, prefill_chunk) <= 0:
            raise ValueError("invalid scheduler limits")
        if policy not in POLICIES:
            raise ValueError(f"invalid policy {policy!r}; one of {POLICIES}")
        self.runner = runner
        self.max_active = 1 if policy == "serial" else min(max_active, runner.max_requests)
        self.token_budget, self.prefill_chunk, self.policy = token_budget, prefill_chunk, policy
        if sampler is None:
            from ..sampling import Sampler
            sampler = Sampler()
        self.sampler = sampler
        self.waiting, self.active, self.requests, self.reserved = deque(), [], {}, {}
        self.trace, self.start, self.rotation = [], time.perf_counter(), 0
        self.overlap, self.inflight = overlap, None

    # -- page accounting ----------------------------------------------------------
    def _pool_pages(self):
        return min(g.pool.n_pages for g in self.runner.cache.groups) if self.runner.cache.groups else 1 << 30

    def _pages_for(self, r):
        # the last generated token is never fed back, so it needs no cache entry
        return math.ceil((len(r.prompt) + max(0, r.max_new_tokens - 1)) / self.runner.page_size)

    # -- requests -------------------------------------------------------------------
    def submit(self, request):
        r = request
        if r.key in self.requests:
            raise ValueError("duplicate request ID")
        if not r.prompt or r.max_new_tokens < 0 or r.arrival_s < 0:
            raise ValueError("invalid request")
        if r.status != "waiting" or r.cursor or r.generated:
            raise ValueError("request already used")
        if any((not 0 <= t < self.runner.model.vocab_size) for t in r.prompt):
            raise ValueError("invalid prompt token")
        if len(r.prompt) + max(0, r.max_new_tokens - 1) > self.runner.max_context:
            raise ValueError("request exceeds context limit")
        if self._pages_for(r) > self._pool_pages():
            raise ValueError("request cannot fit in page pool")
        r.submitted_at = self.start + r.arrival_s
        self.requests[r.key] = r
        self.waiting.append(r)

    def _finish(self, r, status="finished"):
        if r.key in self.reserved:
            self.runner.release(r.key)
            del self.reserved[r.key]
            self.active.remove(r)
        r.status, r.finished_at = status, time.perf_counter()

    def cancel(self, key):
        r = self.requests[key]
        if r.status in ("finished", "cancelled"):
            return
        if r in self.waiting:
            self.waiting.remove(r)
        self._finish(r, "cancelled")

    def _admit(self):
        available = self._pool_pages() - sum(self.reserved.values())
        for r in list(self.waiting):  # scan all: a large request does not block smaller ones
            if len(self.active) >= self.max_active:
                break
            if time.perf_counter() < r.submitted_at:
                continue
            pages = self._pages_for(r)
            if pages > available:
                continue
            self.waiting.remove(r)
            if r.max_new_tokens == 0:
                self._finish(r)
                continue
            self.runner.create(r.key)
            self.reserved[r.key] = pages
            available -= pages
            r.status = "prefill"
            self.active.append(r)

    # -- one tick = one step --------------------------------------------------------
    def plan(self):
        """[(request, n_tokens)] for the next step under the budget; advances the rotation."""
        order = self.active[self.rotation:] + self.active[:self.rotation]
        self.rotation = (self.rotation + 1) % max(1, len(self.active))
        if self.policy == "decode_first":
            order.sort(key=lambda r: r.status != "decode")
        remaining, plan = self.token_budget, []
        for r in order:
            if remaining == 0:
                break
            if r.status == "draining":
                continue
            n = 1 if r.status == "decode" else min(self.prefill_chunk, len(r.prompt) - r.cursor, remaining)
            plan.append((r, n))
            remaining -= n
        return plan

    def tick(self):
        if self.overlap:
            return self._tick_overlapped()
        self._admit()
        if not self.active:
            return bool(self.waiting)
        now = time.perf_counter()
        plan = self.plan()
        entries, sampled = [], []
        for r, n in plan:
            if r.status == "decode":
                entries.append(StepEntry(r.key, [r.generated[-1]], [0]))
                sampled.append(r)
            else:
                last = r.cursor + n == len(r.prompt)
                entries.append(StepEntry(r.key, r.prompt[r.cursor:r.cursor + n], [n - 1] if last else []))
                if last:
                    sampled.append(r)
        logits = self.runner.step(entries)
        choices = self.sampler.pick(logits, [(r.temperature, r.seed, len(r.generated)) for r in sampled])
        completed = time.perf_counter()
        picked = dict(zip((r.key for r in sampled), choices))
        for r, n in plan:
            if r.status == "prefill":
                r.cursor += n
                if r.cursor < len(r.prompt):
                    continue
                r.status = "decode"
            token = int(picked[r.key])
            r.generated.append(token)
            r.token_times.append(completed)
            if r.first_token_at is None:
                r.first_token_at = completed
            if len(r.generated) >= r.max_new_tokens or self._is_eos(r, token):
                self._finish(r)
        cache = self.runner.cache
        self.trace.append({"elapsed_s": time.perf_counter() - self.start, "step_s": time.perf_counter() - now,
                           "processed_tokens": sum(n for _, n in plan), "active": len(self.active),
                           "resident_pages": sum(g.pool.used for g in cache.groups)})
        return bool(self.active or self.waiting)

    def _tick_overlapped(self):
        self._admit()
        if not self.active and self.inflight is None:
            return bool(self.waiting)
        now = time.perf_counter()
        plan = self.plan()
        entries, sampled = [], []
        for r, n in plan:
            if r.status == "decode":
                if r.launched > len(r.generated):     # its last token is still only on the device
                    entries.append(StepEntry(r.key, [0], [0], pending=True))
                else:
                    entries.append(StepEntry(r.key, [r.generated[-1]], [0]))
                sampled.append(r)
            else:
                last = r.cursor + n == len(r.prompt)
                entries.append(StepEntry(r.key, r.prompt[r.cursor:r.cursor + n], [n - 1] if last else []))
                if last:
                    sampled.append(r)
        launched = None
        if entries:
            logits = self.runner.step(entries)
            if sampled:
                picked = self.runner.pick(self.sampler, logits, [(r.temperature, r.seed, r.launched) for r in sampled])
                launched = (picked, sampled)
            for r, n in plan:
                if r.status == "prefill":
                    r.cursor += n
                    if r.cursor < len(r.prompt):
                        continue
                    r.status = "decode"
                r.launched += 1
                if r.launched >= r.max_new_tokens:
                    r.status = "draining"     # nothing more to decode; it ends when this token is read
        previous, self.inflight = self.inflight, launched
        if previous is not None:
            picked, requests = previous
            tokens = picked.tokens()
            completed = time.perf_counter()
            for r, token in zip(requests, tokens):
                if r.status in ("finished", "cancelled"):
                    continue                  # ended by an earlier token, or cancelled: this one is dropped
                r.generated.append(int(token))
                r.token_times.append(completed)
                if r.first_token_at is None:
                    r.first_token_at = completed
                if len(r.generated) >= r.max_new_tokens or self._is_eos(r, token):
                    self._finish(r)
        cache = self.runner.cache
        self.trace.append({"elapsed_s": time.perf_counter() - self.start, "step_s": time.perf_counter() - now,
                           "processed_tokens": sum(n for _, n in plan), "active": len(self.active),
                           "resident_pages": sum(g.pool.used for g in cache.groups)})
        return bool(self.active or self.waiting or self.inflight)

    @staticmethod
    def _is_eos(r, token):
        eos = r.eos_token_id
        return eos is not None and (token in eos if isinstance(eos, (list, tuple, set, frozenset)) else token == eos)

    def run(self):
        while self.tick():
            if not self.active and self.waiting:
                delay = min(r.submitted_at for r in self.waiting) - time.perf_counter()
                if delay > 0:
                    time.sleep(min(delay, 0.01))
        return list(self.requests.values())

    # -- conveniences ---------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder, dtype="bfloat16", pages=128, page_size=16, execution="eager", device="cuda:0", **limits):
        """An engine for the model in `folder` (config.json + safetensors).  pages None (or 0): as many as fit
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
            # (the attention kernels address a site's keys with 32-bit byte offsets: fewer than 2^31 elements)
            widest = max(need.kv_heads * need.head_dim for need in model.cache_needs().values() if need is not None)
            addressable = min(addressable, (2 ** 31 - 1) // (widest * page_size))
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
