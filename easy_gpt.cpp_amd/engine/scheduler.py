"""The scheduler: admits requests, cuts prompts into portions under a token budget, decodes,
finishes and frees.

The reference's ContinuousBatchServer alternates a prefill round (whole left-padded prompts,
at most prefill_batch_size of them) with a decode round (one token for every active request),
on a FIFO queue and a stack of free slots (/root/reference/src/continuous_batch_server.cpp:71-86,
88-158,160-212,222-260,274-327).  Here both kinds of work share one step: every running request
that is decoding contributes its last token, and what is left of the step's token budget goes to
prompt portions in arrival order.

Decoding runs one step ahead of the host where it can: while a decode step is on the GPU, the next one (the same
requests, one token each) is launched behind it with its token ids taken on the device from what the sampler leaves
there, and only then does the host wait for the first step's tokens.  So the GPU goes from step to step without waiting
for the host's bookkeeping, and a request that ends on an end token has computed one token too many, which is thrown
away.  Ends that can be foreseen (the token limit, max_position_embeddings) are not run past.

When pages run out:
  * a request waiting for admission keeps waiting (first in, first out: nobody overtakes it);
  * a prompt portion is cut down to what fits, or skipped for this step;
  * a decoding request that cannot get its next page preempts the most recently admitted
    running request (possibly itself): its pages are freed and it goes back to the front of
    the queue with its prompt extended by what it has generated, to be recomputed later;
  * a request that could not fit even alone fails with an error, the others go on.
"""
from __future__ import annotations

import time
from collections import deque
from dataclasses import dataclass, field

from ..cache import NoFreeSlot
from ..sampling import Sampler, SamplingParams
from .engine import StepEntry


@dataclass
class SchedulerConfig:
    max_active: int = 16            # the reference's --serve-max-active
    max_admit_per_step: int = 4     # the reference's --serve-prefill-batch
    max_tokens_per_step: int = 2048
    prefill_chunk: int = 512        # a request's share of a step's budget; what is left of the budget goes to portions too

    def __post_init__(self):
        for name in ("max_active", "max_admit_per_step", "max_tokens_per_step", "prefill_chunk"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be greater than 0")


@dataclass
class Request:
    request_id: object
    prompt: list[int]
    params: SamplingParams = field(default_factory=SamplingParams)
    max_new_tokens: int = 100
    ignore_eos: bool = False
    # filled by the scheduler
    serial: int = -1
    output: list[int] = field(default_factory=list)
    computed: int = 0               # tokens of prompt + output whose keys and values are in the cache
    status: str = "waiting"         # waiting | running | finished | failed
    finish_reason: str = ""
    preemptions: int = 0
    t_submit: float = 0.0
    t_admit: float = 0.0
    t_finish: float = 0.0

    def all_tokens(self) -> list[int]:
        return self.prompt + self.output

    def tokens(self, start: int, count: int) -> list[int]:
        """all_tokens()[start : start + count] without building the whole list (a decoding request asks for one)."""
        n = len(self.prompt)
        if start >= n:
            return self.output[start - n : start - n + count]
        if start + count <= n:
            return self.prompt[start : start + count]
        return self.prompt[start:] + self.output[: start + count - n]

    def pending(self) -> int:
        """Tokens not yet in the cache: the rest of the prompt, or the one last sampled token."""
        return len(self.prompt) + len(self.output) - self.computed


@dataclass
class PlannedEntry:
    request: Request
    start: int          # index into request.all_tokens()
    count: int
    samples: bool       # True if this portion ends the pending tokens, so a token is sampled after it


@dataclass
class _Launched:
    """A step that is on the GPU: what was planned, and the tokens it will give."""

    entries: list
    tokens: object               # sampling.PendingTokens, or None if no entry of the step samples
    samplers: list
    t0: float


@dataclass
class Stats:
    steps: int = 0
    steps_ahead: int = 0        # decode steps launched before the tokens of the step before them were seen
    discarded: int = 0          # tokens computed for a request after its end token, and thrown away
    prompt_tokens: int = 0
    decode_tokens: int = 0
    generated: int = 0
    preemptions: int = 0
    finished: int = 0
    failed: int = 0
    step_seconds: float = 0.0
    pages_high_water: int = 0


class Scheduler:
    def __init__(self, engine, config: SchedulerConfig | None = None, eos_token_id: int = -1, sampler=None):
        """engine: an object with add_request, finish, step, cache (a CacheManager), max_position."""
        self.engine = engine
        self.cache = engine.cache
        self.config = config or SchedulerConfig()
        self.eos_token_id = eos_token_id
        self.sampler = sampler or Sampler(getattr(engine, "device", "cpu"))
        self.waiting: deque[Request] = deque()
        self.running: list[Request] = []          # in order of admission
        self.done: list[Request] = []
        self.stats = Stats()
        self._serial = 0
        self.lookahead = bool(getattr(engine, "supports_lookahead", False))
        self._ahead: _Launched | None = None      # the step after the one being waited for, already launched
        self._last_end = 0.0                      # when the last step's tokens were there

    # ------------------------------------------------------------------ submitting
    def add(self, request: Request) -> Request:
        if not request.prompt:
            raise ValueError("a request needs at least one prompt token")
        if request.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be greater than 0")
        request.serial = self._serial
        self._serial += 1
        request.t_submit = time.perf_counter()
        request.status = "waiting"
        self.waiting.append(request)
        return request

    def has_work(self) -> bool:
        return bool(self.waiting or self.running or self._ahead is not None)

    # ------------------------------------------------------------------ deciding
    def _fits_alone(self, r: Request) -> bool:
        total = min(len(r.prompt) + r.max_new_tokens, self.engine.max_position)
        # the last generated token is never stored, the one before it is
        need = self.cache.pages_for_tokens(max(len(r.prompt), total - 1))
        ps = self.cache.page_size
        for pool, g in zip(self.cache.pools, self.cache.groups):
            # a windowed group gives pages back as the window passes them: token by token it never holds more than
            # the pages that a window can touch
            most = need if g.window is None else min(need, -(-g.window // ps) + 1)
            if most > pool.num_pages:
                return False
        return True

    def _fail(self, r: Request, reason: str) -> None:
        if r.status == "running":
            self.engine.finish(r.request_id)
            self.running.remove(r)
        r.status, r.finish_reason, r.t_finish = "failed", reason, time.perf_counter()
        self.stats.failed += 1
        self.done.append(r)

    def _preempt(self, r: Request) -> None:
        """Free the request's pages and put it back at the front of the queue; its prompt for the
        recomputation is everything it holds (prompt and generated tokens)."""
        self.engine.finish(r.request_id)
        self.running.remove(r)
        r.computed = 0
        r.status = "waiting"
        r.preemptions += 1
        self.stats.preemptions += 1
        self.waiting.appendleft(r)

    def _plan_decode_only(self) -> list[PlannedEntry] | None:
        """The common step of a busy engine, decided in one pass: nobody waits, every running request decodes, and
        the pages that their next tokens start are free.  The same entries as the general rules give; None if any
        of this does not hold (the general rules then decide, and may preempt)."""
        running = self.running
        if self.waiting or not running or len(running) > self.config.max_tokens_per_step:
            return None
        cache = self.cache
        requests, ps = cache.requests, cache.page_size
        need = [0] * len(cache.pools)
        for r in running:
            if not r.output or len(r.prompt) + len(r.output) - r.computed != 1:
                return None
            rc = requests[r.request_id]
            want = (rc.num_tokens + ps) // ps                   # pages that hold num_tokens + 1 tokens
            for g, have in enumerate(rc.table_lens):
                if want > have:
                    need[g] += want - have
        for n, pool in zip(need, cache.pools):
            if n > pool.free_count:
                return None
        return [PlannedEntry(r, r.computed, 1, True) for r in running]

    def plan(self) -> list[PlannedEntry]:
        """Decide the next step.  May admit, preempt or fail requests; returns what to run."""
        cfg = self.config
        entries = self._plan_decode_only()
        if entries is not None:
            return entries
        while True:
            budget = cfg.max_tokens_per_step
            promised = [0] * len(self.cache.pools)
            entries: list[PlannedEntry] = []
            restart = False

            def take(r: Request, count: int) -> bool:
                need = self.cache.pages_needed(self.cache.requests[r.request_id], count)
                if any(n > pool.free_count - p for n, pool, p in zip(need, self.cache.pools, promised)):
                    return False
                for g, n in enumerate(need):
                    promised[g] += n
                return True

            # 1. decoding requests: one token each, they come first
            for r in list(self.running):
                if r.pending() != 1 or not r.output or budget < 1:
                    continue
                if take(r, 1):
                    entries.append(PlannedEntry(r, r.computed, 1, True))
                    budget -= 1
                    continue
                victim = self.running[-1]
                if victim is r and len(self.running) == 1:
                    self._fail(r, "the cache cannot hold this request even alone")
                else:
                    self._preempt(victim)
                restart = True
                break
            if restart:
                continue
            # 2. prompt portions of running requests, in order of admission
            planned = {id(e.request) for e in entries}
            for r in self.running:
                if (r.pending() == 1 and r.output) or budget < 1 or id(r) in planned:
                    continue
                count = min(r.pending(), cfg.prefill_chunk, budget)
                while count > 0 and not take(r, count):
                    # cut the portion down to what the free pages hold
                    rc = self.cache.requests[r.request_id]
                    room = min(
                        (have + pool.free_count - p) * self.cache.page_size - rc.num_tokens
                        for have, pool, p in zip(rc.table_lens, self.cache.pools, promised)
                    )
                    count = min(count - 1, max(room, 0))
                if count > 0:
                    entries.append(PlannedEntry(r, r.computed, count, count == r.pending()))
                    budget -= count
            # 3. admission, first in first out
            admitted = 0
            while (self.waiting and budget > 0 and len(self.running) < cfg.max_active
                   and admitted < cfg.max_admit_per_step):
                r = self.waiting[0]
                if len(r.prompt) + len(r.output) > self.engine.max_position:
                    self.waiting.popleft()
                    self._fail(r, "the prompt is longer than max_position_embeddings")
                    continue
                if not self._fits_alone(r):
                    self.waiting.popleft()
                    self._fail(r, "the cache cannot hold this request even alone")
                    continue
                count = min(r.pending(), cfg.prefill_chunk, budget)
                room = min((pool.free_count - p) * self.cache.page_size for pool, p in zip(self.cache.pools, promised))
                if count > room:
                    if self.running or room < 1:
                        break           # it waits for pages that the running requests will give back
                    count = room        # nobody runs, so nothing will be given back: its first portion is cut to the free pages
                try:
                    self.engine.add_request(r.request_id)
                except NoFreeSlot:
                    break
                self.waiting.popleft()
                r.status = "running"
                if not r.t_admit:
                    r.t_admit = time.perf_counter()
                self.running.append(r)
                admitted += 1
                ok = take(r, count)
                assert ok
                entries.append(PlannedEntry(r, 0, count, count == r.pending()))
                budget -= count
            # 4. what is left of the budget goes to the portions that were cut at `prefill_chunk`, in their order: a
            # long prompt that is alone in its step has the whole step (few tokens behind a long prefix use the GPU badly)
            for e in entries:
                left = e.request.pending() - e.count
                if budget < 1:
                    break
                if e.samples or left < 1:
                    continue
                rc = self.cache.requests[e.request.request_id]
                more = min(left, budget)
                have = self.cache.pages_needed(rc, e.count)
                need = [a - b for a, b in zip(self.cache.pages_needed(rc, e.count + more), have)]
                if any(n > pool.free_count - p for n, pool, p in zip(need, self.cache.pools, promised)):
                    continue                # (the pages are short: the portion stays as it is)
                for g, n in enumerate(need):
                    promised[g] += n
                e.count += more
                e.samples = e.count == e.request.pending()
                budget -= more
            if entries or not self.running:
                return entries
            # nothing can move although requests are running: free the newest one's pages
            if len(self.running) == 1:
                self._fail(self.running[0], "the cache cannot hold this request even alone")
            else:
                self._preempt(self.running[-1])

    # ------------------------------------------------------------------ running
    def _launch(self, entries: list[PlannedEntry]) -> _Launched:
        """Run a planned step on the engine and start sampling; nothing here waits for the GPU."""
        t0 = time.perf_counter()
        batch = []
        for e in entries:
            toks = e.request.tokens(e.start, e.count)
            batch.append(StepEntry(e.request.request_id, toks, [e.count - 1] if e.samples else []))
        logits = self.engine.step(batch)
        return self._launched(entries, logits, t0, 0)

    def _launched(self, entries, logits, t0, ahead: int) -> _Launched:
        samplers = [e for e in entries if e.samples]
        for e in entries:
            e.request.computed += e.count
            if e.count == 1 and (e.request.output or ahead) and e.samples and e.start >= len(e.request.prompt):
                self.stats.decode_tokens += 1
            else:
                self.stats.prompt_tokens += e.count
        tokens = None
        if samplers:
            tokens = self.sampler.sample_async(
                logits, [e.request.params for e in samplers], [e.request.serial for e in samplers],
                [len(e.request.output) + ahead for e in samplers],
            )
        return _Launched(entries, tokens, samplers, t0)

    def _launch_ahead(self, now: _Launched) -> _Launched | None:
        """The step after `now`, if it is certain to be `now`'s requests decoding one token each: nobody waits (or
        whoever waits cannot be admitted before a running request ends: every slot is taken),
        every running request is sampled in `now`, none of them ends with that token for a reason known before the
        token is (its limit of new tokens, max_position_embeddings), and the pages their next tokens need are free.
        Its token ids are `now`'s sampled tokens, taken on the device."""
        if not self.lookahead or now.tokens is None:
            return None
        if self.waiting and len(self.running) < self.config.max_active:
            return None
        entries = now.entries
        if len(now.samplers) != len(entries) or len(entries) != len(self.running):
            return None
        cache = self.cache
        requests, ps = cache.requests, cache.page_size
        need = [0] * len(cache.pools)
        limit = self.engine.max_position
        for e in entries:
            r = e.request
            n_out = len(r.output) + 1                     # with the token that `now` is sampling
            if n_out >= r.max_new_tokens or len(r.prompt) + n_out >= limit or r.computed != len(r.prompt) + n_out - 1:
                return None
            rc = requests[r.request_id]
            want = (rc.num_tokens + ps) // ps
            for g, have in enumerate(rc.table_lens):
                if want > have:
                    need[g] += want - have
        if any(n > pool.free_count for n, pool in zip(need, cache.pools)):
            return None
        t0 = time.perf_counter()
        logits = self.engine.step_decode_ahead([e.request.request_id for e in entries], now.tokens.device)
        nxt = [PlannedEntry(e.request, e.request.computed, 1, True) for e in entries]
        self.stats.steps_ahead += 1
        return self._launched(nxt, logits, t0, 1)

    def step(self) -> list[Request]:
        """One step: plan it and run it (or take the one that was launched ahead), launch the step after it if that
        can be known, then wait for this step's tokens and finish what is done.  Returns the requests that finished."""
        now, self._ahead = self._ahead, None
        if now is None:
            entries = self.plan()
            if not entries:
                return []
            now = self._launch(entries)
        self._ahead = self._launch_ahead(now)
        finished: list[Request] = []
        if now.samplers:
            tokens = now.tokens.result()
            for e, tok in zip(now.samplers, tokens):
                r = e.request
                if r.status != "running":
                    self.stats.discarded += 1           # launched ahead of the end token that finished the request
                    self.stats.decode_tokens -= 1       # (counted when it was launched)
                    continue
                r.output.append(int(tok))
                self.stats.generated += 1
                reason = ""
                if not r.ignore_eos and self.eos_token_id >= 0 and tok == self.eos_token_id:
                    reason = "eos"               # the end token stays in the output, as in the reference
                elif len(r.output) >= r.max_new_tokens:
                    reason = "length"
                elif len(r.prompt) + len(r.output) > self.engine.max_position:
                    reason = "max_position"
                if reason:
                    self.engine.finish(r.request_id)
                    self.running.remove(r)
                    r.status, r.finish_reason, r.t_finish = "finished", reason, time.perf_counter()
                    self.stats.finished += 1
                    self.done.append(r)
                    finished.append(r)
        self.stats.steps += 1
        # a step launched ahead starts while the step before it is still being waited for: its time counts from
        # that step's end, so that the steps' times add up to the time that passed
        t_end = time.perf_counter()
        self.stats.step_seconds += t_end - max(now.t0, self._last_end)
        self._last_end = t_end
        self.stats.pages_high_water = max(self.stats.pages_high_water, max(p.high_water for p in self.cache.pools))
        return finished

    def run(self, on_step=None) -> list[Request]:
        """Run until every submitted request has finished or failed."""
        while self.has_work():
            before = (len(self.done), self.stats.steps)
            self.step()
            if on_step is not None:
                on_step(self)
            if (len(self.done), self.stats.steps) == before and self.has_work():
                raise RuntimeError("the scheduler cannot make progress")
        return self.done
