"""The scheduler's decisions (no GPU): a fake engine with the real cache manager stands in for the model."""
import random

import pytest
import torch

from emulated_kernels import EmulatedKernels
from easy_gpt.cpp_amd import kernels
from easy_gpt.cpp_amd.cache import CacheManager
from easy_gpt.cpp_amd.engine import StepEntry
from easy_gpt.cpp_amd.engine.scheduler import Request, Scheduler, SchedulerConfig
from easy_gpt.cpp_amd.parts import CacheNeed
from easy_gpt.cpp_amd.sampling import SamplingParams

VOCAB = 50
GREEDY = SamplingParams(greedy=True)


@pytest.fixture(autouse=True)
def emulated_backend():
    kernels.use_backend(EmulatedKernels())
    yield
    kernels.use_backend(None)


class FakeEngine:
    """Keeps the cache manager's books like the real engine; the 'model' predicts
    next = (7 * sum of all tokens so far + position) mod VOCAB, so outputs depend on the whole history."""

    def __init__(self, num_pages, page_size=4, max_requests=8, max_position=1000, needs=None):
        self.cache = CacheManager(needs or [CacheNeed.keys_and_values(1, 8)], page_size, num_pages, max_requests)
        self.max_position = max_position
        self.device = "cpu"
        self.sums = {}
        self.log = []           # per step: list of (id, n_tokens, wants)

    def add_request(self, rid):
        self.sums[rid] = 0
        return self.cache.admit(rid)

    def finish(self, rid):
        self.cache.release(self.cache.requests[rid])
        del self.sums[rid]

    def step(self, entries):
        rows = []
        self.log.append([(e.request_id, len(e.tokens), list(e.want)) for e in entries])
        for e in entries:
            rc = self.cache.requests[e.request_id]
            self.cache.reserve(rc, len(e.tokens))
        for e in entries:
            rc = self.cache.requests[e.request_id]
            for i, t in enumerate(e.tokens):
                self.sums[e.request_id] += t
                if i in e.want:
                    row = torch.zeros(VOCAB)
                    row[(7 * self.sums[e.request_id] + rc.num_tokens + i) % VOCAB] = 5.0
                    rows.append(row)
            self.cache.commit(rc, len(e.tokens))
        self.cache.check()
        return torch.stack(rows) if rows else None


class FakeAheadEngine(FakeEngine):
    """The same with the entry that takes a decode step's token ids from what the sampler left "on the device"."""

    supports_lookahead = True

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.ahead_steps = 0

    def step_decode_ahead(self, request_ids, tokens):
        assert tokens.dtype == torch.int32 and tokens.shape == (len(request_ids),)
        self.ahead_steps += 1
        return self.step([StepEntry(rid, [int(t)], [0]) for rid, t in zip(request_ids, tokens.tolist())])


def expected_output(prompt, n_new, eos=-1):
    toks, out = list(prompt), []
    for _ in range(n_new):
        nxt = (7 * sum(toks) + len(toks) - 1) % VOCAB
        out.append(nxt)
        toks.append(nxt)
        if nxt == eos:
            break
    return out


def test_budget_portions_and_decode_first():
    eng = FakeEngine(num_pages=200)
    s = Scheduler(eng, SchedulerConfig(max_active=4, max_admit_per_step=4, max_tokens_per_step=10, prefill_chunk=6))
    a = s.add(Request("a", list(range(1, 15)), GREEDY, max_new_tokens=3))
    b = s.add(Request("b", list(range(2, 6)), GREEDY, max_new_tokens=3))
    s.run()
    assert eng.log[0] == [("a", 6, []), ("b", 4, [3])]             # chunk 6, then b gets the rest of the budget
    # b decodes first; a goes on with its prompt: its share of 6, and the 2 more that the budget still holds
    assert eng.log[1] == [("b", 1, [0]), ("a", 8, [7])]
    assert eng.log[2] == [("a", 1, [0]), ("b", 1, [0])]
    assert all(sum(n for _, n, _ in step) <= 10 for step in eng.log)
    assert a.output == expected_output(a.prompt, 3) and b.output == expected_output(b.prompt, 3)
    assert a.finish_reason == b.finish_reason == "length"
    assert eng.cache.free_pages() == [200] and not eng.cache.requests
    assert s.stats.generated == 6 and s.stats.prompt_tokens == 18 and s.stats.finished == 2


def test_what_is_left_of_the_budget_goes_to_the_portions():
    # a prompt alone in its steps has the whole budget, not only its share
    eng = FakeEngine(num_pages=200)
    s = Scheduler(eng, SchedulerConfig(max_active=4, max_admit_per_step=4, max_tokens_per_step=10, prefill_chunk=4))
    a = s.add(Request("a", list(range(1, 24)), GREEDY, max_new_tokens=1))
    s.run()
    assert [step[0][1:] for step in eng.log] == [(10, []), (10, []), (3, [2])]
    # three prompts: each its share while the budget lasts, the rest to the first that has tokens left
    eng = FakeEngine(num_pages=200)
    s = Scheduler(eng, SchedulerConfig(max_active=4, max_admit_per_step=4, max_tokens_per_step=16, prefill_chunk=4))
    rs = [s.add(Request(i, list(range(1, n + 1)), GREEDY, max_new_tokens=1)) for i, n in enumerate((3, 20, 20))]
    s.step()
    assert eng.log[0] == [(0, 3, [2]), (1, 9, []), (2, 4, [])]      # 3 + 4 + 4 leave 5, which request 1 takes
    assert all(sum(n for _, n, _ in step) <= 16 for step in eng.log)
    s.run()
    assert all(r.output == expected_output(r.prompt, 1) for r in rs)
    # no pages for more than the share: the portion stays as it is (4 pages of 4 tokens: b's 7 tokens take two, which
    # leaves c's 11 one page beyond the one of its share)
    eng = FakeEngine(num_pages=4)
    s = Scheduler(eng, SchedulerConfig(max_active=2, max_admit_per_step=2, max_tokens_per_step=64, prefill_chunk=4))
    b = s.add(Request("b", list(range(1, 8)), GREEDY, max_new_tokens=1))
    c = s.add(Request("c", list(range(1, 12)), GREEDY, max_new_tokens=1))
    s.step()
    assert eng.log[0] == [("b", 7, [6]), ("c", 4, [])]
    s.run()
    assert b.output == expected_output(b.prompt, 1) and c.output == expected_output(c.prompt, 1)
    assert eng.cache.free_pages() == [4] and not eng.cache.requests


def test_admission_is_first_in_first_out_and_bounded():
    eng = FakeEngine(num_pages=200)
    s = Scheduler(eng, SchedulerConfig(max_active=2, max_admit_per_step=1, max_tokens_per_step=64, prefill_chunk=64))
    rs = [s.add(Request(i, [i + 1] * 5, GREEDY, max_new_tokens=2)) for i in range(4)]
    s.step()
    assert [r.status for r in rs] == ["running", "waiting", "waiting", "waiting"]     # one admission per step
    s.step()
    assert [r.status for r in rs] == ["finished", "running", "waiting", "waiting"]
    s.run()
    admit_order = []
    for step in eng.log:
        for rid, _, _ in step:
            if rid not in admit_order:
                admit_order.append(rid)
    assert admit_order == [0, 1, 2, 3]
    assert max(len(step) for step in eng.log) <= 2                                     # max_active
    for r in rs:
        assert r.output == expected_output(r.prompt, 2)


def test_a_first_portion_is_cut_to_the_free_pages_when_every_layer_has_a_window():
    # a pool of 4 pages of 4 tokens, far smaller than the chunk of 512: every group gives pages back as its window of
    # 6 tokens passes them, so the prompt gets through in portions that the free pages hold; nothing stalls or fails
    eng = FakeEngine(num_pages=4, needs=[CacheNeed.keys_and_values(1, 8, window=6)])
    s = Scheduler(eng, SchedulerConfig(max_active=2, prefill_chunk=512))
    r = s.add(Request("r", list(range(1, 41)), GREEDY, max_new_tokens=5))
    r2 = s.add(Request("r2", list(range(3, 30)), GREEDY, max_new_tokens=4))
    s.run()
    assert r.status == r2.status == "finished"
    assert r.output == expected_output(r.prompt, 5) and r2.output == expected_output(r2.prompt, 4)
    assert eng.log[0] == [("r", 16, [])]                   # the first portion: what four free pages hold
    assert eng.cache.free_pages() == [4]
    # a pool that cannot even hold what one window touches: the request fails alone, with a reason
    eng = FakeEngine(num_pages=2, needs=[CacheNeed.keys_and_values(1, 8, window=6)])
    s = Scheduler(eng, SchedulerConfig())
    r = s.add(Request("r", list(range(1, 41)), GREEDY, max_new_tokens=5))
    s.run()
    assert r.status == "failed" and "even alone" in r.finish_reason


def test_decoding_runs_one_step_ahead_of_the_host():
    # three requests decode side by side: from the step in which the last prompt ends, every step is launched before
    # the tokens of the step before it are seen; ends that can be foreseen are not run past, an end token costs one
    # token that is thrown away, and the outputs are what they are without looking ahead
    prompts = {"a": [3, 4], "b": [5, 6, 7, 8, 9], "c": [1]}
    out_b = expected_output(prompts["b"], 12)
    eos = out_b[6]                                     # b ends on its seventh token
    plain_outputs = {}
    for engine_class in (FakeEngine, FakeAheadEngine):
        eng = engine_class(num_pages=100)
        s = Scheduler(eng, SchedulerConfig(max_active=4), eos_token_id=eos)
        reqs = {k: s.add(Request(k, p, GREEDY, max_new_tokens=n, ignore_eos=(k != "b")))
                for (k, p), n in zip(prompts.items(), (9, 12, 15))}
        s.run()
        outs = {k: r.output for k, r in reqs.items()}
        if engine_class is FakeEngine:
            plain_outputs = outs
            plain_stats = s.stats
            assert s.stats.steps_ahead == 0
            continue
        assert outs == plain_outputs
        # the token that was computed past b's end is not counted as decoded
        assert (s.stats.decode_tokens, s.stats.prompt_tokens) == (plain_stats.decode_tokens, plain_stats.prompt_tokens)
        assert outs["b"] == expected_output(prompts["b"], 12, eos=eos) and reqs["b"].finish_reason == "eos"
        assert reqs["a"].finish_reason == reqs["c"].finish_reason == "length"
        assert s.stats.steps_ahead == eng.ahead_steps > 8 and s.stats.discarded == 1
        # tokens fed per request: the prompt and every output but the last; b one more (the step that was in flight
        # when its end token was seen); a and c end on their limits, which is never run past
        fed = {k: sum(n for step in eng.log for rid, n, _ in step if rid == k) for k in prompts}
        assert fed == {"a": 2 + 8, "b": 5 + len(outs["b"]), "c": 1 + 14}
        assert s.stats.generated == sum(len(o) for o in outs.values())
        assert eng.cache.free_pages() == [100] and not eng.cache.requests and not s.has_work()


def test_looking_ahead_stops_where_pages_or_the_batch_change():
    # so few pages that requests are preempted, and requests that join later: steps are launched ahead only while the
    # batch stays what it is and its next pages are free; the tokens are the same as without looking ahead
    rng = random.Random(5)
    prompts = [[rng.randrange(VOCAB) for _ in range(rng.randint(1, 30))] for _ in range(7)]
    outs = []
    for engine_class in (FakeEngine, FakeAheadEngine):
        eng = engine_class(num_pages=24)
        s = Scheduler(eng, SchedulerConfig(max_active=3, max_admit_per_step=2, max_tokens_per_step=16, prefill_chunk=8))
        reqs = [s.add(Request(i, p, GREEDY, max_new_tokens=10 + i)) for i, p in enumerate(prompts)]
        s.run()
        outs.append([r.output for r in reqs])
        assert all(r.output == expected_output(r.prompt, 10 + i) for i, r in enumerate(reqs))
        assert eng.cache.free_pages() == [24]
    assert outs[0] == outs[1]


def test_looking_ahead_while_requests_wait_for_a_slot():
    # more requests than slots: those that wait cannot be admitted before a running one ends, so decoding still runs
    # ahead of the host; with a slot free (and somebody waiting for it) it does not
    prompts = [[3 + i, 4, 5] for i in range(5)]
    outs = []
    for engine_class in (FakeEngine, FakeAheadEngine):
        eng = engine_class(num_pages=100)
        s = Scheduler(eng, SchedulerConfig(max_active=2, max_admit_per_step=2))
        reqs = [s.add(Request(i, p, GREEDY, max_new_tokens=12)) for i, p in enumerate(prompts)]
        ahead_while_waiting = 0
        while s.has_work():
            before = s.stats.steps_ahead
            s.step()
            if s.waiting and s.stats.steps_ahead > before:
                assert len(s.running) == 2
                ahead_while_waiting += 1
        outs.append([r.output for r in reqs])
        assert all(r.output == expected_output(r.prompt, 12) for r in reqs)
        if engine_class is FakeAheadEngine:
            assert ahead_while_waiting >= 12 and s.stats.discarded == 0
            assert eng.cache.free_pages() == [100]
    assert outs[0] == outs[1]


def test_eos_is_kept_and_stops():
    eng = FakeEngine(num_pages=50)
    prompt = [3, 4]
    out = expected_output(prompt, 10)
    eos = out[2]
    s = Scheduler(eng, SchedulerConfig(), eos_token_id=eos)
    r = s.add(Request("r", prompt, GREEDY, max_new_tokens=10))
    r2 = s.add(Request("r2", prompt, GREEDY, max_new_tokens=10, ignore_eos=True))
    s.run()
    assert r.output == expected_output(prompt, 10, eos=eos) and r.output[-1] == eos and r.finish_reason == "eos"
    assert r2.output == out and r2.finish_reason == "length"


def test_max_position_stops():
    eng = FakeEngine(num_pages=50, max_position=8)
    s = Scheduler(eng, SchedulerConfig())
    r = s.add(Request("r", [1, 2, 3, 4, 5], GREEDY, max_new_tokens=50))
    long = s.add(Request("long", [1] * 9, GREEDY, max_new_tokens=5))
    s.run()
    assert r.finish_reason == "max_position" and len(r.prompt) + len(r.output) == 9
    assert eng.cache.free_pages() == [50]
    assert long.status == "failed" and "max_position" in long.finish_reason


def test_waiting_when_pages_are_short_then_admitted():
    eng = FakeEngine(num_pages=5, page_size=4)
    s = Scheduler(eng, SchedulerConfig(max_tokens_per_step=64, prefill_chunk=64))
    a = s.add(Request("a", [1] * 11, GREEDY, max_new_tokens=2))       # 3 pages
    b = s.add(Request("b", [2] * 10, GREEDY, max_new_tokens=2))       # 3 pages: does not fit beside a
    s.step()
    assert a.status == "running" and b.status == "waiting"
    s.run()
    assert a.output == expected_output(a.prompt, 2) and b.output == expected_output(b.prompt, 2)
    assert s.stats.preemptions == 0


def test_preemption_of_the_newest_when_a_decode_needs_a_page():
    eng = FakeEngine(num_pages=4, page_size=4)
    s = Scheduler(eng, SchedulerConfig(max_tokens_per_step=64, prefill_chunk=64))
    a = s.add(Request("a", [1] * 7, GREEDY, max_new_tokens=6))        # grows to 12 stored tokens: 3 pages
    b = s.add(Request("b", [2] * 7, GREEDY, max_new_tokens=6))
    s.run()
    assert s.stats.preemptions >= 1 and b.preemptions >= 1 and a.preemptions == 0
    assert a.output == expected_output(a.prompt, 6)                   # recomputation gives the same tokens
    assert b.output == expected_output(b.prompt, 6)
    assert eng.cache.free_pages() == [4]
    # the preempted request was recomputed with its generated tokens as part of the prompt
    sizes_b = [n for step in eng.log for rid, n, _ in step if rid == "b"]
    assert any(n > 7 for n in sizes_b)


def test_request_that_cannot_fit_alone_fails_and_the_rest_goes_on():
    eng = FakeEngine(num_pages=3, page_size=4)
    s = Scheduler(eng, SchedulerConfig())
    big = s.add(Request("big", [1] * 20, GREEDY, max_new_tokens=2))
    ok = s.add(Request("ok", [2] * 5, GREEDY, max_new_tokens=3))
    s.run()
    assert big.status == "failed" and "cache" in big.finish_reason
    assert ok.status == "finished" and ok.output == expected_output(ok.prompt, 3)
    assert s.stats.failed == 1 and eng.cache.free_pages() == [3]


def test_prompt_portion_is_cut_to_the_free_pages():
    eng = FakeEngine(num_pages=6, page_size=4)
    s = Scheduler(eng, SchedulerConfig(max_tokens_per_step=64, prefill_chunk=64))
    a = s.add(Request("a", [1] * 12, GREEDY, max_new_tokens=1))       # 3 pages
    s.step()
    b = s.add(Request("b", [2] * 20, GREEDY, max_new_tokens=1))       # 5 pages, only 3 free while a lives
    eng.cache.requests  # a finished in its first step (max_new_tokens=1), so everything is free again
    s.run()
    assert b.output == expected_output(b.prompt, 1)


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("ahead", [False, True])
def test_random_workloads_finish_with_the_right_tokens(seed, ahead):
    rng = random.Random(seed)
    ps = rng.choice([2, 4, 8])
    # room for the longest request alone (30 + 12 tokens) and a little more, so that pages run short often
    eng = (FakeAheadEngine if ahead else FakeEngine)(num_pages=-(-44 // ps) + rng.randint(0, 10), page_size=ps, max_requests=5)
    cfg = SchedulerConfig(max_active=rng.randint(1, 5), max_admit_per_step=rng.randint(1, 3),
                          max_tokens_per_step=rng.randint(4, 40), prefill_chunk=rng.randint(2, 16))
    s = Scheduler(eng, cfg)
    reqs = []
    for i in range(12):
        prompt = [rng.randrange(VOCAB) for _ in range(rng.randint(1, 30))]
        reqs.append(s.add(Request(i, prompt, GREEDY, max_new_tokens=rng.randint(1, 12))))
    s.run()
    for r in reqs:
        assert r.status == "finished", (r.status, r.finish_reason)
        assert r.output == expected_output(r.prompt, r.max_new_tokens)
    assert all(sum(n for _, n, _ in step) <= cfg.max_tokens_per_step for step in eng.log)
    assert all(len(step) <= cfg.max_active for step in eng.log)
    assert eng.cache.free_pages() == [eng.cache.pools[0].num_pages]


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_the_one_pass_decision_for_decoding_requests_is_the_general_one(seed):
    # while every running request decodes and nobody waits, the step is decided in one pass: whenever that pass
    # decides at all, it names the same entries as the general rules; when pages run short it leaves the decision
    # (and the preemption) to them
    rng = random.Random(seed)
    eng = FakeEngine(num_pages=rng.choice([14, 30, 200]), page_size=4, max_requests=6)
    s = Scheduler(eng, SchedulerConfig(max_active=6, max_admit_per_step=6, max_tokens_per_step=64, prefill_chunk=16))
    for i in range(6):
        s.add(Request(i, [rng.randrange(1, VOCAB) for _ in range(rng.randint(1, 9))], GREEDY, max_new_tokens=rng.randint(2, 12)))
    decided = 0
    for _ in range(400):
        if not s.has_work():
            break
        fast = s._plan_decode_only()
        if fast is not None:
            decided += 1
            s._plan_decode_only = lambda: None                    # the general rules alone
            try:
                general = s.plan()
            finally:
                del s._plan_decode_only
            assert [(e.request.request_id, e.start, e.count, e.samples) for e in fast] == \
                   [(e.request.request_id, e.start, e.count, e.samples) for e in general]
        s.step()
    assert not s.has_work() and decided > 0
    for r in s.done:
        if r.status == "finished":
            assert r.output == expected_output(r.prompt, len(r.output))


def test_temperature_sampling_does_not_depend_on_neighbours():
    outs = []
    for others in (0, 3):
        eng = FakeEngine(num_pages=100)
        s = Scheduler(eng, SchedulerConfig())
        # flat logits would make the draw matter: use a fake with two equal peaks instead of one
        params = SamplingParams(temperature=1.0, top_p=1.0, top_k=0, seed=7)
        r = s.add(Request("r", [5, 6, 7], params, max_new_tokens=8))
        for i in range(others):
            s.add(Request(f"o{i}", [i + 1] * 4, params, max_new_tokens=8))
        s.run()
        outs.append(r.output)
    assert outs[0] == outs[1]
