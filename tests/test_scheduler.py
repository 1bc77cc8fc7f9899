"""The scheduler's decisions, driven without a GPU: a stand-in for the step function reserves and commits pages
as the real one does and hands out made-up tokens."""
import random

import pytest

from vt_transformer_amd.cache import CacheManager, GroupSpec
from vt_transformer_amd.engine.scheduler import (FINISHED, RUNNING, WAITING, Request, Scheduled, Scheduler,
                                                  SchedulerConfig)
from vt_transformer_amd.sampling import SamplingParams

EOS = 7


class FakeEngine:
    """Scheduler + cache manager + a step that only does the bookkeeping of the real step function."""

    def __init__(self, num_pages=64, page_size=4, windows=(0,), token=lambda req: 1, group_pages=None, **cfg):
        self.cfg = SchedulerConfig(num_pages=num_pages, page_size=page_size, **cfg)
        group_pages = group_pages or [num_pages] * len(windows)
        self.cache = CacheManager([GroupSpec(i, w, n) for i, (w, n) in enumerate(zip(windows, group_pages))], page_size,
                                  self.cfg.max_running_reqs, self.cfg.max_seq_len)
        self.sched = Scheduler(self.cfg, self.cache, [EOS])
        self.token = token
        self.plans = []

    def add(self, uid, n_prompt, **sp):
        r = Request(uid, list(range(10, 10 + n_prompt)), SamplingParams(**sp))
        self.sched.add_request(r)
        return r

    def step(self):
        plan = self.sched.schedule()
        self.plans.append([(s.request.uid, s.start, s.n_tokens, s.sample) for s in plan])
        if plan:
            items = [(s.request.uid, s.start + s.n_tokens) for s in plan]
            assert self.cache.reserve(items), "the scheduler chose a step that the cache cannot hold"
            for uid, n in items:
                self.cache.commit(uid, n)
        sampled = {s.request.uid: self.token(s.request) for s in plan if s.sample}
        out = self.sched.update(plan, sampled)
        self.cache.check()
        return out

    def run(self, limit=10000):
        results = []
        for _ in range(limit):
            if not self.sched.has_work():
                break
            results.extend(self.step())
        assert not self.sched.has_work(), "the scheduler did not finish"
        return results


def test_three_decode_steps_give_three_results_none_finished():
    """vt-transformer/test/vt_backend_test.cpp:313-333."""
    e = FakeEngine()
    r = e.add("a", 5, max_tokens=10)
    first = e.step()                       # the prompt: its last logits give the first token
    assert [(x.uid, x.finished) for x in first] == [("a", False)]
    for _ in range(3):
        res = e.step()
        assert len(res) == 1 and res[0].uid == "a" and not res[0].finished
    # request bookkeeping of vt_request.hpp:12-33: the newest output token is not in the cache yet
    assert len(r.output) == 4 and r.computed == r.total_len - 1 and r.decoding
    assert e.plans[0] == [("a", 0, 5, True)] and e.plans[1] == [("a", 5, 1, True)]


def test_finish_on_end_token_or_output_limit():
    """vt_scheduler.cpp:431-437."""
    e = FakeEngine(token=lambda r: EOS if len(r.output) == 2 else 1)
    a = e.add("a", 3, max_tokens=10)
    b = e.add("b", 3, max_tokens=10, ignore_eos=True)
    c = e.add("c", 3, max_tokens=2)
    res = e.run()
    assert (a.finish_reason, len(a.output)) == ("eos", 3)
    assert (b.finish_reason, len(b.output)) == ("max_tokens", 10)
    assert (c.finish_reason, len(c.output)) == ("max_tokens", 2)
    assert sum(1 for r in res if r.finished) == 3
    assert e.cache.held_pages() == [0] and e.cache.slots.available == e.cfg.max_running_reqs


def test_context_length_stops_a_request():
    e = FakeEngine(max_seq_len=12)
    a = e.add("a", 8, max_tokens=100)
    e.run()
    assert a.finish_reason == "max_seq_len" and a.total_len == 12


def test_abort_frees_and_gives_no_further_results():
    """vt_backend_test.cpp:338-360."""
    e = FakeEngine()
    e.add("a", 6, max_tokens=50)
    e.add("b", 6, max_tokens=50)
    e.step(); e.step()
    assert e.sched.abort_request("a")
    assert e.cache.held_pages()[0] == sum(1 for p in e.cache.get("b").tables[0] if p >= 0)   # only b holds pages
    for _ in range(3):
        assert all(r.uid == "b" for r in e.step())
    assert not e.sched.abort_request("zzz")
    e.add("c", 3)
    assert e.sched.abort_request("c")            # still waiting: just leaves the line
    assert e.sched.abort_request("b")
    assert not e.sched.has_work() and e.cache.held_pages() == [0]


def test_prompts_are_cut_under_the_token_budget_and_decoding_goes_first():
    e = FakeEngine(num_pages=256, max_extend_tokens=10, chunk_size=6)
    e.add("a", 4, max_tokens=20)
    e.step()                                        # a: whole prompt
    e.add("b", 20, max_tokens=20)
    e.step()
    # a decodes (1 token) and b gets a portion of at most chunk_size within what is left of the budget
    assert e.plans[1] == [("a", 4, 1, True), ("b", 0, 6, False)]
    e.add("c", 9, max_tokens=20)
    e.step()
    # budget 10: a 1, b 6 (older), c the 3 that are left
    assert e.plans[2] == [("a", 5, 1, True), ("b", 6, 6, False), ("c", 0, 3, False)]
    e.step()
    assert e.plans[3] == [("a", 6, 1, True), ("b", 12, 6, False), ("c", 3, 3, False)]
    e.step()
    # b's last portion is short and ends at its newest token: it samples
    assert e.plans[4] == [("a", 7, 1, True), ("b", 18, 2, True), ("c", 6, 3, True)]
    assert all(sum(n for _, _, n, _ in p) <= 10 for p in e.plans)


def test_running_requests_are_bounded_by_slots():
    e = FakeEngine(max_running_reqs=2)
    for i in range(5):
        e.add(i, 3, max_tokens=3)
    e.step()
    assert len(e.sched.running) == 2 and len(e.sched.waiting) == 3
    e.run()
    assert all(e.sched.counters[k] >= 0 for k in e.sched.counters)


def test_when_pages_run_out_the_youngest_is_preempted_and_recomputed():
    # 3 pages of 4: two prompts of 4 tokens take one page each; both then need a second page
    e = FakeEngine(num_pages=3, page_size=4)
    a = e.add("a", 4, max_tokens=6)
    b = e.add("b", 4, max_tokens=6)
    e.step()
    assert len(e.sched.running) == 2
    e.step()                                        # both try to decode: a gets the last page, b must go
    assert b.state == WAITING and b.preemptions == 1 and b.computed == 0 and len(b.output) == 1
    assert e.sched.waiting[0] is b                  # at the head of the line
    assert e.cache.held_pages() == [2]
    e.run()
    assert (a.finish_reason, b.finish_reason) == ("max_tokens", "max_tokens")
    assert len(a.output) == 6 and len(b.output) == 6
    assert a.preemptions == 0
    # b was recomputed from its prompt and what it had produced: one portion of 5 tokens that samples
    assert any(p == [("b", 0, 5, True)] for p in e.plans)
    assert e.cache.held_pages() == [0]


def test_a_request_that_can_never_fit_is_refused_not_waited_for():
    e = FakeEngine(num_pages=2, page_size=4, max_seq_len=100)       # the pool holds 8 tokens
    big = e.add("big", 9)
    ok = e.add("ok", 3, max_tokens=2)
    res = e.run()
    assert big.state == FINISHED and big.finish_reason == "too_long"
    assert [r for r in res if r.uid == "big"][0].finished and [r for r in res if r.uid == "big"][0].next_token is None
    assert ok.finish_reason == "max_tokens"
    e2 = FakeEngine(max_seq_len=8)
    long = e2.add("long", 9)
    e2.run()
    assert long.finish_reason == "too_long"


def test_a_lone_request_that_outgrows_the_pool_ends_with_an_error():
    e = FakeEngine(num_pages=2, page_size=4)
    a = e.add("a", 6, max_tokens=50)
    e.run()
    assert a.finish_reason == "out_of_pages" and a.total_len == 9    # 8 tokens in the cache, the 9th had no page
    assert e.cache.held_pages() == [0]


def _alone(n_prompt, max_tokens, token, **cfg):
    e = FakeEngine(token=token, **cfg)
    r = e.add("x", n_prompt, max_tokens=max_tokens)
    e.run()
    return r.output


@pytest.mark.parametrize("shape", [dict(num_pages=4, page_size=4, chunk_size=4, max_extend_tokens=8, n=12),
                                   dict(num_pages=64, page_size=16, chunk_size=256, max_extend_tokens=8192, n=600)])
def test_two_prompts_that_each_fit_alone_but_not_together_both_finish(shape):
    """Two prompts cut into portions must not end up holding every page half-way through with neither able to go
    on (the reference simply does not run a batch that gets no pages and tries again for ever,
    vt-transformer/core/vt_scheduler.cpp:112-117, 365-371)."""
    shape = dict(shape)
    n = shape.pop("n")
    token = lambda r: 1 + (len(r.output) * 7 + len(r.prompt)) % 5
    e = FakeEngine(token=token, **shape)
    a = e.add("a", n, max_tokens=3)
    b = e.add("b", n, max_tokens=3)
    e.run(limit=200)
    assert (a.finish_reason, b.finish_reason) == ("max_tokens", "max_tokens")
    alone = _alone(n, 3, token, **shape)
    assert a.output == alone and b.output == alone
    assert all(p for p in e.plans), "a step with running requests planned nothing"
    assert e.cache.held_pages() == [0]


def test_requests_inside_their_prompts_that_hold_every_page_do_not_stall():
    """The state that admission now avoids, made by hand: two requests half-way through their prompts hold all four
    pages.  The youngest gives way, the oldest goes on, and both finish."""
    e = FakeEngine(num_pages=4, page_size=4, chunk_size=4, max_extend_tokens=8)
    a = e.add("a", 12, max_tokens=2)
    b = e.add("b", 12, max_tokens=2)
    for r in (a, b):
        e.sched.waiting.remove(r)
        e.cache.admit(r.uid)
        assert e.cache.reserve([(r.uid, 8)])
        e.cache.commit(r.uid, 8)
        r.state, r.computed = RUNNING, 8
        e.sched.running.append(r)
    assert e.cache.available_pages() == [0]
    plan = e.sched.schedule()
    assert [(s.request.uid, s.start, s.n_tokens) for s in plan] == [("a", 8, 4)]
    assert b.state == WAITING and b.preemptions == 1 and e.sched.waiting[0] is b
    e.sched.update([], {})
    e.run(limit=100)
    assert (a.finish_reason, b.finish_reason) == ("max_tokens", "max_tokens")
    assert len(a.output) == 2 and len(b.output) == 2


def test_a_lone_request_inside_its_prompt_that_cannot_go_on_ends_with_an_error():
    e = FakeEngine(num_pages=2, page_size=4, chunk_size=4, max_seq_len=100)
    a = e.add("a", 8, max_tokens=2)
    e.sched.waiting.remove(a)
    e.cache.admit(a.uid)
    # another holder (not the scheduler's) has taken a page: the request's last portion can never get one
    e.cache.admit("other")
    assert e.cache.reserve([("other", 4), (a.uid, 4)])
    e.cache.commit(a.uid, 4)
    a.state, a.computed = RUNNING, 4
    e.sched.running.append(a)
    assert e.sched.schedule() == []
    assert a.finish_reason == "out_of_pages" and not e.sched.running
    assert [r.reason for r in e.sched.update([], {})] == ["out_of_pages"]


def test_a_portion_is_cut_to_the_pages_that_are_left():
    e = FakeEngine(num_pages=6, page_size=4, chunk_size=6, max_extend_tokens=64)
    a = e.add("a", 3, max_tokens=30)
    e.step()                                     # a holds one page
    b = e.add("b", 14, max_tokens=2)             # needs 4 pages: fits beside a's one and one page of head-room
    e.step()
    assert e.plans[1] == [("a", 3, 1, True), ("b", 0, 6, False)]
    e.cache.admit("other")                       # somebody else takes two of the three free pages
    assert e.cache.reserve([("other", 8)])
    e.step()                                     # a: its 5th token takes the last page; b: the 2 slots of its page
    assert e.plans[2] == [("a", 4, 1, True), ("b", 6, 2, False)]
    e.step()                                     # no page for b: it waits while a decodes
    assert e.plans[3] == [("a", 5, 1, True)]
    e.cache.release("other")
    e.run()
    assert b.finish_reason == "max_tokens" and b.preemptions == 0


@pytest.mark.parametrize("seed", range(50))
def test_random_load_always_drains(seed):
    rng = random.Random(seed)
    tight = seed % 2 == 1       # chunk sizes below the prompt lengths, pools below the sum of the prompts
    page_size = rng.choice([1, 2, 4, 16])
    if tight:
        max_len = 64
        num_pages = -(-rng.randint(40, 70) // page_size) + 1
        chunk, budget = rng.randint(2, 8), rng.randint(4, 16)
        prompt = lambda: rng.randint(12, 38)
    else:
        max_len = 64
        num_pages = rng.randint(8, 30)
        chunk, budget = rng.randint(2, 16), rng.randint(4, 40)
        prompt = lambda: rng.randint(1, 40)
    e = FakeEngine(num_pages=num_pages, page_size=page_size, windows=(0, rng.choice([0, 6])),
                   max_running_reqs=rng.randint(1, 6), max_extend_tokens=budget, chunk_size=chunk,
                   max_seq_len=max_len, token=lambda r: rng.choice([1, 2, 3, EOS]))
    reqs = []
    for step in range(300):
        if rng.random() < 0.3:
            reqs.append(e.add(len(reqs), prompt(), max_tokens=rng.randint(1, 12),
                              ignore_eos=rng.random() < 0.3))
        if rng.random() < 0.05 and reqs:
            e.sched.abort_request(rng.choice(reqs).uid)
        e.step()
        assert e.plans[-1] or not e.sched.running, "requests are running and the step planned nothing"
    e.run()
    assert all(r.state == FINISHED for r in reqs)
    assert all(r.finish_reason in ("eos", "max_tokens", "max_seq_len", "abort", "too_long", "out_of_pages") for r in reqs)
    assert e.cache.held_pages() == [0, 0]
    for r in reqs:
        if r.finish_reason == "max_tokens":
            assert len(r.output) == r.params.max_tokens


class AheadEngine(FakeEngine):
    """FakeEngine whose step starts the step after it before it has the tokens, the way Engine.step does: the
    stand-in for the step function reserves and commits the plan's pages when the plan is launched."""

    def __init__(self, **kw):
        super().__init__(**kw)
        self.ahead = None
        self.launched_ahead = 0

    def _launch(self, plan):
        items = [(s.request.uid, s.start + s.n_tokens) for s in plan]
        assert self.cache.reserve(items), "a step was launched that the cache cannot hold"
        for uid, n in items:
            self.cache.commit(uid, n)
        return plan

    def step(self):
        cur, self.ahead = self.ahead, None
        if cur is None:
            plan = self.sched.schedule()
            self.plans.append([(s.request.uid, s.start, s.n_tokens, s.sample) for s in plan])
            if not plan:
                return self.sched.update(plan, {})
            cur = self._launch(plan)
        nxt = self.sched.plan_ahead(cur)
        if nxt is not None:
            self.ahead = self._launch(nxt)
            self.launched_ahead += 1
            self.plans.append([(s.request.uid, s.start, s.n_tokens, s.sample) for s in nxt])
        sampled = {s.request.uid: self.token(s.request) for s in cur if s.sample}
        out = self.sched.update(cur, sampled)
        if self.ahead is not None and not any(s.request.state == RUNNING for s in self.ahead):
            self.ahead = None
        self.cache.check()
        return out

    def run(self, limit=10000):
        results = []
        for _ in range(limit):
            if not (self.sched.has_work() or self.ahead is not None):
                break
            results.extend(self.step())
        assert not self.sched.has_work(), "the scheduler did not finish"
        return results


def test_the_step_ahead_is_checked_against_the_length_after_it():
    """A lone request crosses a page's edge while it decodes ahead of the host and no page is free: the step ahead
    is not planned (the step in flight has committed start + 1 tokens, the step ahead needs room for start + 2),
    and the plain way then ends the request for want of pages instead of raising."""
    e = AheadEngine(num_pages=2, page_size=4, max_running_reqs=2, max_seq_len=64)
    a = e.add("a", 7, max_tokens=20)
    e.step()                                    # the prompt (a portion: nothing is started ahead of it)
    assert e.launched_ahead == 0 and e.cache.get("a").length == 7
    e.step()                                    # token 8 fills the second page; token 9 would need a third one
    assert e.launched_ahead == 0 and e.ahead is None and e.cache.get("a").length == 8
    plan = [Scheduled(a, 7, 1, True)]           # the step that has just run, as Engine.step hands it on
    assert e.sched._fits([(a, 8)]) and not e.sched._fits([(a, 9)])
    assert e.sched.plan_ahead(plan) is None
    e.run()
    assert a.finish_reason == "out_of_pages" and a.total_len == 9 and e.cache.held_pages() == [0]


def test_decoding_ahead_gives_way_to_preemption_when_pages_run_out():
    # 3 pages of 4: a and b decode ahead until both stand at a page's edge with one page free; nothing is launched
    # ahead then, schedule() preempts b, and both finish with the tokens they get alone
    token = lambda r: 1 + (len(r.output) * 5 + len(r.prompt)) % 4
    e = AheadEngine(num_pages=3, page_size=4, token=token)
    a = e.add("a", 2, max_tokens=8)
    b = e.add("b", 2, max_tokens=8)
    e.run(limit=200)
    assert e.launched_ahead > 0 and b.preemptions >= 1 and a.preemptions == 0
    assert (a.finish_reason, b.finish_reason) == ("max_tokens", "max_tokens")
    assert a.output == _alone(2, 8, token) and b.output == a.output
    assert e.cache.held_pages() == [0]


@pytest.mark.parametrize("seed", range(30))
def test_random_load_decoding_ahead_always_drains(seed):
    rng = random.Random(1000 + seed)
    page_size = rng.choice([1, 2, 4, 16])
    e = AheadEngine(num_pages=-(-rng.randint(20, 70) // page_size) + 1, page_size=page_size,
                    max_running_reqs=rng.randint(1, 5), max_extend_tokens=rng.randint(4, 24),
                    chunk_size=rng.randint(2, 12), max_seq_len=64, token=lambda r: rng.choice([1, 2, 3, EOS]))
    reqs = []
    for step in range(200):
        if rng.random() < 0.15:
            reqs.append(e.add(len(reqs), rng.randint(1, 30), max_tokens=rng.randint(1, 20), ignore_eos=rng.random() < 0.5))
        if rng.random() < 0.03 and reqs:
            e.sched.abort_request(rng.choice(reqs).uid)
        e.step()
    e.run()
    assert all(r.state == FINISHED for r in reqs) and e.cache.held_pages() == [0]
    for r in reqs:
        if r.finish_reason == "max_tokens":
            assert len(r.output) == r.params.max_tokens


def test_random_loads_do_decode_ahead():
    launched = 0
    for seed in range(30):
        rng = random.Random(1000 + seed)
        e = AheadEngine(num_pages=40, page_size=4, token=lambda r: rng.choice([1, 2, 3]))
        for i in range(3):
            e.add(i, rng.randint(1, 20), max_tokens=rng.randint(3, 20))
        e.run()
        launched += e.launched_ahead
    assert launched > 100


def test_a_windowed_group_with_few_pages_does_not_bound_a_requests_length():
    """Layers with a window hold a window and a portion of a request, so their pool may be far smaller than a
    prompt: 12 pages of 4 tokens beside prompts of 40 (ten pages in the group that keeps every key).  Nobody is
    refused as too long, both slots are used, everybody finishes."""
    e = FakeEngine(page_size=4, windows=(0, 6), group_pages=[64, 12], max_running_reqs=2, chunk_size=8,
                   max_extend_tokens=16, max_seq_len=128)
    assert e.cache.max_held_pages(1, 8) == 5
    reqs = [e.add(i, 40, max_tokens=6) for i in range(3)]
    e.step()
    assert len(e.sched.running) == 2
    e.run(limit=300)
    assert [r.finish_reason for r in reqs] == ["max_tokens"] * 3 and all(len(r.output) == 6 for r in reqs)
    assert e.cache.held_pages() == [0, 0]
    # with fewer pages than a window and a portion take, the windowed group bounds the length like any other
    small = FakeEngine(page_size=4, windows=(0, 6), group_pages=[64, 4], chunk_size=8, max_seq_len=128)
    r = small.add("x", 40)
    small.run()
    assert r.finish_reason == "too_long"
