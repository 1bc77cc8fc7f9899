"""Admission, portions of prompts under a token budget, decoding, finishing
and freeing; and what happens when pages run out.

After the reference's FullScheduler (vt-transformer/core/vt_scheduler.cpp):
requests wait in arrival order (pending_) and run until they finish
(running_) (vt_scheduler.hpp:132-141); a step's new tokens are bounded by
max_extend_tokens (vt_scheduler.hpp:37); a request finishes on the end token
or at its output limit (vt_scheduler.cpp:431-437); results are
(uid, next_token, finished) (vt_scheduler.hpp:94-103); abort frees at once
(vt_scheduler.cpp:47-88).  Request bookkeeping follows vt_request.hpp:12-33:
the newest output token has no keys and values yet, the next step writes them.

Where it differs: the reference runs either prompts or decoding in a step
(vt_scheduler.cpp:102-110, 305-311), never cuts a prompt (:277, 292-294), and
reserves the whole output budget at admission (:257-299); when a decode step
cannot get a page it simply does not run and is tried again for ever
(:112-117, 365-371).  Here every step carries all decoding requests plus
portions of prompts; a prompt is cut to the budget; and when a decoding
request cannot get a page the youngest running request is preempted: it
gives everything back, returns to the head of the waiting line and is later
recomputed from its prompt and the tokens it has produced.  The same happens
when requests inside their prompts hold every page among them and nothing
can move: a plan is never empty while requests are running.  A request is
admitted only if all it holds so far fits beside what the running requests
still need for their prompts.  A request that could never fit is finished
with an error instead of waiting for ever.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, Hashable, List, Optional, Sequence, Tuple

from ..cache.pages import CacheManager
from ..sampling.params import SamplingParams


@dataclass
class SchedulerConfig:
    """Names and defaults of the reference's SchedulerConfig (vt_scheduler.hpp:28-39) where it has them."""

    max_running_reqs: int = 128     # live requests at a time (= state slots)
    num_pages: int = 1024           # pages per group of layers
    max_seq_len: int = 4096         # prompt + output of one request
    page_size: int = 16             # tokens per page (the reference defaults to 1)
    max_extend_tokens: int = 8192   # new tokens per step, prompts and decoding together
    default_max_output: int = 1024  # output limit of a request that names none
    chunk_size: int = 2048          # longest portion of one prompt in a step
    kv_bytes: Optional[int] = None  # the cache's size in bytes, shared by the groups of layers; sets num_pages
                                    # (num_blocks = budget // bytes of a block, vt-transformer/models/qwen3-0.6b/init.vt:109-113)


WAITING, RUNNING, FINISHED = "waiting", "running", "finished"


@dataclass
class Request:
    uid: Hashable
    prompt: List[int]
    params: SamplingParams
    seed: int = 0
    output: List[int] = field(default_factory=list)
    state: str = WAITING
    computed: int = 0            # tokens whose keys and values are in the cache
    arrival: int = 0
    finish_reason: Optional[str] = None
    preemptions: int = 0

    @property
    def tokens(self) -> List[int]:
        return self.prompt + self.output

    def token_slice(self, start: int, n: int) -> List[int]:
        """tokens[start:start + n] without building the whole list (a decoding step asks for the last one)."""
        np_ = len(self.prompt)
        if start >= np_:
            return self.output[start - np_:start - np_ + n]
        if start + n <= np_:
            return self.prompt[start:start + n]
        return self.prompt[start:] + self.output[:start + n - np_]

    @property
    def total_len(self) -> int:
        return len(self.prompt) + len(self.output)

    @property
    def decoding(self) -> bool:
        """All but the newest token are in the cache: the next step is one token."""
        return self.state == RUNNING and len(self.output) > 0 and self.computed == self.total_len - 1


@dataclass
class Scheduled:
    request: Request
    start: int        # first token of the portion (= request.computed)
    n_tokens: int
    sample: bool      # the portion ends at the request's newest token: its last logits give the next token


@dataclass
class ReqResult:
    uid: Hashable
    next_token: Optional[int]
    finished: bool
    reason: Optional[str] = None


class Scheduler:
    def __init__(self, config: SchedulerConfig, cache: CacheManager, eos_token_ids: Sequence[int] = ()):
        self.config = config
        self.cache = cache
        self.eos = set(int(e) for e in eos_token_ids)
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []
        self._arrivals = 0
        self.finished_early: List[ReqResult] = []   # requests refused before they ever ran
        self.counters = {"steps": 0, "tokens": 0, "preemptions": 0, "refused": 0}

    # -- requests in and out -------------------------------------------------
    def add_request(self, req: Request) -> None:
        if not req.prompt:
            raise ValueError(f"request {req.uid!r} has an empty prompt")
        req.state, req.computed, req.arrival = WAITING, 0, self._arrivals
        self._arrivals += 1
        self.waiting.append(req)

    def abort_request(self, uid: Hashable) -> bool:
        for r in list(self.waiting):
            if r.uid == uid:
                self.waiting.remove(r)
                r.state, r.finish_reason = FINISHED, "abort"
                return True
        for r in self.running:
            if r.uid == uid:
                self._finish(r, "abort")
                return True
        return False

    def has_work(self) -> bool:
        return bool(self.waiting or self.running or self.finished_early)

    # -- one step's decisions ------------------------------------------------
    def _capacity_tokens(self) -> int:
        """The longest request that the pools can hold at all.  A group that keeps every key bounds it by its pages; a
        group with a window holds a window and a portion of any request (CacheManager.max_held_pages) and bounds
        nothing if it has the pages for that."""
        limit = self.config.max_seq_len
        for gi, (g, pool) in enumerate(zip(self.cache.groups, self.cache.pools)):
            if g.window <= 0 or pool.num_pages < self.cache.max_held_pages(gi, self.config.chunk_size):
                limit = min(limit, pool.num_pages * self.cache.page_size)
        return limit

    def _need(self, items: List[Tuple[Request, int]], whole: bool = False) -> List[int]:
        """Pages per group that these (request, new length) pairs would take together: in one step, or (whole) the
        most that they will hold at a time on their way there in portions of at most chunk_size."""
        need = [0] * len(self.cache.pools)
        portion = self.config.chunk_size if whole else None
        for r, new_len in items:
            for gi, k in enumerate(self.cache.pages_needed(self.cache.get(r.uid), new_len, portion)):
                need[gi] += k
        return need

    def _fits(self, items: List[Tuple[Request, int]]) -> bool:
        return all(n <= p.available for n, p in zip(self._need(items), self.cache.pools))

    def _preempt(self, r: Request) -> None:
        self.cache.release(r.uid)
        self.running.remove(r)
        r.state, r.computed = WAITING, 0
        r.preemptions += 1
        self.counters["preemptions"] += 1
        self.waiting.appendleft(r)

    def _finish(self, r: Request, reason: str) -> None:
        if r.state == RUNNING:
            self.cache.release(r.uid)
            self.running.remove(r)
        r.state, r.finish_reason = FINISHED, reason

    def _refuse(self, r: Request, reason: str) -> None:
        r.state, r.finish_reason = FINISHED, reason
        self.counters["refused"] += 1
        self.finished_early.append(ReqResult(r.uid, None, True, reason))

    def schedule(self) -> List[Scheduled]:
        """Choose the step's portions.  Pages are not taken here: the step function reserves them, and this
        choice is made so that it will succeed.

        A plan is never empty while requests are running: if nothing can move (requests inside their prompts hold
        every page among them and none is decoding), the youngest running request is preempted and the choice is
        made again, until something moves or the last one, which cannot go on even alone, ends with an error."""
        while True:
            plan = self._plan_once()
            if plan or not self.running:
                return plan
            victim = max(self.running, key=lambda r: r.arrival)
            if len(self.running) == 1:
                self._finish(victim, "out_of_pages")
                self.finished_early.append(ReqResult(victim.uid, None, True, "out_of_pages"))
            else:
                self._preempt(victim)

    def _free_tokens_for(self, r: Request, planned: List[Tuple[Request, int]]) -> int:
        """How many more tokens of r fit into its last page and the pages that `planned` leaves free."""
        ps = self.cache.page_size
        need = self._need(planned)
        free_pages = min((p.available - n for p, n in zip(self.cache.pools, need)), default=None)
        if free_pages is None:
            return self.config.max_seq_len
        rp = self.cache.get(r.uid)
        slack = (-rp.length) % ps       # room left in the page that holds its newest keys
        return max(0, free_pages) * ps + slack

    def _plan_once(self) -> List[Scheduled]:
        cfg = self.config
        budget = cfg.max_extend_tokens
        plan: List[Scheduled] = []
        planned: List[Tuple[Request, int]] = []

        # 1. every decoding request gets its one token; if pages run out, the youngest running request goes
        decoding = sorted((r for r in self.running if r.decoding), key=lambda r: r.arrival)
        while decoding:
            items = [(r, r.computed + 1) for r in decoding[:budget]]
            if self._fits(items):
                break
            victim = max(self.running, key=lambda r: r.arrival)
            if len(self.running) == 1:
                # alone and still no page: it can never go on
                self._finish(victim, "out_of_pages")
                self.finished_early.append(ReqResult(victim.uid, None, True, "out_of_pages"))
            else:
                self._preempt(victim)
            decoding = [r for r in decoding if r is not victim]
        for r in decoding[:budget]:
            plan.append(Scheduled(r, r.computed, 1, True))
            planned.append((r, r.computed + 1))
        budget -= len(plan)

        # 2. running requests still inside their prompt (or being recomputed), oldest first; a portion is cut to
        #    the pages that are left, and a request that gets none waits for decoding requests to free some
        for r in sorted((r for r in self.running if not r.decoding), key=lambda r: r.arrival):
            if budget <= 0:
                break
            n = min(r.total_len - r.computed, cfg.chunk_size, budget)
            if n > 0 and not self._fits(planned + [(r, r.computed + n)]):
                n = min(n, self._free_tokens_for(r, planned))
            if n <= 0:
                continue
            plan.append(Scheduled(r, r.computed, n, r.computed + n == r.total_len))
            planned.append((r, r.computed + n))
            budget -= n

        # 3. admit from the waiting line, in order, while a slot, budget and pages are there: pages for the whole
        #    of what the request holds so far (prompt and produced tokens), beside what the running requests still
        #    need to finish their prompts, so that requests admitted together can all reach decoding
        while self.waiting and budget > 0 and len(self.running) < cfg.max_running_reqs:
            r = self.waiting[0]
            limit = self._capacity_tokens()
            if r.total_len > limit:
                self.waiting.popleft()
                self._refuse(r, "too_long")
                continue
            if self.cache.slots.available == 0:
                break
            n = min(r.total_len - r.computed, cfg.chunk_size, budget)
            self.cache.admit(r.uid)
            # head-room: one page per running request, so that admission does not starve decoding at once
            reserve_pages = len(self.running)
            promised = [(q, max(new_len, q.total_len)) for q, new_len in planned]
            promised += [(q, q.total_len) for q in self.running if all(q is not p for p, _ in planned)]
            need = self._need(promised + [(r, r.total_len)], whole=True)
            ok = all(p.available - k >= reserve_pages for p, k in zip(self.cache.pools, need))
            if not ok:
                self.cache.release(r.uid)
                if not self.running and not plan:
                    # nothing else holds pages and it still does not fit (layers with a window give pages back as
                    # the prompt goes on): cut the portion to what fits
                    n_fit = min(n, self.cache.available_tokens())
                    if n_fit <= 0:
                        self.waiting.popleft()
                        self._refuse(r, "out_of_pages")
                        continue
                    self.cache.admit(r.uid)
                    n = n_fit
                else:
                    break
            self.waiting.popleft()
            r.state = RUNNING
            self.running.append(r)
            plan.append(Scheduled(r, 0, n, n == r.total_len))
            planned.append((r, n))
            budget -= n
        return plan

    def plan_ahead(self, plan: List[Scheduled]) -> Optional[List[Scheduled]]:
        """The step after `plan`, chosen before `plan`'s tokens are known, or None if it cannot be told yet.
        `plan` has been handed to the step function (its pages are taken and its lengths committed) but `update`
        has not seen it.  It can be told if `plan` is every running request's one decoding token, nobody waits,
        nobody reaches a limit with the token it is about to get (an end-of-sequence token may still finish a
        request: its part of the step ahead is then dropped), and the pages for one more token each are free: a
        request that holds start + 1 tokens after `plan` holds start + 2 after the step ahead."""
        if self.waiting or self.finished_early or len(plan) != len(self.running):
            return None
        ahead: List[Scheduled] = []
        for s in plan:
            r = s.request
            if s.n_tokens != 1 or not s.sample or r.state != RUNNING:
                return None
            if len(r.output) + 2 > r.params.max_tokens or r.total_len + 2 > self.config.max_seq_len:
                return None     # its last or last but one token: the plain way finishes it
            ahead.append(Scheduled(r, s.start + 1, 1, True))
        lengths_after = [(a.request, a.start + a.n_tokens) for a in ahead]
        if not self._fits(lengths_after):
            return None         # a page is missing: the next schedule() preempts or finishes somebody
        return ahead

    # -- after the step ------------------------------------------------------
    def update(self, plan: List[Scheduled], sampled: Dict[Hashable, int]) -> List[ReqResult]:
        """Record what the step stored and the tokens sampled for the portions that asked; finish and free."""
        results: List[ReqResult] = list(self.finished_early)
        self.finished_early = []
        self.counters["steps"] += 1
        for s in plan:
            r = s.request
            if r.state != RUNNING:
                continue   # aborted while the step ran
            r.computed = s.start + s.n_tokens
            self.counters["tokens"] += s.n_tokens
            if not s.sample:
                continue
            tok = int(sampled[r.uid])
            r.output.append(tok)
            reason = None
            if tok in self.eos and not r.params.ignore_eos:
                reason = "eos"
            elif len(r.output) >= r.params.max_tokens:
                reason = "max_tokens"
            elif r.total_len >= self.config.max_seq_len:
                reason = "max_seq_len"
            if reason:
                self._finish(r, reason)
            results.append(ReqResult(r.uid, tok, reason is not None, reason))
        return results
