"""The engine a user holds: requests in, tokens out.

`Engine.step()` is the reference's scheduler step (FullScheduler::step,
vt-transformer/core/vt_scheduler.cpp:96-141): choose a batch, run the step
function, take the results, finish and free; `generate()` is the loop its
back end runs (vt_backend.cpp:94-103) without the sockets.  Token ids go in
and come out; text is the front end's business, as in the reference where
sglfront tokenises and the engine sees ids only.
"""
from __future__ import annotations

import os
import time
from typing import Dict, Hashable, Iterable, List, Optional, Sequence, Union

import torch

from ..config import ModelConfig, load_config
from ..sampling import Sampler, SamplingParams, request_seed
from .loading import load_model, make_runner, random_model
from .scheduler import ReqResult, Request, Scheduled, Scheduler, SchedulerConfig
from .step import ModelRunner, StepEntry


class Engine:
    def __init__(self, model: Optional[str] = None, *, config: Optional[ModelConfig] = None,
                 random_weights_seed: Optional[int] = None, dtype: str = "bfloat16", seed: int = 0,
                 scheduler_config: Optional[SchedulerConfig] = None, decode_graphs: bool = True,
                 tune_gemm: bool = False, single_weight_copy: bool = False, **options):
        """model: a folder with config.json and model.safetensors.  Or `config` with `random_weights_seed`
        for random weights drawn on the device.  `options` override fields of SchedulerConfig
        (max_running_reqs, num_pages or kv_bytes, max_seq_len, page_size, max_extend_tokens, default_max_output,
        chunk_size).
        tune_gemm: let the GEMM library try its algorithms on this model's products at chunk_size rows (and at 128
        and 256 rows, if so many requests may run) once, at start-up (some seconds), and use the fastest from then on.
        single_weight_copy: keep the bfloat16 matrices once (in the few-row kernels' order) instead of twice; long
        prompt portions then unpack each matrix into scratch memory for the GEMM library (a fifth slower at 7B sizes).
        For models that fit the GPU's memory once but not twice."""
        sc = scheduler_config or SchedulerConfig()
        for k, v in options.items():
            if not hasattr(sc, k):
                raise TypeError(f"unknown engine option '{k}'")
            setattr(sc, k, v)
        if model is not None:
            self.model = load_model(model, dtype, keep_row_major=not single_weight_copy, page_size=sc.page_size)
        elif config is not None and random_weights_seed is not None:
            self.model = random_model(config, random_weights_seed, dtype, keep_row_major=not single_weight_copy,
                                      page_size=sc.page_size)
        else:
            raise ValueError("give a model folder, or a config and random_weights_seed")
        spec = self.model.spec
        sc.max_seq_len = min(sc.max_seq_len, spec.max_positions)
        self.config = sc
        self.runner: ModelRunner = make_runner(
            self.model, pool_tokens=None if sc.kv_bytes is not None else sc.num_pages * sc.page_size,
            kv_bytes=sc.kv_bytes, page_size=sc.page_size, max_requests=sc.max_running_reqs, max_seq_len=sc.max_seq_len,
            max_portion=sc.chunk_size)
        sc.num_pages = self.runner.storage.num_pages
        self.runner.decode_graphs = bool(decode_graphs)
        self.scheduler = Scheduler(sc, self.runner.cache, spec.eos_token_ids)
        self.sampler = Sampler(self.model.rt)
        self.seed = int(seed)
        self._next_uid = 0
        self.requests: Dict[Hashable, Request] = {}
        self.pipeline_decode = True     # start the next decoding step before this one's tokens are on the host
        self._ahead = None              # (plan, pending tokens) of a step that is already queued on the GPU
        if tune_gemm:
            self.tune_library_products()
            for rows in (128, 256):     # decoding batches beyond the few-row kernels' 64 rows take the library too
                if rows <= sc.max_running_reqs:
                    self.tune_library_products(rows)

    def tune_library_products(self, rows: Optional[int] = None) -> float:
        """Long portions multiply through the GEMM library (parts/linear.py).  This runs one portion of `rows`
        tokens (default: chunk_size) with the library's algorithm search switched on, so that every product of
        the model is tried at that size; afterwards the search is off again and other sizes take the library's
        default.  What it finds is kept in a file beside the compiled kernels, so a later start is quick.
        Returns the seconds it took."""
        import torch.cuda.tunable as tunable
        sc = self.config
        n = rows or sc.chunk_size
        n = max(65, min(n, sc.max_seq_len - 1, self.runner.cache.available_tokens()))
        t0 = time.time()
        tunable.enable(True)
        # the library reads earlier results from this file and rewrites it when the process ends
        from ..kernels.build import _build_dir
        tunable.set_filename(os.path.join(_build_dir(), "gemm_algorithms.csv"))
        tunable.tuning_enable(True)
        try:
            rid = ("tune", id(self))
            self.runner.admit(rid)
            try:
                self.runner.step([StepEntry(rid, [0] * n, [n - 1])])
                torch.cuda.synchronize()
            finally:
                self.runner.release(rid)
        finally:
            tunable.tuning_enable(False)
        return time.time() - t0

    # -- requests ------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None,
                    uid: Optional[Hashable] = None) -> Hashable:
        if uid is None:
            uid = self._next_uid
            self._next_uid += 1
        if uid in self.requests and self.requests[uid].state != "finished":
            raise ValueError(f"request id {uid!r} is in use")
        params = params or SamplingParams(max_tokens=self.config.default_max_output)
        vocab = self.model.spec.vocab_size
        for t in prompt:
            if not 0 <= int(t) < vocab:
                raise ValueError(f"token id {t} is outside the vocabulary of {vocab}")
        seed = params.seed if params.seed is not None else request_seed(self.seed, uid)
        req = Request(uid, [int(t) for t in prompt], params, seed)
        self.requests[uid] = req
        self.scheduler.add_request(req)
        return uid

    def abort_request(self, uid: Hashable) -> bool:
        return self.scheduler.abort_request(uid)

    def has_work(self) -> bool:
        return self.scheduler.has_work() or self._ahead is not None

    # -- one step ------------------------------------------------------------
    def step(self) -> List[ReqResult]:
        """One step of the scheduler's loop: choose a batch, run it, take the sampled tokens, finish and free.

        While every running request is decoding and nobody waits, the step after this one is started before this
        one's tokens have reached the host (its input is what the sampler left on the device), so the GPU does not
        wait while the host does its bookkeeping.  What that step computes for a request that turns out to have
        finished in this one is dropped; its pages are only reused by work that is queued behind it."""
        cur, self._ahead = self._ahead, None
        if cur is None:
            plan = self.scheduler.schedule()
            if not plan:
                results = self.scheduler.update(plan, {})
                if not results and (self.scheduler.running or self.scheduler.waiting):
                    raise RuntimeError(
                        f"the scheduler has {len(self.scheduler.running)} running and {len(self.scheduler.waiting)} "
                        f"waiting requests and nothing to run: no slot, page or token budget lets any of them move")
                return results
            cur = self._launch(plan, None)
        if self.pipeline_decode:
            nxt = self._plan_ahead(cur[0])
            if nxt is not None:
                self._ahead = self._launch(nxt, cur[1].tokens_dev)
        plan, pending = cur
        sampled: Dict[Hashable, int] = {}
        if pending is not None:
            toks = self.sampler.collect(pending)
            for s, t in zip((s for s in plan if s.sample), toks):
                sampled[s.request.uid] = t
        results = self.scheduler.update(plan, sampled)
        if self._ahead is not None and not any(s.request.state == "running" for s in self._ahead[0]):
            self._ahead = None      # everybody in it has finished meanwhile: nothing of it is wanted
        return results

    def _launch(self, plan: List[Scheduled], ids_dev):
        """Queue the plan's step and its sampling on the GPU; returns (plan, pending tokens or None)."""
        ahead = ids_dev is not None         # the requests' newest tokens are not on the host yet
        entries = []
        for s in plan:
            toks = [0] if ahead else s.request.token_slice(s.start, s.n_tokens)
            entries.append(StepEntry(s.request.uid, toks, [s.n_tokens - 1] if s.sample else []))
        logits = self.runner.step(entries, ids_dev)
        rows = [(s.request.params, s.request.seed, len(s.request.output) + (1 if ahead else 0)) for s in plan if s.sample]
        return plan, (self.sampler.launch(logits, rows) if rows else None)

    def _plan_ahead(self, plan: List[Scheduled]) -> Optional[List[Scheduled]]:
        """The step after `plan`, which is already queued on the GPU, if it can be told without `plan`'s tokens
        (Scheduler.plan_ahead) and goes through a captured graph."""
        if not self.runner.replays(len(plan)):
            return None
        return self.scheduler.plan_ahead(plan)

    # -- the whole loop --------------------------------------------------------
    def generate(self, prompts: Union[Sequence[int], Sequence[Sequence[int]]],
                 params: Union[None, SamplingParams, Sequence[SamplingParams]] = None) -> List[List[int]]:
        """Token ids in, generated token ids out (one list per prompt, in order).  The requests of this call stay
        readable (`requests`, `finish_reason`) until the next call, which forgets every finished request."""
        for u in [u for u, r in self.requests.items() if r.state == "finished"]:
            del self.requests[u]
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        plist = [prompts] if single else list(prompts)
        if params is None or isinstance(params, SamplingParams):
            params = [params] * len(plist)
        uids = [self.add_request(p, sp) for p, sp in zip(plist, params)]
        while self.has_work():
            self.step()         # (raises if requests are left and none can move)
        outs = [self.requests[u].output for u in uids]
        return outs[0:1] if single else outs

    def finish_reason(self, uid: Hashable) -> Optional[str]:
        return self.requests[uid].finish_reason

    def forget(self, uid: Hashable) -> Request:
        """Drop a finished request from the engine's books (a caller of add_request/step does this once it has
        read the request's output, or the books grow for as long as the engine lives); returns the request."""
        req = self.requests[uid]
        if req.state != "finished":
            raise ValueError(f"request {uid!r} has not finished (abort it first)")
        return self.requests.pop(uid)
