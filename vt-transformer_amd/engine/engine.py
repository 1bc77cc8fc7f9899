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
        (max_running_reqs, num_pages, max_seq_len, page_size, max_extend_tokens, default_max_output, chunk_size).
        tune_gemm: let the GEMM library try its algorithms on this model's products at chunk_size rows (and at 128
        and 256 rows, if so many requests may run) once, at start-up (some seconds), and use the fastest from then on.
        single_weight_copy: keep the bfloat16 matrices once (in the few-row kernels' order) instead of twice; long
        prompt portions are then several times slower.  For models that fit the GPU's memory once but not twice."""
        sc = scheduler_config or SchedulerConfig()
        for k, v in options.items():
            if not hasattr(sc, k):
                raise TypeError(f"unknown engine option '{k}'")
            setattr(sc, k, v)
        if model is not None:
            self.model = load_model(model, dtype, keep_row_major=not single_weight_copy)
        elif config is not None and random_weights_seed is not None:
            self.model = random_model(config, random_weights_seed, dtype, keep_row_major=not single_weight_copy)
        else:
            raise ValueError("give a model folder, or a config and random_weights_seed")
        spec = self.model.spec
        sc.max_seq_len = min(sc.max_seq_len, spec.max_positions)
        self.config = sc
        self.runner: ModelRunner = make_runner(self.model, pool_tokens=sc.num_pages * sc.page_size,
                                               page_size=sc.page_size, max_requests=sc.max_running_reqs,
                                               max_seq_len=sc.max_seq_len)
        self.runner.decode_graphs = bool(decode_graphs)
        self.scheduler = Scheduler(sc, self.runner.cache, spec.eos_token_ids)
        self.sampler = Sampler(self.model.rt)
        self.seed = int(seed)
        self._next_uid = 0
        self.requests: Dict[Hashable, Request] = {}
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
        return self.scheduler.has_work()

    # -- one step ------------------------------------------------------------
    def step(self) -> List[ReqResult]:
        plan = self.scheduler.schedule()
        sampled: Dict[Hashable, int] = {}
        if plan:
            entries = []
            for s in plan:
                toks = s.request.token_slice(s.start, s.n_tokens)
                entries.append(StepEntry(s.request.uid, toks, [s.n_tokens - 1] if s.sample else []))
            logits = self.runner.step(entries)
            rows = [(s.request.params, s.request.seed, len(s.request.output)) for s in plan if s.sample]
            if rows:
                toks = self.sampler.sample(logits, rows)
                for s, t in zip((s for s in plan if s.sample), toks):
                    sampled[s.request.uid] = t
        return self.scheduler.update(plan, sampled)

    # -- the whole loop --------------------------------------------------------
    def generate(self, prompts: Union[Sequence[int], Sequence[Sequence[int]]],
                 params: Union[None, SamplingParams, Sequence[SamplingParams]] = None) -> List[List[int]]:
        """Token ids in, generated token ids out (one list per prompt, in order)."""
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        plist = [prompts] if single else list(prompts)
        if params is None or isinstance(params, SamplingParams):
            params = [params] * len(plist)
        uids = [self.add_request(p, sp) for p, sp in zip(plist, params)]
        while self.has_work():
            results = self.step()
            if not results and not self.scheduler.running and self.scheduler.waiting:
                raise RuntimeError("the scheduler cannot place the waiting requests (pool too small?)")
        outs = [self.requests[u].output for u in uids]
        return outs[0:1] if single else outs

    def finish_reason(self, uid: Hashable) -> Optional[str]:
        return self.requests[uid].finish_reason
