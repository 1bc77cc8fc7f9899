"""Building traces (lists of steps in bin/trace_run's format) and checking
their logits against the plain implementation."""
from __future__ import annotations

import json
import os
import subprocess
import sys
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

import plain_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# max |engine - plain| over a row of logits, relative to the row's largest |plain| logit
# (bfloat16 and float16: about twice the worst error that any of the comparisons built on this has shown, 7.5e-3 and
# 9.8e-4)
TOL = {"float32": 2e-5, "bfloat16": 1.5e-2, "float16": 2e-3}


def random_requests(vocab: int, lengths: Sequence[int], seed: int) -> Dict[str, List[int]]:
    rs = np.random.RandomState(seed)
    return {f"r{i}": rs.randint(0, vocab, size=n).tolist() for i, n in enumerate(lengths)}


def cut(tokens: List[int], sizes: Sequence[int]) -> List[Tuple[int, int]]:
    """(start, end) portions of the given sizes, the last size repeated until the tokens end."""
    out, pos, i = [], 0, 0
    while pos < len(tokens):
        n = sizes[min(i, len(sizes) - 1)]
        out.append((pos, min(len(tokens), pos + n)))
        pos += n
        i += 1
    return out


def trace_alone(reqs: Dict[str, List[int]], portions: Dict[str, List[Tuple[int, int]]], want_all=True) -> List[dict]:
    """Each request alone, one after the other, in the given portions; logits wanted at every place."""
    steps = []
    for rid, toks in reqs.items():
        parts = portions[rid]
        for j, (a, b) in enumerate(parts):
            steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks[a:b],
                                                            "want": list(range(b - a)) if want_all else [b - a - 1]}],
                          "end": [rid] if j == len(parts) - 1 else []})
    return steps


def trace_mixed(reqs: Dict[str, List[int]], portions: Dict[str, List[Tuple[int, int]]], max_live: int, seed: int,
                skip_prob: float = 0.2) -> List[dict]:
    """Up to max_live requests at a time; every step takes the next portion of each live request (sometimes leaving
    one out), so portions of prompts stand beside single tokens; a finished request frees its pages for the next."""
    rs = np.random.RandomState(seed)
    waiting = list(reqs)
    live: List[str] = []
    nxt = {r: 0 for r in reqs}
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            live.append(waiting.pop(0))
        entries, end = [], []
        chosen = [r for r in live if rs.rand() >= skip_prob] or [live[0]]
        for r in chosen:
            a, b = portions[r][nxt[r]]
            entries.append({"id": r, "tokens": reqs[r][a:b], "want": list(range(b - a))})
            nxt[r] += 1
            if nxt[r] == len(portions[r]):
                end.append(r)
        steps.append({"step": len(steps), "entries": entries, "end": end})
        live = [r for r in live if r not in end]
    return steps


def max_live_tokens(steps: List[dict], round_to: int = 64) -> int:
    """The most tokens live requests hold at any time, each rounded up to a multiple of round_to."""
    held: Dict[str, int] = {}
    peak = 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        peak = max(peak, sum(-(-n // round_to) * round_to for n in held.values()))
        for r in s["end"]:
            held.pop(r, None)
    return peak


def run_in_process(runner, steps: List[dict]) -> Dict[int, np.ndarray]:
    from vt_transformer_amd.engine import StepEntry
    out = {}
    live = set()
    for s in steps:
        entries = []
        for e in s["entries"]:
            if e["id"] not in live:
                assert runner.admit(e["id"])
                live.add(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e["want"]))
        logits = runner.step(entries)
        if logits is not None:
            out[s["step"]] = logits.float().cpu().numpy().copy()
        for r in s["end"]:
            runner.release(r)
            live.discard(r)
        runner.cache.check()
    return out


def run_trace_run(model_dir: str, dtype: str, steps: List[dict], out_dir: str, max_tokens: int, vocab: int,
                  env=None, extra_args: Tuple[str, ...] = ()) -> Dict[int, np.ndarray]:
    """Drive bin/trace_run as a user would: steps on stdin, `done <step>` awaited after each."""
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype,
           "--out", out_dir, "--max-tokens", str(max_tokens), *extra_args]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            assert line.strip() == f"done {s['step']}", f"trace_run said {line!r} after step {s['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    out = {}
    for s in steps:
        n_want = sum(len(e["want"]) for e in s["entries"])
        path = os.path.join(out_dir, f"{s['step']}.f32")
        if n_want:
            out[s["step"]] = np.fromfile(path, dtype="<f4").reshape(n_want, vocab)
        else:
            assert not os.path.exists(path)
    return out


def check_against_plain(model_dir: str, reqs: Dict[str, List[int]], steps: List[dict], got: Dict[int, np.ndarray],
                        dtype: str, plain_cache: dict = None) -> float:
    """Every wanted row against the plain model's logits at that request's position.  Returns the worst error;
    raises at the first row beyond tolerance, naming step, request and position."""
    cfg, w = plain_model.read_folder(model_dir)
    plain_cache = plain_cache if plain_cache is not None else {}
    ref = {}
    for rid, toks in reqs.items():
        key = (model_dir, tuple(toks))
        if key not in plain_cache:
            plain_cache[key] = plain_model.forward(cfg, w, toks).numpy()
        ref[rid] = plain_cache[key]
    pos = {r: 0 for r in reqs}
    worst = 0.0
    for s in steps:
        row = 0
        for e in s["entries"]:
            for wi in e["want"]:
                p = pos[e["id"]] + wi
                r = ref[e["id"]][p]
                g = got[s["step"]][row].astype(np.float64)
                err = float(np.abs(g - r).max() / max(np.abs(r).max(), 1e-30))
                assert np.isfinite(g).all(), f"step {s['step']} request {e['id']} position {p}: logits are not finite"
                assert err < TOL[dtype], (f"step {s['step']} request {e['id']} position {p} "
                                          f"(portion starts at {pos[e['id']]}): error {err:.3e} > {TOL[dtype]:.0e}")
                worst = max(worst, err)
                row += 1
            pos[e["id"]] += len(e["tokens"])
        assert row == (got[s["step"]].shape[0] if s["step"] in got else 0)
    return worst
