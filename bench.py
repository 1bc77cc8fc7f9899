#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Qwen2-7B layer sizes, random weights, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints one JSON line.  `value` is decoded tokens per second at batch 8 after 1,024-token prompts (a step is one
decode step of the whole batch through scheduler, step function and sampler).  The line also carries the
prefill of one 2,048-token prompt, the decode step's achieved HBM bandwidth against the bytes it has to read,
decode at batch 1 and 64 (`points`, and `points_frac`: their fractions of the same roofline), and what this GPU's
memory and matrix cores were measured to deliver (a kernel that only reads; the library's square product), beside
the published peaks that the fractions are taken against (`vs_measured_peaks`: the same fractions against those).
Run without --sizes or --mixed it then measures the other two workloads that the baseline names, each model built
and freed in turn, and adds them to `points` / `points_frac`: Qwen2-1.5B layer sizes (decode at batch 8; 64 requests
at once with prompts of 16 to 4,096 tokens and 256 decoded tokens each: generated tok/s, its steps and seconds under
`mixed_1.5b`) and Qwen2-72B layer sizes (decode at batch 1 and 16 after 2,048-token prompts).
The reference publishes no number to compare with (vs_baseline is null).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# Qwen2-7B layer sizes (v1/models/qwen2-7b/inference_fp16.dag:1-15 of the reference)
QWEN2_7B = dict(architectures=["Qwen2ForCausalLM"], vocab_size=152064, hidden_size=3584, intermediate_size=18944,
                num_hidden_layers=28, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
                rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=8192,
                hidden_act="silu", use_sliding_window=False)
# Qwen2-72B layer sizes: about 145 GB of bfloat16 weights, which fit one MI355X once (--sizes 72b keeps one copy)
QWEN2_72B = dict(QWEN2_7B, hidden_size=8192, intermediate_size=29568, num_hidden_layers=80, num_attention_heads=64,
                 num_key_value_heads=8)
# Qwen2-1.5B layer sizes (tied head)
QWEN2_15B = dict(QWEN2_7B, vocab_size=151936, hidden_size=1536, intermediate_size=8960, num_attention_heads=12,
                 num_key_value_heads=2, tie_word_embeddings=True, max_position_embeddings=32768)
SIZES = {"7b": ("Qwen2-7B", QWEN2_7B, (1, 64)), "72b": ("Qwen2-72B", QWEN2_72B, (1, 16)),
         "1.5b": ("Qwen2-1.5B", QWEN2_15B, (1, 64))}
HBM_GBPS = 8000.0          # MI355X HBM3E, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "fp32": 157.3e12}   # dense MFMA, published


def size_line(d: dict) -> str:
    """A configuration's sizes as one flat string."""
    return (f"L{d['num_hidden_layers']} H{d['hidden_size']} NH{d['num_attention_heads']} KVH{d['num_key_value_heads']} "
            f"D{d['head_dim']} I{d['intermediate_size']} V{d['vocab_size']} {'tied' if d['tie_word_embeddings'] else 'untied'} "
            f"ctx{d['max_position_embeddings']}")


class Bench:
    """An engine at one configuration's sizes with random weights, and the measurements on it."""

    def __init__(self, sizes_key: str, dtype: str, max_batch: int, pool_tokens: int, ctx_len: int = 0, layers: int = 0,
                 graphs: bool = True, seed: int = 0):
        import numpy as np
        import torch
        from vt_transformer_amd.config import config_from_dict
        from vt_transformer_amd.engine import Engine
        self.torch, self.np = torch, np
        self.model_name, sizes, self.point_batches = SIZES[sizes_key]
        self.full_layers = sizes["num_hidden_layers"]
        self.single_copy = sizes_key == "72b"
        cfg_d = dict(sizes)
        cfg_d["num_hidden_layers"] = layers or self.full_layers
        self.cfg = cfg = config_from_dict(cfg_d)
        self.ctx_len = ctx_len or cfg.max_position_embeddings
        self.rs = np.random.RandomState(seed)
        t0 = time.time()
        self.eng = Engine(config=cfg, random_weights_seed=0, dtype=dtype, page_size=16, num_pages=-(-pool_tokens // 16),
                          max_running_reqs=max(max_batch, 1), max_seq_len=self.ctx_len, max_extend_tokens=8192,
                          chunk_size=2048, decode_graphs=graphs, single_weight_copy=self.single_copy)
        torch.cuda.synchronize()
        print(f"[bench] {self.model_name} sizes: model ready in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
        # sizes for the roofline
        H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
        self.qkv = qkv = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * cfg.head_dim
        layer_params = qkv * H + qkv + cfg.num_attention_heads * cfg.head_dim * H + 3 * I * H + 2 * H
        self.weight_bytes = 2 * (L * layer_params + V * H + H)         # every weight a step uses, once (16 bits each)
        self.kv_bytes_per_token = 2 * 2 * L * cfg.num_key_value_heads * cfg.head_dim

    def close(self) -> None:
        self.eng = None
        import gc
        gc.collect()
        self.torch.cuda.empty_cache()

    def tune(self, rows: int) -> None:
        print(f"[bench] GEMM library algorithm search at {rows} rows: {self.eng.tune_library_products(rows):.1f} s",
              file=sys.stderr, flush=True)

    def hbm_frac(self, batch: int, ctx: int, ms: float) -> float:
        """The decode step's roofline: the weights once and the live requests' keys and values, over its time."""
        return (self.weight_bytes + batch * ctx * self.kv_bytes_per_token) / (ms * 1e-3) / 1e9 / HBM_GBPS

    def decode_run(self, batch: int, steps: int, warmup: int, prompt_len: int):
        """tokens/s, ms/step and the context at mid-run of `steps` decode steps at `batch` after prompts of prompt_len."""
        from vt_transformer_amd.sampling import SamplingParams
        eng, torch = self.eng, self.torch
        sp = SamplingParams(max_tokens=steps + warmup + 8, ignore_eos=True)
        uids = [eng.add_request(self.rs.randint(0, self.cfg.vocab_size, size=prompt_len).tolist(), sp) for _ in range(batch)]
        while any(not eng.requests[u].decoding for u in uids):      # prompts, in portions under the token budget
            eng.step()
        for _ in range(warmup):
            eng.step()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        ctx_mid = prompt_len + 1 + warmup + steps // 2
        for u in uids:
            eng.abort_request(u)
        while eng.has_work():
            eng.step()
        for u in uids:
            eng.forget(u)
        print(f"[bench] {self.model_name} decode batch {batch} after {prompt_len}-token prompts: "
              f"{batch * steps / dt:.1f} tok/s, {dt / steps * 1e3:.3f} ms/step", file=sys.stderr, flush=True)
        return batch * steps / dt, dt / steps * 1e3, ctx_mid

    def prefill_run(self, tokens: int, reps: int = 3):
        from vt_transformer_amd.engine import StepEntry
        runner, torch = self.eng.runner, self.torch
        best = None
        for i in range(reps + 1):
            rid = f"prefill{i}"
            runner.admit(rid)
            ids = self.rs.randint(0, self.cfg.vocab_size, size=tokens).tolist()
            torch.cuda.synchronize()
            t = time.perf_counter()
            runner.step([StepEntry(rid, ids, [tokens - 1])])
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            runner.release(rid)
            if i > 0:
                best = dt if best is None else min(best, dt)
        print(f"[bench] {self.model_name} prefill {tokens} tokens: {best * 1e3:.2f} ms", file=sys.stderr, flush=True)
        return best

    def prefill_flops(self, T: int) -> float:
        cfg = self.cfg
        H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
        mm = 2.0 * T * L * (self.qkv * H + cfg.num_attention_heads * cfg.head_dim * H + 3 * I * H) + 2.0 * V * H
        attn = L * 4.0 * cfg.num_attention_heads * cfg.head_dim * (T * (T + 1) / 2)     # causal: QK^T and PV
        return mm + attn

    def mixed_run(self, lens, decode_tokens: int, reps: int = 2):
        """All requests arrive at once; the scheduler cuts their prompts into portions under its token budget and
        decodes beside them.  Best of `reps` runs: seconds, steps, prompt tokens."""
        from vt_transformer_amd.sampling import SamplingParams
        eng, torch = self.eng, self.torch
        prompts = [self.rs.randint(0, self.cfg.vocab_size, size=int(n)).tolist() for n in lens]
        sp = SamplingParams(max_tokens=decode_tokens, ignore_eos=True)
        best = None
        for rep in range(reps):
            uids = [eng.add_request(p, sp) for p in prompts]
            torch.cuda.synchronize()
            t, steps = time.perf_counter(), 0
            while eng.has_work():
                eng.step()
                steps += 1
            torch.cuda.synchronize()
            dt = time.perf_counter() - t
            for u in uids:
                eng.forget(u)
            print(f"[bench] {self.model_name} mixed run {rep}: {dt:.3f} s, {steps} steps", file=sys.stderr, flush=True)
            best = dt if best is None else min(best, dt)
        return best, steps, int(sum(int(n) for n in lens))


def mixed_lengths(n: int, seed: int = 0):
    import numpy as np
    return np.random.RandomState(seed).randint(16, 4097, size=n)


def mixed_pool(lens, decode_tokens: int) -> int:
    return int(sum(-(-(int(n) + decode_tokens + 16) // 16) * 16 for n in lens))


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=0,
                    help="tokens of the prompts that the decode steps follow (default: 1,024; 2,048 with --sizes 72b, "
                         "as the baseline's workloads have them)")
    ap.add_argument("--sizes", choices=sorted(SIZES), default=None,
                    help="layer sizes (default 7b, followed by the 1.5b and 72b workloads); 72b keeps one copy of the "
                         "weights (long prompt portions unpack each matrix for the library)")
    ap.add_argument("--dtype", choices=["bfloat16", "float16"], default="float16",
                    help="the 16-bit type of weights, activations and cache: float16 as in the reference's "
                         "inference_fp16.dag, or bfloat16 (the same kernels and rates either way)")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (named in config)")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--no-extra", action="store_true", help="skip the 1.5b and 72b workloads behind a default run")
    ap.add_argument("--no-graphs", action="store_true")
    ap.add_argument("--no-prefill", action="store_true", help="skip the prefill measurement (profiling runs)")
    ap.add_argument("--no-peaks", action="store_true", help="skip the measurement of what this GPU's memory and matrix "
                    "cores deliver to a kernel that only reads and to the library's square product")
    ap.add_argument("--no-tune", action="store_true", help="do not let the GEMM library search its algorithms at start-up")
    ap.add_argument("--mixed", type=int, default=0, metavar="REQUESTS",
                    help="another workload instead: this many requests at once with prompt lengths drawn from 16 to "
                         "4,096 and --mixed-decode tokens each, through the scheduler (portions of prompts beside "
                         "decoded tokens); value = generated tokens per second from first arrival to last token")
    ap.add_argument("--mixed-decode", type=int, default=256)
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this engine runs on one GPU; N > 1 is not measured")
        return 2

    import torch

    extra = args.sizes is None and not args.mixed and not args.no_extra and not args.layers
    sizes_key = args.sizes or "7b"
    prompt_len = args.prompt_len or (2048 if sizes_key == "72b" else 1024)
    model_name, sizes, point_batches = SIZES[sizes_key]
    dtype_name = {"bfloat16": "bf16", "float16": "fp16"}[args.dtype]
    lowp = getattr(torch, args.dtype)
    max_batch = max(point_batches) if not args.no_points else max(args.batch, 1)
    max_batch = max(max_batch, args.batch)
    per_req = -(-(prompt_len + args.steps + args.warmup + 32) // 16) * 16
    pool_tokens = max(max_batch * per_req, args.prefill_tokens + 64)
    ctx_len = 0
    if args.mixed:
        mixed_lens = mixed_lengths(args.mixed)
        pool_tokens = mixed_pool(mixed_lens, args.mixed_decode)
        max_batch, ctx_len = args.mixed, min(sizes["max_position_embeddings"], 8192)
    b = Bench(sizes_key, args.dtype, max_batch, pool_tokens, ctx_len=ctx_len, layers=args.layers, graphs=not args.no_graphs)
    cfg, single_copy, ctx_len, FULL_LAYERS = b.cfg, b.single_copy, b.ctx_len, b.full_layers
    if not args.no_tune and not args.no_prefill and not single_copy:
        b.tune(args.prefill_tokens)

    def measured_peaks():
        """What this machine delivers: GB/s of a kernel that only reads 2 GB (beyond the last-level cache), and
        TFLOP/s of the GEMM library on an 8,192-cube in the run's 16-bit type."""
        from vt_transformer_amd.kernels import ops
        buf = torch.randint(0, 1 << 30, (1 << 29,), dtype=torch.int32, device="cuda")
        sums = torch.empty(256 * 16, dtype=torch.int32, device="cuda")
        a = torch.randn(8192, 8192, device="cuda").to(lowp)
        bb = torch.randn(8192, 8192, device="cuda").to(lowp)
        c = torch.empty(8192, 8192, dtype=lowp, device="cuda")

        def best_ms(fn, reps=6):
            best = None
            for i in range(reps):
                st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                st.record()
                fn()
                en.record()
                torch.cuda.synchronize()
                if i:
                    best = st.elapsed_time(en) if best is None else min(best, st.elapsed_time(en))
            return best
        read_ms = best_ms(lambda: ops.stream_read(buf, sums))
        mm_ms = best_ms(lambda: torch.mm(a, bb.t(), out=c))
        out = {"hbm_read_GBps": round(buf.numel() * 4 / read_ms / 1e6, 1),
               "gemm_TFLOPs": round(2 * 8192 ** 3 / mm_ms / 1e9, 1)}
        print(f"[bench] measured peaks: {out}", file=sys.stderr, flush=True)
        return out

    if args.mixed:
        dt, steps, prompt_tokens = b.mixed_run(mixed_lens, args.mixed_decode)
        gen = args.mixed * args.mixed_decode
        print(json.dumps({
            "metric": f"generated tok/s, {args.mixed} requests at once, prompts of 16 to 4,096 tokens, "
                      f"{args.mixed_decode} decoded tokens each, {model_name} layer sizes",
            "value": round(gen / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 0,
            "ms_per_step": round(dt / steps * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": dtype_name, "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
            "config": {"model": f"{model_name} sizes", "layers": cfg.num_hidden_layers, "layers_full": FULL_LAYERS,
                       "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads,
                       "head_dim": cfg.head_dim, "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size,
                       "global_batch": args.mixed, "seq_len": int(mixed_lens.max()), "prompt_tokens": prompt_tokens,
                       "decode_tokens": args.mixed_decode, "context_len": ctx_len, "kv_block": 16,
                       "max_extend_tokens": 8192, "chunk_size": 2048, "parallelism": "1 GPU"},
            "total_tokens_per_s": round((prompt_tokens + gen) / dt, 1), "seconds": round(dt, 3)}), flush=True)
        return 0

    tps, ms, ctx_mid = b.decode_run(args.batch, args.steps, args.warmup, prompt_len)
    achieved = b.hbm_frac(args.batch, ctx_mid, ms) * HBM_GBPS

    T = args.prefill_tokens
    p_dt = b.prefill_run(T) if not args.no_prefill else None
    p_flops = b.prefill_flops(T)

    points, points_frac = {}, {}
    if not args.no_points:
        for pb in point_batches:
            k = max(16, args.steps // 2)
            b_tps, b_ms, b_ctx = b.decode_run(pb, k, 8, prompt_len)
            points[f"decode_b{pb}"] = round(b_tps, 1)
            points_frac[f"decode_b{pb}"] = round(b.hbm_frac(pb, b_ctx, b_ms), 4)

    H, I, V, L = cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {model_name} layer sizes, {prompt_len:,}-token prompts",
        "value": round(tps, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype_name, "data": "synthetic (random weights N(0,0.02), uniform random token ids)",
        "config": {"model": f"{model_name} sizes", "layers": L, "layers_full": FULL_LAYERS, "hidden": H,
                   "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                   "intermediate": I, "vocab": V, "global_batch": args.batch, "seq_len": prompt_len,
                   "context_len": ctx_len, "kv_block": 16, "rope_theta": cfg.rope_theta,
                   "parallelism": "1 GPU", "decode_graphs": not args.no_graphs, "gemm_tuning": not (args.no_tune or single_copy),
                   "weight_copies": 1 if single_copy else 2},
        "prefill": None if p_dt is None else {"value": round(T / p_dt, 1), "tokens": T, "ms": round(p_dt * 1e3, 3),
                                              "frac": round(p_flops / p_dt / PEAK_FLOPS[dtype_name], 4)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_GBPS, 4)},
        "points": points,
        "points_frac": points_frac,
    }
    peaks = None
    if not args.no_peaks:
        peaks = measured_peaks()
        line["measured_peaks"] = peaks

    if extra:
        # the baseline's other two workloads, each model built and freed in turn
        b.close()
        d15 = SIZES["1.5b"][1]
        lens = mixed_lengths(64)
        b15 = Bench("1.5b", args.dtype, 64, max(mixed_pool(lens, 256), 8 * per_req), graphs=not args.no_graphs)
        if not args.no_tune:
            b15.tune(2048)
        k = max(16, args.steps // 2)
        t15, ms15, ctx15 = b15.decode_run(8, k, 8, 1024)
        points["1.5b_decode_b8"] = round(t15, 1)
        points_frac["1.5b_decode_b8"] = round(b15.hbm_frac(8, ctx15, ms15), 4)
        m_dt, m_steps, m_prompt = b15.mixed_run(lens, 256)
        points["1.5b_mixed64"] = round(64 * 256 / m_dt, 1)
        line["mixed_1.5b"] = {"requests": 64, "prompt_tokens": m_prompt, "decode_tokens": 256, "steps": m_steps,
                              "seconds": round(m_dt, 3), "total_tokens_per_s": round((m_prompt + 64 * 256) / m_dt, 1)}
        line["config"]["sizes_1.5b"] = size_line(d15) + "; decode at batch 8 after 1,024-token prompts; 64 requests at " \
            "once, prompts of 16 to 4,096 tokens, 256 decoded tokens each"
        b15.close()
        d72 = SIZES["72b"][1]
        per72 = -(-(2048 + k + 8 + 32) // 16) * 16
        b72 = Bench("72b", args.dtype, 16, 16 * per72, graphs=not args.no_graphs)
        for pb in (1, 16):
            t72, ms72, ctx72 = b72.decode_run(pb, k if pb > 1 else max(16, k // 2), 4, 2048)
            points[f"72b_decode_b{pb}"] = round(t72, 1)
            points_frac[f"72b_decode_b{pb}"] = round(b72.hbm_frac(pb, ctx72, ms72), 4)
        line["config"]["sizes_72b"] = size_line(d72) + "; decode at batch 1 and 16 after 2,048-token prompts; one copy " \
            "of the weights"
        b72.close()

    if peaks is not None:
        # the same fractions against what this machine was measured to deliver
        vs = {"decode": round(achieved / peaks["hbm_read_GBps"], 4)}
        if p_dt is not None:
            vs["prefill"] = round(p_flops / p_dt / (peaks["gemm_TFLOPs"] * 1e12), 4)
        for k_, f in points_frac.items():
            vs[k_] = round(f * HBM_GBPS / peaks["hbm_read_GBps"], 4)
        line["vs_measured_peaks"] = vs
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
