"""Command line of the engine, in the manner of the reference's front ends.

    python -m vt_transformer_amd --model DIR --prompt-ids 1,2,3 --max-tokens 16
    python -m vt_transformer_amd --model DIR --shell-mode
    python -m vt_transformer_amd --write-random-model DIR --config config.json --seed 1

Option names and meanings follow the reference where it has them:
`--model-path` / `--model` / `--tokenizer-path`, `--model-name` and `--shell-mode` of
sglfront (sglfront/sglfront/server/args.py:88-202); the sampling options of its
SamplingParams (sglfront/sglfront/core.py:6-16); the shell's commands /exit and /reset and
its defaults from SGLFRONT_SHELL_MAX_TOKENS, _TOP_K, _TOP_P, _TEMPERATURE
(sglfront/sglfront/server/api_server.py:352-365, sglfront/sglfront/env.py:50-53); the
scheduler's options of SchedulerConfig (vt-transformer/core/vt_scheduler.hpp:28-39); and the
closing line of v1's chat driver, "Generated N tokens, using S seconds"
(v1/models/qwen2-7b/chat.cpp:112-117), whose `!` also resets the history (:61-68).
Token ids go in and out; with a tokenizer.json (in the model folder or at --tokenizer-path)
text does too.  There is no HTTP server here.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from typing import List, Optional


def _env(name: str, default, conv):
    v = os.getenv("SGLFRONT_" + name)
    if v is None:
        return default
    try:
        return conv(v)
    except ValueError:
        return default


def build_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(prog="python -m vt_transformer_amd", description="Qwen2 inference on one MI355X")
    p.add_argument("--model-path", "--model", dest="model", type=str, help="folder with config.json and model.safetensors")
    p.add_argument("--tokenizer-path", type=str, default="", help="folder or file of a tokenizer.json (default: the model folder)")
    p.add_argument("--model-name", type=str, default="vt_transformer_amd", help="name shown by the shell")
    p.add_argument("--shell-mode", action="store_true", help="interactive shell: a prompt per line, /reset, /exit")
    # (the reference's tool spells them fp16, bf16 and fp32: vt-transformer/models/qwen3-0.6b/tools/verify/reference.py:42-46, 75)
    p.add_argument("--dtype", choices=["bfloat16", "float16", "float32", "bf16", "fp16", "fp32"], default="bfloat16")
    # prompts
    p.add_argument("--prompt-ids", action="append", default=[], help="token ids, comma separated (may be repeated)")
    p.add_argument("--prompt-file", type=str, help="one prompt per line: token ids separated by commas or blanks")
    p.add_argument("--prompt", action="append", default=[], help="text (needs a tokenizer; may be repeated)")
    # sampling (sglfront/core.py)
    p.add_argument("--max-tokens", type=int, default=None)
    p.add_argument("--temperature", type=float, default=None)
    p.add_argument("--top-k", type=int, default=None)
    p.add_argument("--top-p", type=float, default=None)
    p.add_argument("--ignore-eos", action="store_true")
    p.add_argument("--seed", type=int, default=0)
    # scheduler (vt_scheduler.hpp)
    p.add_argument("--max-running-reqs", type=int, default=128)
    p.add_argument("--num-pages", type=int, default=None, help="cache pages per group of layers (default: for max-running-reqs/4 full sequences)")
    p.add_argument("--kv-bytes", type=int, default=None,
                   help="size of the cache in bytes, shared by all groups of layers (instead of --num-pages)")
    p.add_argument("--max-seq-len", type=int, default=4096)
    p.add_argument("--page-size", type=int, default=16)
    p.add_argument("--max-extend-tokens", type=int, default=8192)
    p.add_argument("--default-max-output", type=int, default=1024)
    p.add_argument("--chunk-size", type=int, default=2048)
    p.add_argument("--no-decode-graphs", action="store_true")
    p.add_argument("--tune-gemm", action="store_true", help="let the GEMM library search its algorithms at start-up (seconds)")
    p.add_argument("--single-weight-copy", action="store_true",
                   help="keep the bfloat16 matrices once instead of twice (half the memory, slower prompts)")
    # random weights
    p.add_argument("--plugin", action="append", default=[], metavar="FILE.py|MODULE",
                   help="code that registers further architectures or parts (may be repeated; also $VT_TRANSFORMER_PLUGINS)")
    p.add_argument("--write-random-model", type=str, metavar="DIR", help="write config.json and model.safetensors with random weights")
    p.add_argument("--config", type=str, help="config.json for --write-random-model")
    return p


def _load_tokenizer(path: str, model: Optional[str]):
    cands = [path] if path else []
    if model:
        cands.append(model)
    for c in cands:
        f = c if os.path.isfile(c) else os.path.join(c, "tokenizer.json")
        if os.path.isfile(f):
            from tokenizers import Tokenizer
            return Tokenizer.from_file(f)
    if path:
        raise SystemExit(f"no tokenizer.json at {path}")
    return None


def _parse_ids(text: str) -> List[int]:
    return [int(x) for x in text.replace(",", " ").split()]


def main(argv: Optional[List[str]] = None) -> int:
    args = build_parser().parse_args(argv)
    from .plugins import load_plugins
    load_plugins(args.plugin)
    if args.write_random_model:
        if not args.config:
            raise SystemExit("--write-random-model needs --config FILE")
        from .config import config_from_dict
        from .weights import write_random_model
        with open(args.config) as f:
            cfg = config_from_dict(json.load(f))
        write_random_model(cfg, args.write_random_model, args.seed)
        print(f"wrote {args.write_random_model}/config.json and model.safetensors (seed {args.seed})")
        return 0
    if not args.model:
        raise SystemExit("--model DIR is required")

    from .engine import Engine
    from .sampling import SamplingParams
    tok = _load_tokenizer(args.tokenizer_path, args.model)
    shell = args.shell_mode
    max_tokens = args.max_tokens if args.max_tokens is not None else (_env("SHELL_MAX_TOKENS", 2048, int) if shell else args.default_max_output)
    temperature = args.temperature if args.temperature is not None else (_env("SHELL_TEMPERATURE", 0.6, float) if shell else 0.0)
    top_k = args.top_k if args.top_k is not None else (_env("SHELL_TOP_K", -1, int) if shell else -1)
    top_p = args.top_p if args.top_p is not None else (_env("SHELL_TOP_P", 1.0, float) if shell else 1.0)
    if args.kv_bytes is not None and args.num_pages is not None:
        raise SystemExit("give --num-pages or --kv-bytes, not both")
    num_pages = args.num_pages or max(64, (args.max_seq_len // args.page_size) * max(1, args.max_running_reqs // 4))
    eng = Engine(args.model, dtype=args.dtype, seed=args.seed, max_running_reqs=args.max_running_reqs,
                 num_pages=num_pages, kv_bytes=args.kv_bytes, max_seq_len=args.max_seq_len, page_size=args.page_size,
                 max_extend_tokens=args.max_extend_tokens, default_max_output=args.default_max_output,
                 chunk_size=args.chunk_size, decode_graphs=not args.no_decode_graphs, tune_gemm=args.tune_gemm,
                 single_weight_copy=args.single_weight_copy)

    def params() -> SamplingParams:
        return SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, ignore_eos=args.ignore_eos,
                              max_tokens=max_tokens)

    def run(prompts: List[List[int]]) -> List[List[int]]:
        t0 = time.time()
        outs = eng.generate(prompts, params())
        n = sum(len(o) for o in outs)
        for o in outs:
            print(",".join(str(t) for t in o))
            if tok is not None:
                print(tok.decode(o))
        print(f"Generated {n} tokens, using {time.time() - t0:.3f} seconds")
        return outs

    if shell:
        print(f"{args.model_name}: a prompt per line ({'text' if tok else 'token ids'}); /reset (or !) forgets the history, /exit leaves")
        history: List[int] = []
        while True:
            try:
                line = input("$ ").strip()
            except EOFError:
                break
            if not line:
                continue
            if line == "/exit":
                break
            if line in ("/reset", "!"):
                history = []
                continue
            if line.startswith("/"):
                print(f"Unknown command: {line}")
                continue
            try:
                ids = tok.encode(line).ids if tok is not None else _parse_ids(line)
            except ValueError:
                print("token ids are whole numbers separated by commas or blanks")
                continue
            history = history + ids
            out = run([history])[0]
            history = history + out
        print("Exiting shell...")
        return 0

    prompts: List[List[int]] = [_parse_ids(p) for p in args.prompt_ids]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            prompts += [_parse_ids(line) for line in f if line.strip()]
    if args.prompt:
        if tok is None:
            raise SystemExit("--prompt needs a tokenizer.json (see --tokenizer-path); use --prompt-ids otherwise")
        prompts += [tok.encode(p).ids for p in args.prompt]
    if not prompts:
        raise SystemExit("nothing to do: give --prompt-ids, --prompt-file, --prompt or --shell-mode")
    run(prompts)
    return 0


if __name__ == "__main__":
    sys.exit(main())
