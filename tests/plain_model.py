"""Plain, slow implementation of the Qwen2 decoder, written from the
reference's formulas: whole sequences, no cache, one function per part, in
float64 on the CPU.  It shares no code with the engine; the tests compare
the engine against it.

Each function cites where the reference computes the same thing
(paths under the reference's root).
"""
from __future__ import annotations

import json
import math
import os
import struct
from typing import Dict, List, Optional

import numpy as np
import torch

DT = torch.float64


# ---------------------------------------------------------------------------
# reading a model folder (own reader: 8-byte length, JSON header, raw data;
# vt-transformer/core/safetensors.hpp:159-201)
# ---------------------------------------------------------------------------
def read_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    path = os.path.join(folder, "model.safetensors")
    with open(path, "rb") as f:
        (hlen,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hlen))
        data = f.read()
    tensors = {}
    for name, e in header.items():
        if name == "__metadata__":
            continue
        b, en = e["data_offsets"]
        raw = np.frombuffer(data, dtype=np.uint8, count=en - b, offset=b).copy()
        if e["dtype"] == "BF16":
            u = raw.view(np.uint16).astype(np.uint32) << 16
            arr = u.view(np.float32)
        elif e["dtype"] == "F32":
            arr = raw.view(np.float32)
        elif e["dtype"] == "F16":
            arr = raw.view(np.float16).astype(np.float32)
        else:
            raise ValueError(e["dtype"])
        tensors[name] = torch.from_numpy(arr.astype(np.float64)).reshape(e["shape"])
    return cfg, tensors


# ---------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------
def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """v1/tensortype/hip_kernels/rmsnorm.cpp:15-41: sum of squares / dim, + eps inside rsqrt, out = w*x*r."""
    ss = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return w * x * torch.rsqrt(ss + eps)


def linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """v1/tensortype/hip_tensor.cpp:479-539: y = x W^T with W [out, in]; bias added after
    (v1/tensortype/hip_kernels/add_bias.cpp:8-17)."""
    y = x @ w.t()
    return y + b if b is not None else y


def rotary_angles(positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """v1/tensortype/common.cpp:6-24: inv_freq[i/2] = 1/base^(i/dims) for even i; angle = position * inv_freq.
    [T, dims/2]"""
    i = torch.arange(0, dims, 2, dtype=DT, device=positions.device)
    inv = 1.0 / torch.pow(torch.tensor(base, dtype=DT, device=positions.device), i / dims)
    return positions.to(DT)[:, None] * inv[None, :]


def rotary(x: torch.Tensor, positions: torch.Tensor, base: float) -> torch.Tensor:
    """v1/tensortype/hip_kernels/rotary_embed.cpp:20-26: for i < D/2, ii = i + D/2:
    out[i] = cos*x[i] - sin*x[ii]; out[ii] = cos*x[ii] + sin*x[i] (both entries of a pair share the angle,
    common.cpp:10-14).  x: [T, heads, D]"""
    d = x.shape[-1]
    ang = rotary_angles(positions, d, base)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat([c * x1 - s * x2, c * x2 + s * x1], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: int = 0,
              positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, NH, D], k/v [T, KVH, D] -> [T, NH, D].
    Query head h reads kv head h // (NH/KVH) (v1/tensortype/hip_kernels/transpose_0213.cpp:89-103);
    scores scaled by 1/sqrt(D) (v1/tensortype/hip_tensor.cpp:691); key f allowed for new token t iff
    f <= position of t (v1/tensortype/hip_kernels/causal_mask.cpp:57-83); softmax over keys with the
    maximum subtracted (v1/tensortype/hip_kernels/softmax.cpp:10-43); weighted sum of values
    (hip_tensor.cpp:848-877).  window > 0: only the last `window` keys, the token's own included
    (not in the reference; the documented meaning of the checkpoint's sliding_window key)."""
    t, nh, d = q.shape
    kvh = k.shape[1]
    rep = nh // kvh
    out = torch.zeros_like(q)
    cols = torch.arange(t, device=q.device)
    # (rows in blocks of 2,048 so that a long sequence's score matrix need not exist all at once; every row still
    # sees the whole sequence)
    for r0 in range(0, t, 2048):
        rows = torch.arange(r0, min(t, r0 + 2048), device=q.device)
        allowed = cols[None, :] <= rows[:, None]
        if window > 0:
            allowed &= cols[None, :] > rows[:, None] - window
        for h in range(nh):
            kh, vh = k[:, h // rep, :], v[:, h // rep, :]
            s = (q[rows, h, :] @ kh.t()) / math.sqrt(d)
            s = torch.where(allowed, s, torch.tensor(float("-inf"), dtype=s.dtype, device=s.device))
            s = s - s.max(dim=-1, keepdim=True).values
            p = torch.exp(s)
            p = p / p.sum(dim=-1, keepdim=True)
            out[rows, h, :] = p @ vh
    return out


def swiglu(x: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """v1/models/qwen2-7b/inference_fp16.dag:333-337 with w1 = gate_proj, w2 = up_proj, o_proj = down_proj
    (v1/models/qwen2-7b/dump_from_huggingface.py:89-99); act/(1+exp(-act)) * up
    (v1/tensortype/hip_kernels/silu_product.cpp:8-16)."""
    g = linear(x, w_gate)
    u = linear(x, w_up)
    return linear(g / (1.0 + torch.exp(-g)) * u, w_down)


# ---------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------
def layer_window(cfg: dict, i: int) -> int:
    if not cfg.get("use_sliding_window", False):
        return 0
    first = cfg.get("max_window_layers")
    if first is None:
        first = cfg["num_hidden_layers"]
    return int(cfg["sliding_window"]) if i >= first else 0


def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: List[int], first_position: int = 0,
            device: Optional[str] = None) -> torch.Tensor:
    """Logits [T, V] of a whole sequence, float64.
    Order of v1/models/qwen2-7b/inference_fp16.dag:287-345 (layer) and :368-388 (outer program).
    device: where torch does the arithmetic (None: the tensors' own, the CPU; sequences of many thousands of
    tokens are given a GPU, still in float64 and with these same functions); the logits come back on the CPU."""
    if device is not None:
        w = {k: v.to(device) for k, v in w.items()}
    nh = cfg["num_attention_heads"]
    kvh = cfg.get("num_key_value_heads", nh)
    hidden = cfg["hidden_size"]
    d = cfg.get("head_dim") or hidden // nh
    eps = cfg.get("rms_norm_eps", 1e-6)
    base = cfg.get("rope_theta", 1000000.0)
    t = len(ids)
    dev = w["model.embed_tokens.weight"].device
    pos = torch.arange(first_position, first_position + t, device=dev)
    x = w["model.embed_tokens.weight"][torch.tensor(ids, dtype=torch.long, device=dev)]   # dag :372-375
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        a = rmsnorm(x, w[p + "input_layernorm.weight"], eps)                              # :290
        k = linear(a, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"])    # :296
        k = rotary(k.reshape(t, kvh, d), pos, base)                                       # :297
        q = linear(a, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"])    # :302
        q = rotary(q.reshape(t, nh, d), pos, base)                                        # :303
        v = linear(a, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"])    # :312
        o = attention(q, k, v.reshape(t, kvh, d), window=layer_window(cfg, i))            # :307-318
        x = x + linear(o.reshape(t, nh * d), w[p + "self_attn.o_proj.weight"])            # :322-323
        b = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)                     # :326
        x = x + swiglu(b, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],     # :333-340
                       w[p + "mlp.down_proj.weight"])
    x = rmsnorm(x, w["model.norm.weight"], eps)                                           # :383
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings", False) else w["lm_head.weight"]
    return linear(x, head).cpu()                                                          # :384-388


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    """argmax decoding by recomputing the whole sequence each step (dag :393, lowest index on ties)."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(cfg, w, ids)[-1]
        nxt = int(torch.argmax(logits))
        out.append(nxt)
        ids.append(nxt)
    return out
