"""Each part alone against the plain implementation's function for it; the order of layers as data; and parts
that the framework does not have (a mixer with state of its own, another position encoding), defined here,
registered, built and stepped without touching the framework's files."""
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_model as pm
from vt_transformer_amd.config.base import LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
TOL = {torch.float32: 5e-6, torch.bfloat16: 2e-2, torch.float16: 3e-3}


def rel(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def runtime(dtype):
    from vt_transformer_amd.parts import Runtime
    return Runtime(DEV, dtype)


def rand_weights(part, seed, scale=0.3):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, decl in part.tensors().items():
        t = torch.randn(decl.shape, generator=g) * scale
        if decl.role == "gain":
            t += 1.0
        out[name] = t.to(torch.bfloat16).float()       # representable in both dtypes
    return out


class OneMixer:
    """The least a ModelRunner needs to give a single mixer a cache and a context."""

    def __init__(self, mixer, vocab=100):
        self.schedule = [ScheduleEntry(0)]
        self.layers = [SimpleNamespace(mixer=mixer)]
        self.spec = SimpleNamespace(vocab_size=vocab)


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_rmsnorm_part(dtype):
    from vt_transformer_amd.parts import NORMS
    rt = runtime(dtype)
    norm = NORMS.build(PartSpec("rmsnorm", {"eps": 1e-5, "name": "ln.weight"}), rt=rt, width=200, prefix="x.")
    w = rand_weights(norm, 1)
    assert list(w) == ["x.ln.weight"]
    norm.load(w.__getitem__, rt)
    g = torch.Generator().manual_seed(2)
    h, delta = torch.randn(6, 200, generator=g), torch.randn(6, 200, generator=g).to(dtype)
    hd = h.to(DEV)
    out = norm.forward(hd, delta.to(DEV))
    x = h.double() + delta.double()
    assert rel(out, pm.rmsnorm(x, w["x.ln.weight"].double(), 1e-5)) < TOL[dtype]
    assert rel(hd, x) < 1e-6                                       # the residual stream took the sum, in fp32


def test_rotary_part_tables():
    from vt_transformer_amd.parts import POSITIONS
    rot = POSITIONS.build(PartSpec("rotary", {"theta": 1e6, "dim": 48}), rt=runtime(torch.float32))
    cos, sin = rot.rotary_tables(300)
    ang = pm.rotary_angles(torch.arange(300), 48, 1e6)
    assert cos.shape == (300, 24)
    assert float((cos.cpu().double() - torch.cos(ang)).abs().max()) < 1e-7   # double angles, one rounding to float
    assert float((sin.cpu().double() - torch.sin(ang)).abs().max()) < 1e-7


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("nh,kvh,d,window", [(6, 2, 32, 0), (5, 5, 16, 7), (4, 1, 64, 0)])
def test_attention_part(dtype, nh, kvh, d, window):
    from vt_transformer_amd.engine.step import ModelRunner, StepEntry
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width = 72
    mixer = MIXERS.build(PartSpec("attention", dict(num_heads=nh, num_kv_heads=kvh, head_dim=d, qkv_bias=True,
                                                    window=window, position=PartSpec("rotary", {"theta": 1e4, "dim": d}))),
                         rt=rt, width=width, prefix="a.", shared={})
    w = rand_weights(mixer, 3)
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 4, 256)
    t = 45
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(4)) * 0.5).to(dtype)
    runner.admit("r")
    outs = []
    for a, b in [(0, 20), (20, 21), (21, 45)]:       # a portion, one token, another portion
        assert runner.cache.reserve([("r", b)])
        ctx = runner.build_context([StepEntry("r", [0] * (b - a), [])])
        cache = runner.storage.layer_caches(ctx.block_tables)[0]
        outs.append(mixer.forward(x[a:b].to(DEV).contiguous(), ctx, cache).float().cpu().clone())
        runner.cache.commit("r", b)
    got = torch.cat(outs)
    xd = x.double()
    wd = {k: v.double() for k, v in w.items()}
    pos = torch.arange(t)
    q = pm.rotary(pm.linear(xd, wd["a.q_proj.weight"], wd["a.q_proj.bias"]).reshape(t, nh, d), pos, 1e4)
    k = pm.rotary(pm.linear(xd, wd["a.k_proj.weight"], wd["a.k_proj.bias"]).reshape(t, kvh, d), pos, 1e4)
    v = pm.linear(xd, wd["a.v_proj.weight"], wd["a.v_proj.bias"]).reshape(t, kvh, d)
    ref = pm.linear(pm.attention(q, k, v, window=window).reshape(t, nh * d), wd["a.o_proj.weight"])
    assert rel(got, ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [3, 100])
def test_gated_mlp_part(dtype, n):
    from vt_transformer_amd.parts import FEED_FORWARDS
    rt = runtime(dtype)
    ffn = FEED_FORWARDS.build(PartSpec("gated_mlp", {"intermediate_size": 200}), rt=rt, width=96, prefix="m.")
    w = rand_weights(ffn, 5, scale=0.2)
    ffn.load(w.__getitem__, rt)
    x = torch.randn(n, 96, generator=torch.Generator().manual_seed(6)).to(dtype)
    got = ffn.forward(x.to(DEV))
    wd = {k: v.double() for k, v in w.items()}
    ref = pm.swiglu(x.double(), wd["m.gate_proj.weight"], wd["m.up_proj.weight"], wd["m.down_proj.weight"])
    assert rel(got, ref) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_embedding_and_head_parts(dtype):
    from vt_transformer_amd.parts import EMBEDDINGS, HEADS
    rt = runtime(dtype)
    emb = EMBEDDINGS.build(PartSpec("embedding", {"name": "wte"}), rt=rt, width=80, vocab_size=203)
    head = HEADS.build(PartSpec("linear_head", {"name": "head", "tied_to": None}), rt=rt, width=80, vocab_size=203)
    tied = HEADS.build(PartSpec("linear_head", {"name": "head", "tied_to": "wte"}), rt=rt, width=80, vocab_size=203)
    w = {**rand_weights(emb, 7), **rand_weights(head, 8)}
    emb.load(w.__getitem__, rt)
    head.load(w.__getitem__, rt)
    tied.load(w.__getitem__, rt, shared={"wte": emb.table})
    ids = torch.tensor([5, 202, 0, 77], dtype=torch.int32)
    h = emb.forward(ids.to(DEV))
    assert torch.equal(h.cpu(), w["wte"][ids.long()])
    x = torch.randn(70, 80, generator=torch.Generator().manual_seed(9)).to(dtype)
    assert rel(head.forward(x.to(DEV)), x.double() @ w["head"].double().t()) < TOL[dtype]
    assert rel(tied.forward(x.to(DEV)), x.double() @ w["wte"].double().t()) < TOL[dtype]
    assert head.forward(x.to(DEV)).dtype == torch.float32          # logits stay in 32-bit


# ---------------------------------------------------------------------------
# the order of layers is data: a layer named twice, an entry that reads another entry's cache
# ---------------------------------------------------------------------------
def qwen_like_spec(schedule):
    from conftest import TINY_A
    from vt_transformer_amd.config import config_from_dict
    spec = config_from_dict(dict(TINY_A, tie_word_embeddings=False)).to_spec()
    return ModelSpec(**{**spec.__dict__, "schedule": schedule})


def plain_scheduled(cfg, w, ids, schedule):
    """plain_model.forward with the run order given as data (float64)."""
    nh, kvh, hidden = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["hidden_size"]
    d, eps, base, t = cfg["head_dim"], cfg["rms_norm_eps"], cfg["rope_theta"], len(ids)
    pos = torch.arange(t)
    x = w["model.embed_tokens.weight"][torch.tensor(ids)]
    kept = {}
    for i, e in enumerate(schedule):
        p = f"model.layers.{e.layer}."
        a = pm.rmsnorm(x, w[p + "input_layernorm.weight"], eps)
        q = pm.rotary(pm.linear(a, w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"]).reshape(t, nh, d), pos, base)
        if e.cache_from is None:
            k = pm.rotary(pm.linear(a, w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"]).reshape(t, kvh, d), pos, base)
            v = pm.linear(a, w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"]).reshape(t, kvh, d)
            kept[i] = (k, v)
        else:
            k, v = kept[e.cache_from]
        x = x + pm.linear(pm.attention(q, k, v).reshape(t, nh * d), w[p + "self_attn.o_proj.weight"])
        b = pm.rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + pm.swiglu(b, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return pm.linear(pm.rmsnorm(x, w["model.norm.weight"], eps), w["lm_head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
def test_run_order_is_data(dtype):
    from conftest import TINY_A
    from vt_transformer_amd.engine import StepEntry, make_runner, parse_dtype
    from vt_transformer_amd.models import DecoderModel
    from vt_transformer_amd.parts import Runtime
    from vt_transformer_amd.weights import random_tensor
    schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1), ScheduleEntry(0, cache_from=0), ScheduleEntry(1, cache_from=2)]
    spec = qwen_like_spec(schedule)
    model = DecoderModel(spec, Runtime(DEV, parse_dtype(dtype)))
    decl = model.tensors()
    w = {n: random_tensor(n, d, 11, torch.device("cpu"), torch.bfloat16).float() * (4.0 if d.role == "matrix" else 1.0)
         for n, d in decl.items()}
    w = {n: t.to(torch.bfloat16).float() for n, t in w.items()}
    model.load(w.__getitem__)
    runner = make_runner(model, pool_tokens=128, page_size=16, max_requests=2, max_seq_len=128)
    # three entries keep pages (0, 1, 2), two read another's: one group of three layers' worth of pages
    assert runner.storage.pages[0]["k"].shape[0] == 3 and runner.storage.writes == [True, True, True, False, False]
    ids = np.random.RandomState(0).randint(0, TINY_A["vocab_size"], size=41).tolist()
    runner.admit("r")
    got = []
    for a, b in [(0, 17), (17, 18), (18, 41)]:
        got.append(runner.step([StepEntry("r", ids[a:b], list(range(b - a)))]).cpu())
    ref = plain_scheduled(dict(TINY_A), {n: t.double() for n, t in w.items()}, ids, schedule)
    assert rel(torch.cat(got), ref) < {"float32": 2e-5, "bfloat16": 1.5e-2, "float16": 2e-3}[dtype]


# ---------------------------------------------------------------------------
# parts of the test's own: a mixer with per-request state, another position encoding, a feed-forward with routing
# ---------------------------------------------------------------------------
def register_toy_parts():
    from vt_transformer_amd.parts import FEED_FORWARDS, MIXERS, POSITIONS, Part, StateNeed, TensorDecl

    @FEED_FORWARDS.register("toy_routed")
    class ToyRouted(Part):
        """Every token goes to the one expert (a matrix) whose router logit is largest, weighted by the softmax
        of the router's logits."""

        def __init__(self, *, rt, width, prefix, experts):
            self.rt, self.width, self.experts, self.prefix = rt, width, int(experts), prefix

        def tensors(self):
            t = {self.prefix + "router.weight": TensorDecl((self.experts, self.width), "matrix")}
            for e in range(self.experts):
                t[f"{self.prefix}experts.{e}.weight"] = TensorDecl((self.width, self.width), "matrix")
            return t

        def load(self, get, rt):
            self.router = rt.place(get(self.prefix + "router.weight"), "matrix").float()
            self.w = torch.stack([rt.place(get(f"{self.prefix}experts.{e}.weight"), "matrix").float()
                                  for e in range(self.experts)])

        def forward(self, x, ctx=None):
            xf = x.float()
            p = torch.softmax(xf @ self.router.t(), dim=-1)
            top = p.argmax(dim=-1)
            y = torch.einsum("tk,tmk->tm", xf, self.w[top]) * p.gather(1, top[:, None])
            return y.to(x.dtype)

    @MIXERS.register("toy_decay")
    class ToyDecay(Part):
        """s_t = decay * s_{t-1} + x_t per request (state carried between steps); y_t = s_t W^T."""

        def __init__(self, *, rt, width, prefix, decay, shared=None):
            self.rt, self.width, self.decay, self.name = rt, width, float(decay), prefix + "mix.weight"

        def cache_need(self):
            return None

        def state_need(self):
            return StateNeed((self.width,), torch.float32)

        def tensors(self):
            return {self.name: TensorDecl((self.width, self.width), "matrix")}

        def load(self, get, rt):
            self.w = rt.place(get(self.name), "matrix").float()

        def forward(self, x, ctx, cache, state):
            out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
            for e in range(ctx.n_entries):
                slot = int(ctx.h_state_slots[e])
                s = state[slot]
                for t in range(int(ctx.h_entry_start[e]), int(ctx.h_entry_start[e + 1])):
                    s = self.decay * s + x[t].float()
                    out[t] = s @ self.w.t()
                state[slot] = s
            return out.to(x.dtype)

    @MIXERS.register("toy_latent")
    class ToyLatent(Part):
        """Attention over one latent vector per token: c_t = x_t Wd^T is what the pages keep (one tensor, float32
        whatever the runtime's dtype, [slot][rank]); y_t = softmax_s<=t(q_t . c_s / sqrt(rank)) c_s Wu^T with
        q_t = x_t Wq^T.  The page's layout is this mixer's own: the cache manager allocates what cache_need() lists."""

        def __init__(self, *, rt, width, prefix, rank, shared=None):
            self.rt, self.width, self.rank, self.prefix = rt, width, int(rank), prefix

        def cache_need(self):
            from vt_transformer_amd.parts import CacheNeed, PageTensor
            return CacheNeed((PageTensor("latent", (self.rank,), 0, torch.float32),))

        def state_need(self):
            return None

        def tensors(self):
            return {self.prefix + "down.weight": TensorDecl((self.rank, self.width), "matrix"),
                    self.prefix + "q.weight": TensorDecl((self.rank, self.width), "matrix"),
                    self.prefix + "up.weight": TensorDecl((self.width, self.rank), "matrix")}

        def load(self, get, rt):
            self.wd, self.wq, self.wu = (rt.place(get(self.prefix + n + ".weight"), "matrix").float() for n in ("down", "q", "up"))

        def forward(self, x, ctx, cache, state):
            pages = cache["latent"]                              # [pages][slot][rank]
            ps = pages.shape[1]
            xf = x.float()
            c, q = xf @ self.wd.t(), xf @ self.wq.t()
            pos, ent = ctx.positions.long(), ctx.tok_entry.long()
            page = cache.block_table[ent, pos // ps].long()
            pages[page, pos % ps] = c                            # this step's tokens into their slots
            out = torch.empty(x.shape[0], self.width, dtype=torch.float32, device=x.device)
            for e in range(ctx.n_entries):
                t0, t1, p0 = int(ctx.h_entry_start[e]), int(ctx.h_entry_start[e + 1]), int(ctx.h_entry_pos0[e])
                n_keys = p0 + (t1 - t0)
                lat = pages[cache.block_table[e, :-(-n_keys // ps)].long()].reshape(-1, self.rank)[:n_keys]
                sc = (q[t0:t1] @ lat.t()) / math.sqrt(self.rank)
                seen = torch.arange(n_keys, device=x.device)[None, :] <= (p0 + torch.arange(t1 - t0, device=x.device))[:, None]
                out[t0:t1] = (torch.softmax(sc.masked_fill(~seen, float("-inf")), dim=-1) @ lat) @ self.wu.t()
            return out.to(x.dtype)

    @POSITIONS.register("toy_offset")
    class ToyOffset(Part):
        """Not a rotation: adds position * slope to the first dim of queries and keys."""

        def __init__(self, *, rt, slope):
            self.rt, self.slope, self.dim = rt, float(slope), 1

        def rotary_tables(self, n_positions):
            return None

        def apply(self, q, k, positions):
            add = positions.float() * self.slope
            q = q.clone()
            q[:, :, 0] += add[:, None].to(q.dtype)
            if k is not None:
                k = k.clone()
                k[:, :, 0] += add[:, None].to(k.dtype)
            return q, k


class ToyConfig(ModelConfig):
    architecture = "ToyStateForCausalLM"

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(d)

    def to_dict(self):
        return dict(self.d)

    def to_spec(self):
        d = self.d
        norm = lambda name: PartSpec("rmsnorm", {"eps": d["eps"], "name": name})
        layers = []
        for i in range(d["n_layer"]):
            if i % 2 == 0:
                mixer = PartSpec("toy_decay", {"decay": d["decay"], "prefix": "toy."})
            else:
                mixer = PartSpec("attention", {"num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "prefix": "attn.",
                                               "position": PartSpec("toy_offset", {"slope": d["slope"]})})
            if i % 4 == 3:
                ffn = PartSpec("toy_routed", {"experts": d["experts"], "prefix": "moe."})
            else:
                ffn = PartSpec("gated_mlp", {"intermediate_size": d["inter"], "prefix": "ffn."})
            layers.append(LayerSpec(PartSpec("prenorm", {}), mixer, ffn,
                                    {"input": norm("n1.weight"), "post_mixer": norm("n2.weight")}, f"blocks.{i}."))
        return ModelSpec("ToyStateForCausalLM", d["vocab"], d["width"], PartSpec("embedding", {"name": "emb.weight"}),
                         layers, [ScheduleEntry(i) for i in range(d["n_layer"])], norm("final.weight"),
                         PartSpec("linear_head", {"name": "emb.weight", "tied_to": "emb.weight"}), 256)


class ToyLatentConfig(ModelConfig):
    """Layers that keep one latent vector per token beside layers of grouped-query attention: two groups of pages
    with different contents."""
    architecture = "ToyLatentForCausalLM"

    def __init__(self, d):
        self.d = d

    @classmethod
    def from_dict(cls, d):
        return cls(d)

    def to_dict(self):
        return dict(self.d)

    def to_spec(self):
        d = self.d
        norm = lambda name: PartSpec("rmsnorm", {"eps": d["eps"], "name": name})
        layers = []
        for i in range(d["n_layer"]):
            if i % 2 == 0:
                mixer = PartSpec("toy_latent", {"rank": d["rank"], "prefix": "lat."})
            else:
                mixer = PartSpec("attention", {"num_heads": 2, "num_kv_heads": 1, "head_dim": 16, "prefix": "attn."})
            layers.append(LayerSpec(PartSpec("prenorm", {}), mixer,
                                    PartSpec("gated_mlp", {"intermediate_size": d["inter"], "prefix": "ffn."}),
                                    {"input": norm("n1.weight"), "post_mixer": norm("n2.weight")}, f"blocks.{i}."))
        return ModelSpec("ToyLatentForCausalLM", d["vocab"], d["width"], PartSpec("embedding", {"name": "emb.weight"}),
                         layers, [ScheduleEntry(i) for i in range(d["n_layer"])], norm("final.weight"),
                         PartSpec("linear_head", {"name": "emb.weight", "tied_to": "emb.weight"}), 256)


def toy_latent_plain(d, w, ids):
    """The latent toy model whole, float64."""
    t = len(ids)
    x = w["emb.weight"][torch.tensor(ids)]
    causal = torch.tril(torch.ones(t, t, dtype=torch.bool))
    for i in range(d["n_layer"]):
        p = f"blocks.{i}."
        a = pm.rmsnorm(x, w[p + "n1.weight"], d["eps"])
        if i % 2 == 0:
            c, q = a @ w[p + "lat.down.weight"].t(), a @ w[p + "lat.q.weight"].t()
            sc = (q @ c.t() / math.sqrt(d["rank"])).masked_fill(~causal, float("-inf"))
            y = (torch.softmax(sc, dim=-1) @ c) @ w[p + "lat.up.weight"].t()
        else:
            q = pm.linear(a, w[p + "attn.q_proj.weight"]).reshape(t, 2, 16)
            k = pm.linear(a, w[p + "attn.k_proj.weight"]).reshape(t, 1, 16)
            v = pm.linear(a, w[p + "attn.v_proj.weight"]).reshape(t, 1, 16)
            y = pm.linear(pm.attention(q, k, v).reshape(t, 32), w[p + "attn.o_proj.weight"])
        x = x + y
        b = pm.rmsnorm(x, w[p + "n2.weight"], d["eps"])
        x = x + pm.swiglu(b, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
    return pm.rmsnorm(x, w["final.weight"], d["eps"]) @ w["emb.weight"].t()


def toy_plain(d, w, ids):
    """The toy model whole, float64."""
    t = len(ids)
    pos = torch.arange(t)
    x = w["emb.weight"][torch.tensor(ids)]
    for i in range(d["n_layer"]):
        p = f"blocks.{i}."
        a = pm.rmsnorm(x, w[p + "n1.weight"], d["eps"])
        if i % 2 == 0:
            s = torch.zeros(d["width"], dtype=torch.float64)
            ys = []
            for j in range(t):
                s = d["decay"] * s + a[j]
                ys.append(s @ w[p + "toy.mix.weight"].t())
            y = torch.stack(ys)
        else:
            q = pm.linear(a, w[p + "attn.q_proj.weight"]).reshape(t, 2, 16)
            k = pm.linear(a, w[p + "attn.k_proj.weight"]).reshape(t, 1, 16)
            v = pm.linear(a, w[p + "attn.v_proj.weight"]).reshape(t, 1, 16)
            q[:, :, 0] += (pos.double() * d["slope"])[:, None]
            k[:, :, 0] += (pos.double() * d["slope"])[:, None]
            y = pm.linear(pm.attention(q, k, v).reshape(t, 32), w[p + "attn.o_proj.weight"])
        x = x + y
        b = pm.rmsnorm(x, w[p + "n2.weight"], d["eps"])
        if i % 4 == 3:
            pr = torch.softmax(b @ w[p + "moe.router.weight"].t(), dim=-1)
            top = pr.argmax(dim=-1)
            x = x + torch.stack([(w[f"{p}moe.experts.{int(top[j])}.weight"] @ b[j]) * pr[j, top[j]] for j in range(t)])
        else:
            x = x + pm.swiglu(b, w[p + "ffn.gate_proj.weight"], w[p + "ffn.up_proj.weight"], w[p + "ffn.down_proj.weight"])
    return pm.rmsnorm(x, w["final.weight"], d["eps"]) @ w["emb.weight"].t()


def test_toy_mixer_with_state_toy_position_encoding_and_toy_routing():
    """Registered here, built by the framework's model builder from a spec, stepped by its step function in
    portions and beside another request, with the state slot cleared when a slot is used again."""
    from vt_transformer_amd.config import config_from_dict, register_architecture
    from vt_transformer_amd.engine import StepEntry, build_model, make_runner
    from vt_transformer_amd.weights import random_tensor
    register_toy_parts()
    register_architecture("ToyStateForCausalLM", ToyConfig)
    d = {"architectures": ["ToyStateForCausalLM"], "n_layer": 4, "width": 48, "inter": 64, "vocab": 90, "eps": 1e-6,
         "decay": 0.9, "slope": 0.01, "experts": 3}
    cfg = config_from_dict(d)
    assert isinstance(cfg, ToyConfig)
    model = build_model(cfg, "float32")
    w = {n: random_tensor(n, dc, 3, torch.device("cpu"), torch.float32) * (3.0 if dc.role == "matrix" else 1.0)
         for n, dc in model.tensors().items()}
    model.load(w.__getitem__)
    runner = make_runner(model, pool_tokens=128, page_size=16, max_requests=2, max_seq_len=128)
    assert [s is not None for s in runner.storage.state] == [True, False, True, False]    # state slots for the toy
    assert runner.storage.state[0].shape == (2, 48)
    assert runner.storage.n_groups == 1 and runner.storage.pages[0]["k"].shape[0] == 2               # pages for attention only
    wd = {n: t.double() for n, t in w.items()}
    rs = np.random.RandomState(1)
    a, b, c = (rs.randint(0, 90, size=n).tolist() for n in (30, 21, 12))
    ra, rb, rc = toy_plain(d, wd, a), toy_plain(d, wd, b), toy_plain(d, wd, c)
    runner.admit("a"); runner.admit("b")
    got_a, got_b = [], []
    plan = [((0, 7), (0, 1)), ((7, 9), (1, 2)), ((9, 10), (2, 19)), ((10, 30), (19, 21))]
    for (a0, a1), (b0, b1) in plan:
        out = runner.step([StepEntry("a", a[a0:a1], list(range(a1 - a0))), StepEntry("b", b[b0:b1], list(range(b1 - b0)))]).cpu()
        got_a.append(out[:a1 - a0]); got_b.append(out[a1 - a0:])
    assert rel(torch.cat(got_a), ra) < 2e-5 and rel(torch.cat(got_b), rb) < 2e-5
    runner.release("a")
    runner.admit("c")                                   # takes a's slot: its state must start from zero again
    assert runner.cache.get("c").slot == 0
    got_c = runner.step([StepEntry("c", c, list(range(12)))]).cpu()
    assert rel(got_c, rc) < 2e-5
    assert not runner._stateless and not runner._replayable     # such a model is never replayed from a captured graph


def test_the_toy_architecture_through_the_engine_with_preemption():
    """The mixer with state of its own through Engine.generate (scheduler, sampler, no captured steps and no decoding
    ahead, since its steps cannot be replayed), with three pages for two requests: the younger one is preempted when
    both need a second page, gives its state slot back, and is recomputed later from its prompt and what it had
    produced, into a slot that starts from zero again.  Both end with the tokens they get alone."""
    from vt_transformer_amd.config import config_from_dict, register_architecture
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    register_toy_parts()
    register_architecture("ToyStateForCausalLM", ToyConfig)
    d = {"architectures": ["ToyStateForCausalLM"], "n_layer": 4, "width": 48, "inter": 64, "vocab": 90, "eps": 1e-6,
         "decay": 0.9, "slope": 0.01, "experts": 3}
    rs = np.random.RandomState(4)
    prompts = [rs.randint(0, 90, size=n).tolist() for n in (10, 9)]
    sp = SamplingParams(max_tokens=14, ignore_eos=True)
    eng = Engine(config=config_from_dict(d), random_weights_seed=5, dtype="float32", num_pages=3, max_running_reqs=2,
                 max_seq_len=64)
    assert not eng.runner.replays(2)
    outs = eng.generate(prompts, sp)
    assert [eng.finish_reason(i) for i in (0, 1)] == ["max_tokens"] * 2
    assert eng.requests[1].preemptions > 0 and eng.requests[0].preemptions == 0
    assert sum(eng.runner.cache.held_pages()) == 0 and eng.runner.cache.slots.available == 2
    alone = Engine(config=config_from_dict(d), random_weights_seed=5, dtype="float32", num_pages=4, max_running_reqs=1,
                   max_seq_len=64)
    assert outs == [alone.generate(p, sp)[0] for p in prompts]


def test_a_plugin_file_brings_an_architecture_to_the_replay_program(tmp_path):
    """A model folder of an architecture that the package does not know, written with random weights, replayed by
    bin/trace_run through its loader, cache (pages and state slots), step function and kernels: all it takes is a
    file that registers the architecture and its parts, named on the command line."""
    import os
    from replay_helpers import cut, max_live_tokens, random_requests, run_trace_run, trace_mixed
    from vt_transformer_amd.config import config_from_dict, register_architecture
    from vt_transformer_amd.weights import write_random_model
    register_toy_parts()
    register_architecture("ToyStateForCausalLM", ToyConfig)
    d = {"architectures": ["ToyStateForCausalLM"], "n_layer": 4, "width": 48, "inter": 64, "vocab": 90, "eps": 1e-6,
         "decay": 0.9, "slope": 0.01, "experts": 3}
    folder = write_random_model(config_from_dict(d), str(tmp_path / "toy"), seed=4, dtype=torch.float32)
    plugin = tmp_path / "toy_plugin.py"
    plugin.write_text(
        "import sys\n"
        f"sys.path.insert(0, {os.path.dirname(os.path.abspath(__file__))!r})\n"
        "import test_parts_gpu as toy\n"
        "from vt_transformer_amd.config import register_architecture\n"
        "toy.register_toy_parts()\n"
        "register_architecture('ToyStateForCausalLM', toy.ToyConfig)\n")
    reqs = random_requests(d["vocab"], [23, 9, 31, 14, 18], seed=5)
    portions = {r: cut(t, [5, 2, 7, 1]) for r, t in reqs.items()}
    steps = trace_mixed(reqs, portions, max_live=3, seed=6)
    got = run_trace_run(folder, "float32", steps, str(tmp_path / "out"), max_live_tokens(steps), d["vocab"],
                        extra_args=("--plugin", str(plugin)))
    _, w = pm.read_folder(folder)
    ref = {r: toy_plain(d, w, t) for r, t in reqs.items()}
    pos = {r: 0 for r in reqs}
    for s in steps:
        row = 0
        for e in s["entries"]:
            for j in e["want"]:
                want = ref[e["id"]][pos[e["id"]] + j]
                assert rel(torch.from_numpy(got[s["step"]][row].copy()), want) < 2e-5, (s["step"], e["id"], j)
                row += 1
            pos[e["id"]] += len(e["tokens"])


def test_a_mixer_that_keeps_one_latent_vector_per_token_in_pages_of_its_own(tmp_path):
    """What a page holds is the mixer's own affair: a mixer defined here keeps one float32 vector per token,
    [slot][rank], beside attention layers that keep keys and values of another shape in the runtime's dtype.  Written
    as a model folder and replayed by bin/trace_run in mixed steps with so few pages that they are used again, with
    nothing but a plugin file (no change under the package's cache or engine folders); and in-process in bfloat16."""
    import os
    from replay_helpers import cut, max_live_tokens, random_requests, run_in_process, run_trace_run, trace_mixed
    from vt_transformer_amd.config import config_from_dict, register_architecture
    from vt_transformer_amd.engine import load_model, make_runner
    from vt_transformer_amd.weights import write_random_model
    register_toy_parts()
    register_architecture("ToyLatentForCausalLM", ToyLatentConfig)
    d = {"architectures": ["ToyLatentForCausalLM"], "n_layer": 4, "width": 48, "inter": 64, "vocab": 90, "eps": 1e-6,
         "rank": 24}
    folder = write_random_model(config_from_dict(d), str(tmp_path / "toy"), seed=9, dtype=torch.float32)
    # larger projections, so that the scores differ and a latent vector read from a wrong slot would show
    from vt_transformer_amd.weights.safetensors_io import WeightStore, write_safetensors
    store = WeightStore(folder)
    tensors = [(n, store.get(n).float() * (8.0 if ".lat." in n or "_proj" in n else 1.0)) for n in store.names()]
    store.close()
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    plugin = tmp_path / "toy_plugin.py"
    plugin.write_text(
        "import sys\n"
        f"sys.path.insert(0, {os.path.dirname(os.path.abspath(__file__))!r})\n"
        "import test_parts_gpu as toy\n"
        "from vt_transformer_amd.config import register_architecture\n"
        "toy.register_toy_parts()\n"
        "register_architecture('ToyLatentForCausalLM', toy.ToyLatentConfig)\n")
    reqs = random_requests(d["vocab"], [23, 9, 31, 14, 18, 40], seed=5)
    portions = {r: cut(t, [5, 2, 7, 1]) for r, t in reqs.items()}
    steps = trace_mixed(reqs, portions, max_live=3, seed=6)
    _, w = pm.read_folder(folder)
    ref = {r: toy_latent_plain(d, w, t) for r, t in reqs.items()}

    def check(got, tol):
        pos = {r: 0 for r in reqs}
        for s in steps:
            row = 0
            for e in s["entries"]:
                for j in e["want"]:
                    want = ref[e["id"]][pos[e["id"]] + j]
                    assert rel(torch.from_numpy(got[s["step"]][row].copy()), want) < tol, (s["step"], e["id"], j)
                    row += 1
                pos[e["id"]] += len(e["tokens"])
    check(run_trace_run(folder, "float32", steps, str(tmp_path / "out"), max_live_tokens(steps), d["vocab"],
                        extra_args=("--plugin", str(plugin))), 2e-5)
    model = load_model(folder, "bfloat16")
    runner = make_runner(model, pool_tokens=max_live_tokens(steps), page_size=16, max_requests=3, max_seq_len=128)
    assert runner.storage.n_groups == 2
    assert set(runner.storage.pages[0]) == {"latent"} and runner.storage.pages[0]["latent"].dtype == torch.float32
    assert runner.storage.pages[0]["latent"].shape[2:] == (16, 24) and set(runner.storage.pages[1]) == {"k", "v"}
    # (scores of ten and more, rounded to bfloat16 on their way: a few per cent on the weights; a latent vector read
    # from a wrong slot moves a row by its whole size)
    check(run_in_process(runner, steps), 8e-2)
    assert sum(runner.cache.held_pages()) == 0
