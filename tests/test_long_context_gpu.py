"""Contexts of many thousands of tokens, checked: 8,192 (the context that the bench times, four portions of 2,048
and then token by token) and beyond 20,000 (block tables of more than a thousand entries, decoding with every
entry's keys cut into sixteen ranges, 2,048-token portions behind tens of thousands of cached keys), in float32 and
bfloat16, against the plain implementation run in float64 on the GPU.

The reference stops at 4,096 (MAX_CONTEXT, v1/models/qwen2-7b/inference_fp16.dag:14; its softmax kernel takes
fewer than 8,192 keys, v1/tensortype/hip_kernels/softmax.cpp:111).

With N(0, 0.02) weights the scores of a small model are nearly equal, every key gets 1/T of the weight, and a block
of keys that went missing or was read from the wrong page would change the result by less than bfloat16 rounds
away.  The query and key projections are therefore scaled up so that scores spread over several units: each row's
weight then sits on a few keys that lie anywhere in the context."""
import os

import numpy as np
import pytest
import torch

import plain_model
from replay_helpers import random_requests

pytestmark = pytest.mark.gpu

LONG = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=320, hidden_size=128,
            intermediate_size=256, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, head_dim=128,
            rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=32768,
            hidden_act="silu", use_sliding_window=False, torch_dtype="bfloat16")
QK_SCALE = 6.0
# about twice the worst error seen (relative to a row's largest logit): 1.1e-6 in float32, 7.3e-3 in bfloat16
TOL = {"float32": 3e-6, "bfloat16": 1.5e-2, "float16": 2e-3}


@pytest.fixture(scope="module")
def long_folder(tmp_path_factory):
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights.random_init import declared_tensors, random_tensor
    from vt_transformer_amd.weights.safetensors_io import write_safetensors
    cfg = config_from_dict(dict(LONG))
    folder = str(tmp_path_factory.mktemp("long") / "m")
    os.makedirs(folder)
    cfg.save(folder)

    def tensors():
        for name, decl in declared_tensors(cfg).items():
            if decl.optional:
                continue
            t = random_tensor(name, decl, 11, torch.device("cpu"), torch.bfloat16)
            if "q_proj" in name or "k_proj" in name:
                t = (t.float() * QK_SCALE).to(torch.bfloat16)
            yield name, t
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors(), metadata={"format": "pt"})
    return folder


_ref = {}


def reference(folder, toks):
    key = (folder, len(toks), toks[0], toks[-1])
    if key not in _ref:
        cfg, w = plain_model.read_folder(folder)
        _ref[key] = plain_model.forward(cfg, w, toks, device="cuda").numpy()
    return _ref[key]


def test_the_long_model_spreads_its_weight_over_far_keys(long_folder):
    """What makes the comparisons below mean something: in the plain model the last row's logits change by far more
    than the tolerance when 64 tokens in the middle of its context are replaced by others (positions stay: what
    changes is only what the later rows read from those keys and values)."""
    cfg, w = plain_model.read_folder(long_folder)
    toks = random_requests(LONG["vocab_size"], [6000], seed=5)["r0"]
    other = list(toks)
    other[3000:3064] = [(t + 1) % LONG["vocab_size"] for t in toks[3000:3064]]
    full = plain_model.forward(cfg, w, toks, device="cuda")[-1]
    changed = plain_model.forward(cfg, w, other, device="cuda")[-1]
    effect = float((full - changed).abs().max() / full.abs().max())
    print(f"effect of 64 far tokens among 6,000 on the last row: {effect:.3e}")
    assert effect > 2.5 * TOL["bfloat16"], effect


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("n_long", [8192, 20480])
def test_long_context_in_portions_then_token_by_token_beside_another_prompt(long_folder, dtype, n_long):
    from vt_transformer_amd.engine import StepEntry, load_model, make_runner
    vocab = LONG["vocab_size"]
    a = random_requests(vocab, [n_long + 32], seed=n_long)["r0"]
    b = random_requests(vocab, [2048 + 6], seed=n_long + 1)["r0"]
    ref_a, ref_b = reference(long_folder, a), reference(long_folder, b)
    model = load_model(long_folder, dtype)
    runner = make_runner(model, pool_tokens=n_long + 64 + 2112, page_size=16, max_requests=4, max_seq_len=32768)
    runner.decode_graphs = True
    worst = [0.0]

    def check(logits, rows):
        got = logits.float().cpu().numpy().astype(np.float64)
        assert np.isfinite(got).all()
        for g, (name, ref, pos) in zip(got, rows):
            err = float(np.abs(g - ref[pos]).max() / np.abs(ref[pos]).max())
            assert err < TOL[dtype], f"request {name} position {pos}: error {err:.3e}"
            worst[0] = max(worst[0], err)

    assert runner.admit("a") and runner.admit("b")
    sample = [0, 1, 777, 1023, 1024, 2047]
    for p0 in range(0, n_long, 2048):
        logits = runner.step([StepEntry("a", a[p0:p0 + 2048], sample)])
        check(logits, [("a", ref_a, p0 + i) for i in sample])
    for i in range(n_long, n_long + 32):
        entries, rows = [StepEntry("a", a[i:i + 1], [0])], [("a", ref_a, i)]
        j = i - n_long - 10
        if j == 0:        # a decoded token of the long request beside a whole 2,048-token portion of another one
            entries.append(StepEntry("b", b[:2048], [0, 2047]))
            rows += [("b", ref_b, 0), ("b", ref_b, 2047)]
        elif 0 < j <= 6:  # ... and then the two decode side by side, 20,000 keys beside 2,000
            entries.insert(0, StepEntry("b", b[2047 + j:2048 + j], [0]))
            rows.insert(0, ("b", ref_b, 2047 + j))
        check(runner.step(entries), rows)
    assert len(runner.cache.get("a").tables[0]) == (n_long + 32 + 15) // 16
    if dtype != "float32":
        assert runner._graphs, "decoding did not go through captured steps"
    runner.release("a"); runner.release("b")
    assert sum(runner.cache.held_pages()) == 0
    print(f"long context {n_long} {dtype}: worst relative error {worst[0]:.3e}")
    folder = os.environ.get("VT_TEST_REPORT_DIR")
    if folder:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "engine_errors.txt"), "a") as f:
            f.write(f"long context {n_long} {dtype}: worst relative error {worst[0]:.3e}\n")


# ---------------------------------------------------------------------------
# A needle: one token whose key every later query scores far above all others, and whose value row is large.
# ---------------------------------------------------------------------------
NEEDLE = LONG["vocab_size"] - 1      # its token id; the other tokens of a needle sequence are drawn from below it
NEEDLE_DIM = 5                       # the one hidden dim that its embedding has
Q_BIAS, K_GAIN = 5.0, 6.0            # every query has Q_BIAS in the slowest rotary pair, the needle's key K_GAIN * sqrt(H)


@pytest.fixture(scope="module")
def needle_folder(long_folder, tmp_path_factory):
    """The long model with one more trick: token NEEDLE's embedding is a unit vector (after the norm: sqrt(H) in one
    dim, nothing elsewhere), the key projection sends that dim to the head's slowest rotary pair (dims D/2 - 1 and
    D - 1 turn by 0.03 radians over 20,000 positions: the score does not depend on the distance), every query has a
    constant there, and the value projection sends it to a large row.  A query that sees the needle scores it
    Q_BIAS * K_GAIN = 30 above its other keys and puts all its weight there; one that has lost it (the key's
    16-key block skipped, read from another page, or one key range of a split dropped) gives a different row."""
    from vt_transformer_amd.weights.safetensors_io import WeightStore, write_safetensors
    folder = str(tmp_path_factory.mktemp("needle") / "m")
    os.makedirs(folder)
    with open(os.path.join(long_folder, "config.json")) as f, open(os.path.join(folder, "config.json"), "w") as g:
        g.write(f.read())
    store = WeightStore(long_folder)
    h, d, nh, kvh = LONG["hidden_size"], LONG["head_dim"], LONG["num_attention_heads"], LONG["num_key_value_heads"]
    gen = torch.Generator().manual_seed(77)
    tensors = []
    for name in store.names():
        t = store.get(name).float().clone()
        if name == "model.embed_tokens.weight":
            t[NEEDLE] = 0.0
            t[NEEDLE, NEEDLE_DIM] = 1.0
        elif name.endswith("k_proj.weight"):
            for head in range(kvh):
                t[head * d + d // 2 - 1] = 0.0
                t[head * d + d // 2 - 1, NEEDLE_DIM] = K_GAIN
        elif name.endswith("q_proj.bias"):
            for head in range(nh):
                t[head * d + d // 2 - 1] = Q_BIAS
        elif name.endswith("v_proj.weight"):
            t[:, NEEDLE_DIM] = torch.randn(t.shape[0], generator=gen) * 0.3
        tensors.append((name, t.to(torch.bfloat16)))
    store.close()
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors, metadata={"format": "pt"})
    return folder


def needle_sequence(n, seed):
    """n tokens without the needle's id, and the needle at a place drawn from `seed`."""
    rs = np.random.RandomState(seed)
    toks = rs.randint(0, NEEDLE, size=n).tolist()
    place = int(rs.randint(16, n - 64))
    toks[place] = NEEDLE
    return toks, place


def needle_seed():
    """Another place every run (VT_NEEDLE_SEED repeats a run that failed: the seed is in every message)."""
    return int(os.environ.get("VT_NEEDLE_SEED", int.from_bytes(os.urandom(3), "little")))


def test_losing_the_needles_block_changes_the_plain_models_rows(needle_folder):
    """In the plain model: with the 16 tokens of the needle's block replaced by others, the last row moves by more
    than ten times the bfloat16 tolerance."""
    cfg, w = plain_model.read_folder(needle_folder)
    seed = needle_seed()
    toks, place = needle_sequence(6000, seed)
    lost = list(toks)
    b0 = place // 16 * 16
    lost[b0:b0 + 16] = [(t + 1) % NEEDLE for t in toks[b0:b0 + 16]]
    full = plain_model.forward(cfg, w, toks, device="cuda")[-1]
    without = plain_model.forward(cfg, w, lost, device="cuda")[-1]
    effect = float((full - without).abs().max() / full.abs().max())
    print(f"needle at {place} of 6,000 (seed {seed}): losing its block moves the last row by {effect:.3e}")
    assert effect > 10 * TOL["bfloat16"], (seed, place, effect)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "float16"])
@pytest.mark.parametrize("n_long", [8192, 20480])
def test_a_needle_anywhere_in_a_long_context_is_found(needle_folder, dtype, n_long):
    """The needle lies at a place drawn anew every run; portions of 2,048 (the tiled kernel, items cut into key
    ranges), then 24 tokens one by one through captured steps (every entry's keys cut into up to sixteen ranges),
    beside a second request with a needle of its own."""
    from vt_transformer_amd.engine import StepEntry, load_model, make_runner
    seed = needle_seed()
    a, place_a = needle_sequence(n_long + 24, seed)
    b, place_b = needle_sequence(700 + 24, seed + 1)
    where = f"seed {seed}: needles at {place_a} of {n_long + 24} and {place_b} of {len(b)}"
    ref_a, ref_b = reference(needle_folder, a), reference(needle_folder, b)
    model = load_model(needle_folder, dtype)
    runner = make_runner(model, pool_tokens=n_long + 64 + 768, page_size=16, max_requests=4, max_seq_len=32768)
    runner.decode_graphs = True
    worst = 0.0

    def check(logits, rows):
        nonlocal worst
        got = logits.float().cpu().numpy().astype(np.float64)
        assert np.isfinite(got).all(), where
        for g, (name, ref, pos) in zip(got, rows):
            err = float(np.abs(g - ref[pos]).max() / np.abs(ref[pos]).max())
            assert err < TOL[dtype], f"{where}; request {name} position {pos}: error {err:.3e}"
            worst = max(worst, err)

    assert runner.admit("a") and runner.admit("b")
    sample = [0, 1, 777, 1023, 1024, 2047]
    for p0 in range(0, n_long, 2048):
        check(runner.step([StepEntry("a", a[p0:p0 + 2048], sample)]), [("a", ref_a, p0 + i) for i in sample])
    check(runner.step([StepEntry("b", b[:700], [0, 699])]), [("b", ref_b, 0), ("b", ref_b, 699)])
    for i in range(24):
        logits = runner.step([StepEntry("a", a[n_long + i:n_long + i + 1], [0]), StepEntry("b", b[700 + i:701 + i], [0])])
        check(logits, [("a", ref_a, n_long + i), ("b", ref_b, 700 + i)])
    if dtype != "float32":
        assert runner._graphs, "decoding did not go through captured steps"
    runner.release("a"); runner.release("b")
    print(f"needle, {where}, {dtype}: worst relative error {worst:.3e}")
