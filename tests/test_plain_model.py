"""What fixes the plain implementation beside the reference's text: special cases that reduce to a library
routine, and invariants, each chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong
place, eps outside the root) fails it."""
import math

import numpy as np
import pytest
import torch

import plain_model as pm
from conftest import TINY_A, TINY_B, TINY_W

DT = torch.float64


def rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=DT)


# ---- RMSNorm ---------------------------------------------------------------
def test_rmsnorm_with_unit_gain_is_x_over_root_mean_square():
    x = rand(5, 24).numpy()
    ref = x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6)
    assert np.allclose(pm.rmsnorm(torch.from_numpy(x), torch.ones(24, dtype=DT), 1e-6).numpy(), ref, atol=1e-12)


def test_rmsnorm_eps_is_inside_the_root_and_added_to_the_mean():
    x = torch.full((1, 8), 2.0, dtype=DT)          # mean square 4
    out = pm.rmsnorm(x, torch.ones(8, dtype=DT), 5.0)
    assert torch.allclose(out, torch.full((1, 8), 2.0 / 3.0, dtype=DT))      # 2 / sqrt(4 + 5), not 2 / (2 + 5)
    # eps -> 0: scaling the input leaves the output unchanged; the gain multiplies elementwise
    y = rand(3, 16)
    g = rand(16, seed=1)
    assert torch.allclose(pm.rmsnorm(7 * y, g, 1e-30), pm.rmsnorm(y, g, 1e-30), atol=1e-10)
    assert torch.allclose(pm.rmsnorm(y, g, 1e-6), g * pm.rmsnorm(y, torch.ones(16, dtype=DT), 1e-6))


# ---- linear ----------------------------------------------------------------
def test_linear_is_x_w_transposed_plus_bias():
    x, w, b = rand(4, 6).numpy(), rand(3, 6, seed=1).numpy(), rand(3, seed=2).numpy()
    got = pm.linear(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b)).numpy()
    assert np.allclose(got, x @ w.T + b)


# ---- rotary ----------------------------------------------------------------
def test_rotary_position_zero_is_identity_and_pairs_keep_their_norm():
    x = rand(1, 3, 16)
    assert torch.allclose(pm.rotary(x, torch.tensor([0]), 10000.0), x)
    y = pm.rotary(rand(4, 2, 16), torch.tensor([3, 17, 100, 1000]), 10000.0)
    x4 = rand(4, 2, 16)
    for i in range(8):                              # pair (i, i + D/2), not (2i, 2i + 1)
        n_in = x4[..., i] ** 2 + x4[..., i + 8] ** 2
        y4 = pm.rotary(x4, torch.tensor([3, 17, 100, 1000]), 10000.0)
        assert torch.allclose(y4[..., i] ** 2 + y4[..., i + 8] ** 2, n_in)


def test_rotary_explicit_vector():
    """D = 4, base = 100: angles of position p are p * [1, 0.1].  One nonzero entry shows pairing and sign."""
    x = torch.zeros(1, 1, 4, dtype=DT)
    x[0, 0, 0] = 1.0                                # first half of pair 0 = (dims 0, 2)
    y = pm.rotary(x, torch.tensor([2]), 100.0)[0, 0]
    assert torch.allclose(y, torch.tensor([math.cos(2.0), 0.0, math.sin(2.0), 0.0], dtype=DT))
    x = torch.zeros(1, 1, 4, dtype=DT)
    x[0, 0, 3] = 1.0                                # second half of pair 1 = (dims 1, 3), angle 0.2
    y = pm.rotary(x, torch.tensor([2]), 100.0)[0, 0]
    assert torch.allclose(y, torch.tensor([0.0, -math.sin(0.2), 0.0, math.cos(0.2)], dtype=DT))


def test_rotary_scores_depend_only_on_distance():
    q, k = rand(1, 1, 32), rand(1, 1, 32, seed=1)
    def score(m, n):
        return float((pm.rotary(q, torch.tensor([m]), 1e6) * pm.rotary(k, torch.tensor([n]), 1e6)).sum())
    assert abs(score(5, 2) - score(105, 102)) < 1e-9
    assert abs(score(5, 2) - score(2, 5)) > 1e-3    # direction matters


def test_rotary_angles_match_the_table_formula():
    """v1/tensortype/common.cpp:9-13: inv_freq[i/2] = 1 / base^(i/dims) for even i."""
    a = pm.rotary_angles(torch.tensor([3]), 8, 10000.0)[0]
    ref = torch.tensor([3.0 / 10000.0 ** (i / 8) for i in (0, 2, 4, 6)], dtype=DT)
    assert torch.allclose(a, ref)


# ---- attention -------------------------------------------------------------
def test_attention_without_groups_is_the_library_routine():
    t, nh, d = 9, 3, 8
    q, k, v = rand(t, nh, d), rand(t, nh, d, seed=1), rand(t, nh, d, seed=2)
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                                           is_causal=True).transpose(0, 1)
    assert torch.allclose(pm.attention(q, k, v), ref, atol=1e-12)


def test_grouped_attention_is_attention_with_repeated_heads():
    t, nh, kvh, d = 7, 6, 2, 4
    q, k, v = rand(t, nh, d), rand(t, kvh, d, seed=1), rand(t, kvh, d, seed=2)
    rep_k = k.repeat_interleave(nh // kvh, dim=1)    # head h reads kv head h // 3
    rep_v = v.repeat_interleave(nh // kvh, dim=1)
    assert torch.allclose(pm.attention(q, k, v), pm.attention(q, rep_k, rep_v))
    wrong = pm.attention(q, k.repeat(1, nh // kvh, 1), v.repeat(1, nh // kvh, 1))   # h % kvh would be this
    assert not torch.allclose(pm.attention(q, k, v), wrong)


def test_attention_special_rows():
    t, d = 6, 4
    k, v = rand(t, 1, d, seed=1), rand(t, 1, d, seed=2)
    out = pm.attention(torch.zeros(t, 2, d, dtype=DT), k, v)
    assert torch.allclose(out[0, 0], v[0, 0])                         # one key: the value row
    assert torch.allclose(out[4, 1], v[:5, 0].mean(0))                # zero query: mean of the allowed values
    # scale 1/sqrt(D): with q = k_j * c the weight on key j follows exp(c |k_j|^2 / sqrt(D))
    q = torch.zeros(2, 1, d, dtype=DT)
    q[1, 0] = k[1, 0]
    s = torch.tensor([float(k[1, 0] @ k[0, 0]), float(k[1, 0] @ k[1, 0])], dtype=DT) / math.sqrt(d)
    p = torch.softmax(s, 0)
    assert torch.allclose(pm.attention(q, k[:2], v[:2])[1, 0], p[0] * v[0, 0] + p[1] * v[1, 0])


def test_attention_is_causal_and_window_counts_the_token_itself():
    t, d = 8, 4
    q, k, v = rand(t, 2, d), rand(t, 2, d, seed=1), rand(t, 2, d, seed=2)
    base = pm.attention(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[5:], v2[5:] = 9.0, -9.0
    assert torch.allclose(pm.attention(q, k2, v2)[:5], base[:5])      # later keys do not matter
    assert torch.allclose(pm.attention(q, k, v, window=t), base)      # a window of everything is no window
    assert torch.allclose(pm.attention(q, k, v, window=1), v.repeat_interleave(1, 1))   # only itself
    w3 = pm.attention(q, k, v, window=3)
    assert torch.allclose(w3[6], pm.attention(q[4:7], k[4:7], v[4:7])[2])      # keys 4, 5, 6 for token 6


# ---- feed-forward ----------------------------------------------------------
def test_swiglu():
    x, wg, wu, wd = rand(3, 6), rand(10, 6, seed=1), rand(10, 6, seed=2), rand(6, 10, seed=3)
    ref = (torch.nn.functional.silu(x @ wg.t()) * (x @ wu.t())) @ wd.t()
    assert torch.allclose(pm.swiglu(x, wg, wu, wd), ref, atol=1e-12)
    assert float(pm.swiglu(x, torch.zeros_like(wg), wu, wd).abs().max()) == 0.0     # gate 0 -> 0
    assert not torch.allclose(pm.swiglu(x, wu, wg, wd), ref)                          # gate and up are not symmetric


# ---- whole model -----------------------------------------------------------
def tiny_weights(cfg, seed=0):
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights import declared_tensors, random_tensor
    decl = declared_tensors(config_from_dict(dict(cfg)))
    return {n: random_tensor(n, d, seed, torch.device("cpu"), torch.float32).double() * (5.0 if d.role != "gain" else 1.0)
            for n, d in decl.items() if not d.optional}


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_W])
def test_logits_do_not_see_the_future_and_depend_on_distances_only(cfg):
    w = tiny_weights(cfg)
    ids = list(np.random.RandomState(0).randint(0, cfg["vocab_size"], size=60))
    full = pm.forward(cfg, w, ids)
    other = ids[:30] + list(np.random.RandomState(1).randint(0, cfg["vocab_size"], size=30))
    assert torch.allclose(pm.forward(cfg, w, other)[:30], full[:30], atol=1e-10)
    # a shift of all positions changes nothing: only distances enter the scores
    assert torch.allclose(pm.forward(cfg, w, ids, first_position=77), full, atol=1e-8)


def test_zero_output_projections_leave_only_the_embedding():
    cfg = TINY_B
    w = tiny_weights(cfg)
    for i in range(cfg["num_hidden_layers"]):
        w[f"model.layers.{i}.self_attn.o_proj.weight"].zero_()
        w[f"model.layers.{i}.mlp.down_proj.weight"].zero_()
    ids = [3, 1, 4, 1, 5]
    x = w["model.embed_tokens.weight"][torch.tensor(ids)]
    ref = pm.rmsnorm(x, w["model.norm.weight"], cfg["rms_norm_eps"]) @ w["lm_head.weight"].t()
    assert torch.allclose(pm.forward(cfg, w, ids), ref, atol=1e-12)


def test_tied_head_uses_the_embedding():
    w = tiny_weights(TINY_A)
    assert "lm_head.weight" not in w
    logits = pm.forward(TINY_A, w, [1, 2, 3])
    assert logits.shape == (3, TINY_A["vocab_size"])
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"] * 2
    assert torch.allclose(pm.forward(dict(TINY_A, tie_word_embeddings=False), w2, [1, 2, 3]), 2 * logits)


def test_window_layers_follow_max_window_layers():
    assert [pm.layer_window(TINY_W, i) for i in range(4)] == [0, 0, 40, 40]
    assert pm.layer_window(TINY_A, 1) == 0
    w = tiny_weights(TINY_W)
    ids = list(np.random.RandomState(2).randint(0, TINY_W["vocab_size"], size=90))
    nowin = dict(TINY_W, use_sliding_window=False)
    a, b = pm.forward(TINY_W, w, ids), pm.forward(nowin, w, ids)
    assert torch.allclose(a[:40], b[:40], atol=1e-10)          # the window only bites from the 41st token on
    assert not torch.allclose(a[60:], b[60:], atol=1e-6)


def test_plain_reader_agrees_with_the_library(tmp_path):
    from safetensors.torch import load_file
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights import write_random_model
    folder = write_random_model(config_from_dict(dict(TINY_B)), str(tmp_path / "m"), seed=3)
    cfg, w = pm.read_folder(folder)
    lib = load_file(str(tmp_path / "m" / "model.safetensors"))
    assert set(lib) == set(w)
    for n in lib:
        assert torch.equal(lib[n].double(), w[n])
    assert cfg["hidden_size"] == 96
