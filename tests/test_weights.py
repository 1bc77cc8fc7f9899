"""Safetensors by tensor name, the one error for everything that does not fit, and random weights."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY_A, TINY_B
from vt_transformer_amd.config import config_from_dict
from vt_transformer_amd.weights import (SafetensorsFile, WeightError, WeightFileError, WeightStore, check_tensors,
                                        declared_tensors, random_tensor, write_random_model, write_safetensors)


def test_writer_and_reader_agree_with_the_safetensors_library(tmp_path):
    from safetensors import safe_open
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(0)
    tensors = {"a.weight": torch.randn(5, 7, generator=g).to(torch.bfloat16), "b": torch.randn(3, generator=g),
               "c.table": torch.arange(6, dtype=torch.int32).reshape(2, 3), "h": torch.randn(4, 2, generator=g).half()}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, tensors.items(), metadata={"seed": 3})
    with safe_open(ours, framework="pt") as f:          # the library reads what we wrote
        assert set(f.keys()) == set(tensors)
        for k, v in tensors.items():
            assert torch.equal(f.get_tensor(k), v)
    theirs = str(tmp_path / "theirs.safetensors")
    save_file(tensors, theirs)
    f = SafetensorsFile(theirs)                          # and we read what the library wrote
    assert set(f.names()) == set(tensors)
    for k, v in tensors.items():
        assert f.info(k) == (v.dtype, tuple(v.shape))
        assert torch.equal(f.get(k), v)


def test_sharded_folder(tmp_path):
    write_safetensors(str(tmp_path / "s1.safetensors"), [("x", torch.ones(2))])
    write_safetensors(str(tmp_path / "s2.safetensors"), [("y", torch.zeros(3))])
    with open(tmp_path / "model.safetensors.index.json", "w") as f:
        json.dump({"weight_map": {"x": "s1.safetensors", "y": "s2.safetensors"}}, f)
    st = WeightStore(str(tmp_path))
    assert sorted(st.names()) == ["x", "y"] and torch.equal(st.get("y"), torch.zeros(3))


def test_broken_files_are_named(tmp_path):
    p = str(tmp_path / "model.safetensors")
    write_safetensors(p, [("x", torch.ones(100))])
    data = open(p, "rb").read()
    open(p, "wb").write(data[:-10])
    with pytest.raises(WeightFileError, match="truncated"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 5) + b"{nope")
    with pytest.raises(WeightFileError, match="JSON"):
        SafetensorsFile(p)
    with pytest.raises(WeightFileError, match="neither"):
        WeightStore(str(tmp_path / "empty"))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = config_from_dict(dict(TINY_B))
    folder = write_random_model(cfg, str(tmp_path / "m"), seed=1)
    st = WeightStore(folder)
    infos = {n: st.info(n) for n in st.names()}
    expected = declared_tensors(cfg)
    check_tensors(expected, infos, folder)                      # as written: fine
    del infos["model.layers.1.mlp.up_proj.weight"]
    del infos["model.norm.weight"]
    infos["model.layers.0.self_attn.rotary_emb.inv_freq"] = (torch.float32, (16,))
    infos["model.layers.2.self_attn.k_proj.bias"] = (torch.bfloat16, (95,))
    infos["lm_head.weight"] = (torch.bfloat16, (96, 320))
    with pytest.raises(WeightError) as e:
        check_tensors(expected, infos, folder)
    msg = str(e.value)
    for word in ("model.layers.1.mlp.up_proj.weight", "model.norm.weight", "rotary_emb.inv_freq",
                 "k_proj.bias is [95], expected [96]", "lm_head.weight is [96, 320], expected [320, 96]",
                 "missing (2)", "unexpected (1)", "wrong shape (2)"):
        assert word in msg, word
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]


def test_tied_head_needs_no_tensor_of_its_own(tmp_path):
    cfg = config_from_dict(dict(TINY_A))
    folder = write_random_model(cfg, str(tmp_path / "m"), seed=1)
    st = WeightStore(folder)
    assert "lm_head.weight" not in st.names()
    check_tensors(declared_tensors(cfg), {n: st.info(n) for n in st.names()}, folder)
    untied = config_from_dict(dict(TINY_A, tie_word_embeddings=False))
    with pytest.raises(WeightError, match="lm_head.weight"):
        check_tensors(declared_tensors(untied), {n: st.info(n) for n in st.names()}, folder)


def test_random_weights(tmp_path):
    cfg = config_from_dict(dict(TINY_B))
    a = WeightStore(write_random_model(cfg, str(tmp_path / "a"), seed=5))
    b = WeightStore(write_random_model(cfg, str(tmp_path / "b"), seed=5))
    c = WeightStore(write_random_model(cfg, str(tmp_path / "c"), seed=6))
    assert os.path.isfile(tmp_path / "a" / "config.json")
    names = sorted(a.names())
    assert names == sorted(b.names())
    for n in names:
        assert torch.equal(a.get(n), b.get(n))            # the seed fixes everything
        assert a.info(n)[0] == torch.bfloat16             # kept in bfloat16
    assert not torch.equal(a.get("lm_head.weight"), c.get("lm_head.weight"))
    w = a.get("model.layers.0.mlp.down_proj.weight").float()
    assert abs(float(w.mean())) < 2e-3 and 0.018 < float(w.std()) < 0.022          # N(0, 0.02)
    gain = a.get("model.norm.weight").float()
    assert abs(float(gain.mean()) - 1.0) < 0.01 and float(gain.std()) < 0.03      # 1 + N(0, 0.02)
    bias = a.get("model.layers.1.self_attn.q_proj.bias").float()
    assert abs(float(bias.mean())) < 0.01
    # a tensor's values do not depend on which other tensors exist
    decl = declared_tensors(cfg)["model.layers.2.self_attn.v_proj.weight"]
    alone = random_tensor("model.layers.2.self_attn.v_proj.weight", decl, 5, torch.device("cpu"), torch.bfloat16)
    assert torch.equal(alone, a.get("model.layers.2.self_attn.v_proj.weight"))


def test_counter_based_generator_is_a_function_of_key_and_index():
    """Pinned values (so that the device's twin and any later rewrite must make these very bits), independence of
    how the elements are cut into pieces, and the distribution: close to normal with the asked deviation."""
    import numpy as np
    from vt_transformer_amd.weights.random_init import counter_normal, normal_scale, tensor_key
    assert tensor_key(5, "model.norm.weight") == tensor_key(5, "model.norm.weight") != tensor_key(6, "model.norm.weight")
    x = counter_normal(12345, 0, 200000, 0.02, 0.0)
    assert x.dtype == np.float32
    # the sum of the twelve 16-bit fields of three SplitMix64 words, by hand for element 7
    def mix(z):
        z &= (1 << 64) - 1
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & ((1 << 64) - 1)
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & ((1 << 64) - 1)
        return z ^ (z >> 31)
    total = 0
    for j in (1, 2, 3):
        w = mix(12345 + (3 * 7 + j) * 0x9E3779B97F4A7C15)
        total += sum((w >> s) & 0xFFFF for s in (0, 16, 32, 48))
    assert x[7] == np.float32(total - 393210) * np.float32(normal_scale(0.02))
    pieces = np.concatenate([counter_normal(12345, a, b - a, 0.02, 0.0) for a, b in ((0, 7), (7, 1000), (1000, 200000))])
    assert np.array_equal(pieces, x)
    assert abs(float(x.mean())) < 2e-4 and abs(float(x.std()) - 0.02) < 2e-4
    z = x / x.std()
    assert abs(float((z ** 3).mean())) < 0.03 and 2.8 < float((z ** 4).mean()) < 3.0      # a sum of twelve: kurtosis 2.9
    assert np.array_equal(counter_normal(12345, 0, 1000, 0.02, 1.0), x[:1000] + np.float32(1.0))
    assert not np.array_equal(counter_normal(12346, 0, 1000, 0.02, 0.0), x[:1000])


def test_a_tensor_stored_in_32_bit_stays_so():
    from vt_transformer_amd.parts.base import Runtime
    rt = Runtime(torch.device("cpu"), torch.bfloat16)
    assert rt.place(torch.ones(3, dtype=torch.bfloat16), "gain").dtype == torch.float32   # small vectors: fp32, exact
    assert rt.place(torch.ones(3, dtype=torch.float32), "bias").dtype == torch.float32
    assert rt.place(torch.ones(2, 2, dtype=torch.bfloat16), "matrix").dtype == torch.bfloat16
    assert rt.place(torch.ones(2, dtype=torch.int64), "table").dtype == torch.int32
    rt32 = Runtime(torch.device("cpu"), torch.float32)
    assert rt32.place(torch.ones(2, 2, dtype=torch.bfloat16), "matrix").dtype == torch.float32
