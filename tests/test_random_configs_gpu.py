"""Configurations drawn at random (heads, groups, head sizes in steps of 16, widths and vocabularies that are no
power of two, windows on some layers, eps, tied or untied head): the engine against the plain implementation, whole,
cut at random, decoded one by one, and decoded through captured graphs."""
import numpy as np
import pytest
import torch

import plain_model
from replay_helpers import check_against_plain, cut, max_live_tokens, random_requests, run_in_process, trace_mixed

pytestmark = pytest.mark.gpu


def draw_config(seed: int) -> dict:
    rs = np.random.RandomState(seed)
    kvh = int(rs.choice([1, 2, 3, 4]))
    group = int(rs.choice([1, 2, 3, 5, 7, 8, 16]))
    d = int(rs.choice(range(16, 257, 16)))
    if kvh * group * d > 4096:
        group = max(1, 4096 // (kvh * d))
    layers = int(rs.randint(1, 5))
    return dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=int(rs.choice([97, 203, 320, 1001, 4099])),
                hidden_size=int(rs.choice([40, 72, 96, 104, 120, 200, 328])), intermediate_size=int(rs.choice([56, 88, 136, 200, 520])),
                num_hidden_layers=layers, num_attention_heads=kvh * group, num_key_value_heads=kvh, head_dim=d,
                rope_theta=float(rs.choice([1e4, 5e4, 1e6])), rms_norm_eps=float(rs.choice([1e-6, 1e-5, 3e-3])),
                tie_word_embeddings=bool(rs.rand() < 0.5), max_position_embeddings=1024, hidden_act="silu",
                use_sliding_window=bool(rs.rand() < 0.4), sliding_window=int(rs.choice([5, 17, 40, 64])),
                max_window_layers=int(rs.randint(0, layers + 1)), torch_dtype="bfloat16")


@pytest.mark.parametrize("seed", range(8))
def test_random_configuration(seed, tmp_path):
    check_configuration(draw_config(100 + seed), seed, tmp_path)


@pytest.mark.parametrize("hidden,inter", [(100, 100), (104, 84), (76, 136)])
def test_widths_that_are_no_multiple_of_eight(hidden, inter, tmp_path):
    """The vectorised kernels (16-byte accesses, fused norm and residual) do not take these widths: the any-shape
    kernels must, in every mode."""
    cfg = dict(draw_config(3), hidden_size=hidden, intermediate_size=inter, num_hidden_layers=2, max_window_layers=1)
    check_configuration(cfg, hidden, tmp_path)


def check_configuration(cfg, seed, tmp_path):
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import StepEntry, load_model, make_runner
    from vt_transformer_amd.weights import write_random_model
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(cfg), folder, seed=seed)
    pcfg, w = plain_model.read_folder(folder)
    rs = np.random.RandomState(seed)
    n = int(rs.randint(70, 200))
    toks = rs.randint(0, cfg["vocab_size"], size=n).tolist()
    ref = plain_model.forward(pcfg, w, toks)
    worst = {}
    for dtype, tol in (("float32", 3e-5), ("bfloat16", 1.5e-2), ("float16", 2e-3)):
        model = load_model(folder, dtype)
        for mode in ("whole", "cut", "decode", "graph"):
            runner = make_runner(model, pool_tokens=-(-n // 16) * 16 + 32, page_size=16, max_requests=2, max_seq_len=512)
            runner.decode_graphs = mode == "graph"
            runner.admit("r")
            if mode == "whole":
                cuts = [(0, n)]
            elif mode == "cut":
                cuts, a = [], 0
                while a < n:
                    b = min(n, a + int(rs.choice([2, 3, 5, 16, 17, 31, 64])))
                    cuts.append((a, b))
                    a = b
            else:
                cuts = [(0, n - 32)] + [(i, i + 1) for i in range(n - 32, n)]
            got = torch.cat([runner.step([StepEntry("r", toks[a:b], list(range(b - a)))]).float().cpu() for a, b in cuts])
            err = float((got.double() - ref).abs().max() / ref.abs().max())
            assert err < tol, (cfg, dtype, mode, err)
            worst[dtype] = max(worst.get(dtype, 0.), err)
        # several requests at a time, portions of some beside decoded tokens of others, pages used again
        reqs = random_requests(cfg["vocab_size"], [int(x) for x in rs.randint(1, 70, size=7)], seed=seed)
        portions = {}
        for r, t in reqs.items():
            n_head = max(0, len(t) - int(rs.randint(1, 10)))
            parts = cut(t[:n_head], [int(x) for x in rs.choice([2, 3, 5, 8, 11, 16, 17], size=2)]) if n_head else []
            portions[r] = parts + [(j, j + 1) for j in range(n_head, len(t))]
        steps = trace_mixed(reqs, portions, max_live=4, seed=seed)
        runner = make_runner(model, pool_tokens=max_live_tokens(steps), page_size=16, max_requests=4, max_seq_len=512)
        runner.decode_graphs = True
        worst[dtype] = max(worst[dtype], check_against_plain(folder, reqs, steps, run_in_process(runner, steps), dtype))
        assert sum(runner.cache.held_pages()) == 0
    print(f"random configuration {seed}: worst relative error {worst}")


def size_tolerance(dtype: str, width: int) -> float:
    """The comparisons with the plain model at real layer sizes, relative to a row's largest logit.  The rounding of a
    16-bit model grows with the length of its sums: measured 9.2e-3, 1.2e-2 and 1.9e-2 in bfloat16 at widths 1,536, 3,584
    and 8,192 (float16: an eighth of that, three more bits; float32: 3.5e-6 to 1.2e-5), about the square root of the
    width.  Twice what was measured at the largest width, following the root of the width."""
    per_root = {"bfloat16": 4.2e-4, "float16": 5.0e-5, "float32": 2.6e-7}[dtype]
    return per_root * width ** 0.5


@pytest.mark.parametrize("name,hidden,heads,kv,inter", [("7B", 3584, 28, 4, 18944), ("1.5B", 1536, 12, 2, 8960),
                                                        ("72B", 8192, 64, 8, 29568)])
def test_real_layer_sizes(name, hidden, heads, kv, inter, tmp_path):
    """Two layers at Qwen2-7B, 1.5B and 72B layer sizes (a small vocabulary): the kernels choose their launch shapes
    by these sizes (waves per block, k ranges, which product kernel), so the tiny configurations do not reach them.
    Whole, cut, decoded one by one (eagerly and through captured graphs), and 40 copies of the request decoding side
    by side (the 17-to-64-row kernels)."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import StepEntry, load_model, make_runner
    from vt_transformer_amd.weights import write_random_model
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=4099, hidden_size=hidden,
               intermediate_size=inter, num_hidden_layers=2, num_attention_heads=heads, num_key_value_heads=kv, head_dim=128,
               rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=name == "1.5B", max_position_embeddings=8192,
               hidden_act="silu", use_sliding_window=False, torch_dtype="bfloat16")
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(cfg), folder, seed=1)
    pcfg, w = plain_model.read_folder(folder)
    n = 200
    toks = np.random.RandomState(0).randint(0, 4099, size=n).tolist()
    ref = plain_model.forward(pcfg, w, toks)
    scale = ref.abs().max()
    for dtype in ("bfloat16", "float16", "float32"):
        tol = size_tolerance(dtype, hidden)
        model = load_model(folder, dtype)
        for mode in ("whole", "cut", "decode", "graph", "batch"):
            runner = make_runner(model, pool_tokens=10240, page_size=16, max_requests=48, max_seq_len=512)
            runner.decode_graphs = mode == "graph"
            if mode == "whole":
                cuts = [(0, n)]
            elif mode == "cut":
                cuts = [(0, 70), (70, 87), (87, 150), (150, 152), (152, 200)]
            else:
                cuts = [(0, n - 32)] + [(i, i + 1) for i in range(n - 32, n)]
            if mode == "batch":
                ids = [f"r{i}" for i in range(40)]
                for i in ids:
                    runner.admit(i)
                    runner.step([StepEntry(i, toks[:n - 32], [])])
                got = torch.stack([runner.step([StepEntry(i, toks[a:b], [0]) for i in ids]).float().cpu()
                                   for a, b in cuts[1:]]).double()          # [32, 40, vocab]
                err = float((got - ref[n - 32:, None, :]).abs().max() / scale)
            else:
                runner.admit("r")
                got = torch.cat([runner.step([StepEntry("r", toks[a:b], list(range(b - a)))]).float().cpu() for a, b in cuts])
                err = float((got.double() - ref).abs().max() / scale)
            assert err < tol, (name, dtype, mode, err)
            print(f"layer sizes {name} {dtype} {mode}: relative error {err:.3e}")
        del model


@pytest.mark.parametrize("n_req", [96, 160])
def test_many_requests_decoding_side_by_side_at_7b_layer_sizes(n_req, tmp_path):
    """More decoding requests than the few-row kernels take (64): the products of 65 to 255 rows go to the GEMM
    library, except the gated pair up to 128 rows and the down projection, which stay on the packed matrices with 128
    tokens to a block.  96 (and 160) requests with prompts of their own, of different lengths, decode eight tokens side by
    side; every row against the plain implementation (in float64 on the GPU: 96 sequences at these sizes take the
    CPU minutes).  In bfloat16 once through a captured step, which holds library products here, and once launched
    kernel by kernel; between two replays of the captured step another request's prompt runs, as any serving loop
    would have it, and every replay is checked."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import StepEntry, load_model, make_runner
    from vt_transformer_amd.weights import write_random_model
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=4099, hidden_size=3584,
               intermediate_size=18944, num_hidden_layers=2, num_attention_heads=28, num_key_value_heads=4, head_dim=128,
               rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=8192,
               hidden_act="silu", use_sliding_window=False, torch_dtype="bfloat16")
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(cfg), folder, seed=2)
    pcfg, w = plain_model.read_folder(folder)
    w = {k: v.to("cuda") for k, v in w.items()}
    rs = np.random.RandomState(1)
    n_dec = 8
    reqs = [rs.randint(0, 4099, size=int(rs.randint(20, 120)) + n_dec).tolist() for _ in range(n_req)]
    refs = [plain_model.forward(pcfg, w, t)[-n_dec:] for t in reqs]            # [n_dec, vocab] each
    late = rs.randint(0, 4099, size=90).tolist()                               # a request that comes in between
    late_ref = plain_model.forward(pcfg, w, late)[-1]
    del w
    torch.cuda.empty_cache()
    variants = (("bfloat16", True, 2e-2), ("float16", True, 3e-3), ("bfloat16", False, 2e-2), ("float32", False, 3e-5))
    for dtype, graphs, tol in variants[:4 if n_req == 96 else 2]:
        model = load_model(folder, dtype)
        runner = make_runner(model, pool_tokens=(n_req + 1) * 144, page_size=16, max_requests=n_req + 1, max_seq_len=512)
        runner.decode_graphs = graphs
        for i, t in enumerate(reqs):
            runner.admit(i)
        # the prompts in steps of 24 requests, then all of them decode together
        for i0 in range(0, n_req, 24):
            runner.step([StepEntry(i, reqs[i][:-n_dec], []) for i in range(i0, min(n_req, i0 + 24))])
        worst = 0.0
        for j in range(n_dec):
            got = runner.step([StepEntry(i, [reqs[i][len(reqs[i]) - n_dec + j]], [0]) for i in range(n_req)]).float().cpu().double()
            for i in range(n_req):
                err = float((got[i] - refs[i][j]).abs().max() / refs[i][j].abs().max())
                assert err < tol, (dtype, graphs, "request", i, "token", j, err)
                worst = max(worst, err)
            if j == 3:
                runner.admit("late")
                got = runner.step([StepEntry("late", late, [len(late) - 1])]).float().cpu().double()[0]
                assert float((got - late_ref).abs().max() / late_ref.abs().max()) < tol, (dtype, graphs, "the request in between")
                runner.release("late")
        assert bool(runner._graphs) == graphs          # (a captured step takes up to 192 entries)
        print(f"{n_req} decoding requests {dtype}{' captured' if graphs else ''}: worst relative error {worst:.3e}")
        del model, runner


@pytest.mark.parametrize("tied", [False, True])
@pytest.mark.parametrize("name,hidden,heads,kv,inter", [("7B", 3584, 28, 4, 18944), ("72B", 8192, 64, 8, 29568)])
def test_the_whole_vocabulary(name, hidden, heads, kv, inter, tied):
    """One layer at Qwen2-7B and 72B widths under the real vocabulary of 152,064 (9,504 tile rows of the head; at
    width 8,192 its matrix has 1.25 G elements, beyond 32-bit byte offsets), tied and untied: the logits of a
    40-token portion (the 17-to-64-row kernels) and of 3 tokens decoded one by one (the few-row kernels), and the
    embedding's rows of the first and the last token id (the reference's head and lookup:
    v1/tensortype/hip_tensor.cpp:923-991, v1/tensortype/hip_kernels/embed.cpp:7-37), against float64, in the three
    dtypes.  The tensors are drawn on the device and the plain model runs there in float64: on the host the head
    alone would be 10 GB."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import StepEntry, build_model, make_runner
    V = 152064
    cfg = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=V, hidden_size=hidden,
               intermediate_size=inter, num_hidden_layers=1, num_attention_heads=heads, num_key_value_heads=kv, head_dim=128,
               rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=tied, max_position_embeddings=8192,
               hidden_act="silu", use_sliding_window=False, torch_dtype="bfloat16")
    config = config_from_dict(cfg)
    gen = torch.Generator(device="cuda").manual_seed(hidden + tied)
    expected = build_model(config, "float32").tensors()
    w16 = {}
    for tname, decl in expected.items():
        if decl.optional:
            continue
        t = torch.randn(decl.shape, generator=gen, device="cuda") * 0.02
        if decl.role == "gain":
            t += 1.0
        w16[tname] = t.to(torch.bfloat16)
    toks = [0, V - 1] + np.random.RandomState(hidden).randint(0, V, size=41).tolist()
    ref = plain_model.forward(cfg, {k: v.double() for k, v in w16.items()}, toks)          # [43, V] float64, on the host
    torch.cuda.empty_cache()
    for dtype in ("bfloat16", "float16", "float32"):
        model = build_model(config, dtype)
        model.load(w16.__getitem__)
        rows = model.embedding.forward(torch.tensor([0, V - 1], dtype=torch.int32, device="cuda"))
        table = w16["model.embed_tokens.weight"]
        # (as the model holds them: float16 has subnormals where bfloat16 still has eight bits)
        assert torch.equal(rows.cpu(), table[[0, V - 1]].to(model.rt.dtype).float().cpu()), (name, dtype, "embedding rows")
        runner = make_runner(model, pool_tokens=64, page_size=16, max_requests=2, max_seq_len=64)
        runner.admit("r")
        got = [runner.step([StepEntry("r", toks[:40], list(range(40)))]).float().cpu()]
        got += [runner.step([StepEntry("r", toks[i:i + 1], [0])]).float().cpu() for i in (40, 41, 42)]
        got = torch.cat(got).double()
        assert got.shape == (43, V)
        err = float(((got - ref).abs().max(dim=1).values / ref.abs().max(dim=1).values).max())
        print(f"whole vocabulary {name} tied={tied} {dtype}: relative error {err:.3e}")
        assert err < size_tolerance(dtype, hidden), (name, tied, dtype, err)
        # the head's far end alone: the last tile row of the matrix against the same rows of the reference
        tail = float((got[:, V - 16:] - ref[:, V - 16:]).abs().max() / ref.abs().max())
        assert tail < size_tolerance(dtype, hidden), (name, tied, dtype, "last tile row", tail)
        del model, runner
        torch.cuda.empty_cache()
