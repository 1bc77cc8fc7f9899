"""The engine against the plain implementation, in float32 and bfloat16, under
every way of cutting the work: whole requests, the last 32 tokens one by
one, portions of changing size, and mixed batches with so few pages that
they are used again."""
import os

import numpy as np
import pytest
import torch

import plain_model
from conftest import TINY
from replay_helpers import (check_against_plain, cut, max_live_tokens, random_requests, run_in_process,
                            run_trace_run, trace_alone, trace_mixed)

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16", "float16"]
CONFIGS = ["A", "B", "W"]
_plain_cache = {}
_models = {}
TOL_BF16 = 1.5e-2


def get_model(folders, name, dtype):
    from vt_transformer_amd.engine import load_model
    key = (name, dtype)
    if key not in _models:
        _models[key] = load_model(folders[name], dtype)
    return _models[key]


def runner_for(model, pool_tokens, max_requests=8, page_size=16):
    from vt_transformer_amd.engine import make_runner
    return make_runner(model, pool_tokens=pool_tokens, page_size=page_size, max_requests=max_requests,
                       max_seq_len=min(model.spec.max_positions, max(pool_tokens, 16)))


def report(name, worst):
    """The worst error of a comparison: printed (pytest -s shows it) and, with VT_TEST_REPORT_DIR set, appended
    to engine_errors.txt in that folder."""
    line = f"{name}: worst relative error {worst:.3e}"
    print(line)
    folder = os.environ.get("VT_TEST_REPORT_DIR")
    if folder:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "engine_errors.txt"), "a") as f:
            f.write(line + "\n")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", CONFIGS)
def test_whole_requests(model_folders, cfg, dtype):
    """Each request alone and whole, logits at every position."""
    reqs = random_requests(TINY[cfg]["vocab_size"], [5, 9, 13, 1, 70, 150], seed=1)
    steps = trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
    runner = runner_for(get_model(model_folders, cfg, dtype), 192)
    got = run_in_process(runner, steps)
    worst = check_against_plain(model_folders[cfg], reqs, steps, got, dtype, _plain_cache)
    report(f"whole {cfg} {dtype}", worst)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", CONFIGS)
def test_last_32_one_by_one(model_folders, cfg, dtype):
    """Most of a request in one step, its last 32 tokens decoded one by one."""
    reqs = random_requests(TINY[cfg]["vocab_size"], [40, 97, 33], seed=2)
    portions = {r: [(0, len(t) - 32)] + [(i, i + 1) for i in range(len(t) - 32, len(t))] for r, t in reqs.items()}
    steps = trace_alone(reqs, portions)
    runner = runner_for(get_model(model_folders, cfg, dtype), 128)
    got = run_in_process(runner, steps)
    worst = check_against_plain(model_folders[cfg], reqs, steps, got, dtype, _plain_cache)
    report(f"last32 {cfg} {dtype}", worst)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", CONFIGS)
def test_portions_of_changing_size(model_folders, cfg, dtype):
    reqs = random_requests(TINY[cfg]["vocab_size"], [61, 100, 47], seed=3)
    sizes = {"r0": [7, 2, 5, 3, 2, 16, 2, 9], "r1": [2, 2, 31, 17, 1, 2, 15, 16, 3], "r2": [15, 1, 16, 2, 13]}
    steps = trace_alone(reqs, {r: cut(t, sizes[r]) for r, t in reqs.items()})
    runner = runner_for(get_model(model_folders, cfg, dtype), 128)
    got = run_in_process(runner, steps)
    worst = check_against_plain(model_folders[cfg], reqs, steps, got, dtype, _plain_cache)
    report(f"portions {cfg} {dtype}", worst)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", CONFIGS)
def test_mixed_batches_with_page_reuse(model_folders, cfg, dtype):
    """Up to four live requests, portions of some beside decoded tokens of others; the pool is only as large as
    the trace needs at its peak, so later requests get the pages of finished ones."""
    lengths = [31, 16, 7, 1, 50, 33, 64, 20, 45, 18]
    reqs = random_requests(TINY[cfg]["vocab_size"], lengths, seed=4)
    portions = {}
    for i, (r, t) in enumerate(reqs.items()):
        head = [8, 3, 2] if i % 2 == 0 else [5, 11]
        n_head = max(0, len(t) - 9)
        parts = [p for p in cut(t[:n_head], head)] if n_head else []
        parts += [(j, j + 1) for j in range(n_head, len(t))]   # the last tokens one by one
        portions[r] = parts
    steps = trace_mixed(reqs, portions, max_live=4, seed=5)
    pool = max_live_tokens(steps)
    runner = runner_for(get_model(model_folders, cfg, dtype), pool, max_requests=4)
    got = run_in_process(runner, steps)
    worst = check_against_plain(model_folders[cfg], reqs, steps, got, dtype, _plain_cache)
    report(f"mixed {cfg} {dtype} pool={pool}", worst)
    assert sum(runner.cache.held_pages()) == 0


@pytest.mark.parametrize("page_size", [1, 2, 4])
@pytest.mark.parametrize("cfg", ["B", "W"])
def test_small_pages_in_float32(model_folders, cfg, page_size):
    """Pages of 4 tokens (the workload of the second tiny configuration), of 2 and of 1 (the reference's default,
    vt-transformer/core/vt_scheduler.hpp:33; ids 0, 2 with pages of two, vt-transformer/test/vt_cache_test.cpp:108-116):
    all four ways of cutting the work in float32, whose attention kernel takes any page size."""
    dtype = "float32"
    model = get_model(model_folders, cfg, dtype)
    vocab = TINY[cfg]["vocab_size"]
    reqs = random_requests(vocab, [5, 13, 70], seed=71)
    steps = trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
    worst = check_against_plain(model_folders[cfg], reqs, steps, run_in_process(runner_for(model, 192, page_size=page_size), steps),
                                dtype, _plain_cache)
    reqs = random_requests(vocab, [40, 97], seed=72)
    steps = trace_alone(reqs, {r: [(0, len(t) - 32)] + [(i, i + 1) for i in range(len(t) - 32, len(t))] for r, t in reqs.items()})
    worst = max(worst, check_against_plain(model_folders[cfg], reqs, steps,
                                           run_in_process(runner_for(model, 128, page_size=page_size), steps), dtype, _plain_cache))
    reqs = random_requests(vocab, [61, 47], seed=73)
    sizes = {"r0": [7, 2, 5, 3, 2, 16, 2, 9], "r1": [15, 1, 16, 2, 13]}
    steps = trace_alone(reqs, {r: cut(t, sizes[r]) for r, t in reqs.items()})
    worst = max(worst, check_against_plain(model_folders[cfg], reqs, steps,
                                           run_in_process(runner_for(model, 128, page_size=page_size), steps), dtype, _plain_cache))
    reqs = random_requests(vocab, [31, 16, 7, 1, 50, 33, 20, 45], seed=74)
    portions = {}
    for i, (r, t) in enumerate(reqs.items()):
        n_head = max(0, len(t) - 9)
        portions[r] = (cut(t[:n_head], [8, 3, 2] if i % 2 == 0 else [5, 11]) if n_head else []) + \
            [(j, j + 1) for j in range(n_head, len(t))]
    steps = trace_mixed(reqs, portions, max_live=4, seed=75)
    pool = max_live_tokens(steps, round_to=max(page_size, 4))       # as few pages as the trace can do with
    runner = runner_for(model, pool, max_requests=4, page_size=page_size)
    worst = max(worst, check_against_plain(model_folders[cfg], reqs, steps, run_in_process(runner, steps), dtype, _plain_cache))
    assert sum(runner.cache.held_pages()) == 0
    report(f"page size {page_size} {cfg} {dtype}", worst)


def test_what_bfloat16_kernels_refuse_is_said_when_the_model_or_engine_is_built(model_folders, tmp_path):
    """Pages that are no multiple of 16 tokens and head sizes that are no multiple of 16: refused in bfloat16 before
    anything runs (and before weights are read), taken in float32."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import Engine, build_model, make_runner
    from vt_transformer_amd.weights import write_random_model
    (tmp_path / "cfg_only").mkdir()
    config_from_dict(dict(TINY["A"])).save(str(tmp_path / "cfg_only"))          # (no tensors: they are never asked for)
    with pytest.raises(ValueError, match="page size 4.*multiple of 16"):
        Engine(str(tmp_path / "cfg_only"), dtype="bfloat16", page_size=4)
    with pytest.raises(ValueError, match="page size 24"):
        make_runner(get_model(model_folders, "A", "bfloat16"), pool_tokens=96, page_size=24)
    odd = config_from_dict(dict(TINY["A"], head_dim=24, num_attention_heads=2, num_key_value_heads=1))
    with pytest.raises(ValueError, match="head size 24"):
        build_model(odd, "bfloat16")
    # float32 takes both: pages of 24 tokens, heads of 24
    folder = write_random_model(odd, str(tmp_path / "odd"), seed=3)
    reqs = random_requests(TINY["A"]["vocab_size"], [50], seed=76)
    steps = trace_alone(reqs, {r: cut(t, [20, 1, 1, 11, 2]) for r, t in reqs.items()})
    from vt_transformer_amd.engine import load_model
    runner = runner_for(load_model(folder, "float32"), 96, page_size=24)
    check_against_plain(folder, reqs, steps, run_in_process(runner, steps), "float32", {})


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cfg", ["A", "W"])
def test_long_decoding(model_folders, cfg, dtype):
    """Three tokens of prompt, then 300 tokens one by one, two requests side by side."""
    reqs = random_requests(TINY[cfg]["vocab_size"], [303, 280], seed=6)
    portions = {r: [(0, 3)] + [(i, i + 1) for i in range(3, len(t))] for r, t in reqs.items()}
    steps = trace_mixed(reqs, portions, max_live=2, seed=7, skip_prob=0.0)
    runner = runner_for(get_model(model_folders, cfg, dtype), 640)
    got = run_in_process(runner, steps)
    worst = check_against_plain(model_folders[cfg], reqs, steps, got, dtype, _plain_cache)
    report(f"long decoding {cfg} {dtype}", worst)


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens(model_folders, dtype):
    """The very first positions, each as a step of its own."""
    reqs = random_requests(TINY["B"]["vocab_size"], [4, 3], seed=8)
    steps = trace_alone(reqs, {r: [(i, i + 1) for i in range(len(t))] for r, t in reqs.items()})
    runner = runner_for(get_model(model_folders, "B", dtype), 64)
    got = run_in_process(runner, steps)
    check_against_plain(model_folders["B"], reqs, steps, got, dtype, _plain_cache)


def test_wanted_rows_equal_rows_of_all(model_folders):
    """Logits only at the wanted places are the same rows as when every place is wanted."""
    from vt_transformer_amd.engine import StepEntry
    model = get_model(model_folders, "B", "float32")
    toks = random_requests(TINY["B"]["vocab_size"], [23], seed=9)["r0"]
    r1 = runner_for(model, 64)
    r1.admit("x")
    full = r1.step([StepEntry("x", toks, list(range(23)))]).cpu()
    r2 = runner_for(model, 64)
    r2.admit("x")
    some = r2.step([StepEntry("x", toks, [22, 0, 7])]).cpu()
    assert torch.equal(some, full[[22, 0, 7]])
    r3 = runner_for(model, 64)
    r3.admit("x")
    assert r3.step([StepEntry("x", toks, [])]) is None


def test_fp32_does_not_depend_on_cut_or_batch(model_folders):
    """In float32 the same position gives bit-equal logits whole, token by token, and beside other requests."""
    from vt_transformer_amd.engine import StepEntry
    model = get_model(model_folders, "A", "float32")
    reqs = random_requests(TINY["A"]["vocab_size"], [37, 20], seed=10)
    a, b = reqs["r0"], reqs["r1"]
    r = runner_for(model, 256)
    r.admit("w")
    whole = r.step([StepEntry("w", a, [36])]).cpu()
    r.admit("s"); r.admit("o")
    r.step([StepEntry("s", a[:30], []), StepEntry("o", b[:5], [])])
    for i in range(30, 36):
        r.step([StepEntry("s", a[i:i + 1], []), StepEntry("o", b[5 + i - 30:6 + i - 30], [0])])
    last = r.step([StepEntry("o", b[11:13], [1]), StepEntry("s", a[36:37], [0])]).cpu()
    assert torch.equal(last[1], whole[0])


def rows_by_place(steps, got):
    """{(request, position): logits row} of a replayed trace."""
    out, pos = {}, {}
    for s in steps:
        row = 0
        for e in s["entries"]:
            p0 = pos.get(e["id"], 0)
            for wi in e["want"]:
                out[(e["id"], p0 + wi)] = got[s["step"]][row]
                row += 1
            pos[e["id"]] = p0 + len(e["tokens"])
    return out


@pytest.mark.parametrize("cfg", CONFIGS)
def test_float32_rows_are_bit_equal_under_every_cutting(model_folders, cfg):
    """In float32 a position's logits are the same bits however its request is cut into steps, whatever else is in
    the batch and whichever pages hold it (the reference has one program for prompts and for decoding,
    v1/models/qwen2-7b/inference_fp16.dag:368-396): every wanted row of the last-32-one-by-one, the changing-portions
    and the mixed replay (four live requests, pages used again) against the same place's row of the whole run."""
    vocab = TINY[cfg]["vocab_size"]
    reqs = random_requests(vocab, [61, 100, 47, 33, 70, 18], seed=23)
    model = get_model(model_folders, cfg, "float32")
    whole_steps = trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
    whole = rows_by_place(whole_steps, run_in_process(runner_for(model, 128), whole_steps))
    assert len(whole) == sum(len(t) for t in reqs.values())
    sizes = [[7, 2, 5, 3, 2, 16, 2, 9], [2, 2, 31, 17, 1, 2, 15, 16, 3], [15, 1, 16, 2, 13], [33], [1, 64, 5], [2]]
    modes = {
        "last 32 one by one": trace_alone(reqs, {r: ([(0, len(t) - 32)] if len(t) > 32 else []) +
                                                 [(i, i + 1) for i in range(max(0, len(t) - 32), len(t))]
                                                 for r, t in reqs.items()}),
        "portions": trace_alone(reqs, {r: cut(t, sizes[i]) for i, (r, t) in enumerate(reqs.items())}),
        "mixed": trace_mixed(reqs, {r: cut(t[:max(0, len(t) - 9)], [8, 3, 2] if i % 2 == 0 else [5, 11]) +
                                    [(j, j + 1) for j in range(max(0, len(t) - 9), len(t))]
                                    for i, (r, t) in enumerate(reqs.items())}, max_live=4, seed=29),
    }
    for name, steps in modes.items():
        pool = max_live_tokens(steps) if name == "mixed" else 128
        runner = runner_for(model, pool, max_requests=4)
        rows = rows_by_place(steps, run_in_process(runner, steps))
        assert set(rows) == set(whole), name
        for place, row in rows.items():
            assert np.array_equal(row, whole[place]), f"{cfg} {name}: request {place[0]} position {place[1]} differs " \
                f"from the whole run by {np.abs(row - whole[place]).max():.3e}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_run_program(model_folders, dtype, tmp_path):
    """The replay program itself, as a child process fed step by step."""
    cfg = "B"
    reqs = random_requests(TINY[cfg]["vocab_size"], [20, 35, 9, 41, 12], seed=11)
    portions = {r: cut(t, [6, 2, 9, 1]) for r, t in reqs.items()}
    steps = trace_mixed(reqs, portions, max_live=4, seed=12)
    steps[1]["entries"][0]["want"] = []          # a step may want nothing from an entry
    got = run_trace_run(model_folders[cfg], dtype, steps, str(tmp_path / "out"), max_live_tokens(steps),
                        TINY[cfg]["vocab_size"])
    worst = check_against_plain(model_folders[cfg], reqs, steps, got, dtype, _plain_cache)
    report(f"trace_run {cfg} {dtype}", worst)
    # most of each request in one step, its last tokens one by one beside the others' (decoding steps, which the
    # program runs through captured graphs as the engine does), with so few pages that they are used again
    reqs = random_requests(TINY[cfg]["vocab_size"], [40, 33, 52, 45, 38, 47], seed=13)
    portions = {r: [(0, len(t) - 14)] + [(j, j + 1) for j in range(len(t) - 14, len(t))] for r, t in reqs.items()}
    steps = trace_mixed(reqs, portions, max_live=3, seed=14)
    got = run_trace_run(model_folders[cfg], dtype, steps, str(tmp_path / "out2"), max_live_tokens(steps),
                        TINY[cfg]["vocab_size"])
    worst = check_against_plain(model_folders[cfg], reqs, steps, got, dtype, _plain_cache)
    report(f"trace_run decode {cfg} {dtype}", worst)


@pytest.mark.parametrize("dtype", DTYPES)
def test_random_weights_drawn_on_the_device_are_the_written_folders_model(dtype, tmp_path):
    """`random_model(config, seed)` draws its tensors on the device, the only way a model of 145 GB can be made;
    `write_random_model(config, folder, seed)` draws them on the host.  Both use one counter-based generator, so
    they are the same model: the device's one, under all four ways of cutting the work, against the plain
    implementation reading the written folder."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import random_model
    from vt_transformer_amd.weights import write_random_model
    cfg = "B"
    folder = write_random_model(config_from_dict(dict(TINY[cfg])), str(tmp_path / "m"), seed=77)
    model = random_model(config_from_dict(dict(TINY[cfg])), seed=77, dtype=dtype)
    vocab = TINY[cfg]["vocab_size"]
    cache = {}
    # whole; last 32 one by one; portions of changing size; mixed with page reuse
    reqs = random_requests(vocab, [9, 70], seed=61)
    steps = trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
    worst = check_against_plain(folder, reqs, steps, run_in_process(runner_for(model, 128), steps), dtype, cache)
    reqs = random_requests(vocab, [50], seed=62)
    steps = trace_alone(reqs, {r: [(0, len(t) - 32)] + [(i, i + 1) for i in range(len(t) - 32, len(t))] for r, t in reqs.items()})
    worst = max(worst, check_against_plain(folder, reqs, steps, run_in_process(runner_for(model, 64), steps), dtype, cache))
    reqs = random_requests(vocab, [61], seed=63)
    steps = trace_alone(reqs, {r: cut(t, [7, 2, 5, 3, 2, 16, 2, 9]) for r, t in reqs.items()})
    worst = max(worst, check_against_plain(folder, reqs, steps, run_in_process(runner_for(model, 64), steps), dtype, cache))
    reqs = random_requests(vocab, [31, 16, 7, 50, 33, 20], seed=64)
    portions = {r: cut(t[:max(0, len(t) - 6)], [8, 3, 2]) + [(j, j + 1) for j in range(max(0, len(t) - 6), len(t))]
                for r, t in reqs.items()}
    steps = trace_mixed(reqs, portions, max_live=4, seed=65)
    runner = runner_for(model, max_live_tokens(steps), max_requests=4)
    worst = max(worst, check_against_plain(folder, reqs, steps, run_in_process(runner, steps), dtype, cache))
    report(f"random_model {cfg} {dtype}", worst)


# ---------------------------------------------------------------------------
# the entry point: scheduler, step function and sampler together
# ---------------------------------------------------------------------------
def test_greedy_generation_through_entry_point(model_folders):
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    cfg = "A"
    pc, pw = plain_model.read_folder(model_folders[cfg])
    prompts = list(random_requests(TINY[cfg]["vocab_size"], [5, 9, 13], seed=20).values())
    want = [plain_model.greedy(pc, pw, p, 8) for p in prompts]
    eng = Engine(model_folders[cfg], dtype="float32", num_pages=12, max_running_reqs=3, max_seq_len=64)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    assert got == want
    assert sum(eng.runner.cache.held_pages()) == 0
    # bfloat16: every chosen token is the plain model's best or within rounding of it
    eng = Engine(model_folders[cfg], dtype="bfloat16", num_pages=12, max_running_reqs=3, max_seq_len=64)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    for p, g in zip(prompts, got):
        logits = plain_model.forward(pc, pw, p + g)
        for i, tok in enumerate(g):
            row = logits[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= TOL_BF16 * float(row.abs().max())


def test_chunked_prompts_mixed_with_decoding_and_temperature(model_folders):
    """Prompts of 1/7/16/31 tokens in portions of 8 beside decoding requests, temperature 0.8 from a fixed seed:
    the same tokens whatever the batch looks like (alone, together, preempted)."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    cfg = "B"
    prompts = list(random_requests(TINY[cfg]["vocab_size"], [1, 7, 16, 31], seed=21).values())
    sp = [SamplingParams(temperature=0.8, max_tokens=8, ignore_eos=True, seed=1000 + i) for i in range(4)]
    together = Engine(model_folders[cfg], dtype="float32", num_pages=32, max_running_reqs=4, max_seq_len=128,
                      chunk_size=8, max_extend_tokens=12)
    got = together.generate(prompts, sp)
    for i, p in enumerate(prompts):
        alone = Engine(model_folders[cfg], dtype="float32", num_pages=8, max_running_reqs=1, max_seq_len=128)
        assert alone.generate([p], [sp[i]])[0] == got[i]


def test_preemption_recomputes_the_same_tokens(model_folders):
    """Three pages for two requests that each grow into a second page while decoding: the younger one is
    preempted, gives its pages back, waits, and is recomputed from its prompt and the tokens it had produced.
    Its tokens are those it produces alone."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    cfg = "B"
    prompts = list(random_requests(TINY[cfg]["vocab_size"], [15, 16], seed=23).values())
    sp = [SamplingParams(temperature=0.8, max_tokens=8, ignore_eos=True, seed=2000 + i) for i in range(2)]
    alone = []
    for i, p in enumerate(prompts):
        eng = Engine(model_folders[cfg], dtype="float32", num_pages=4, max_running_reqs=1, max_seq_len=128)
        alone.append(eng.generate([p], [sp[i]])[0])
    tight = Engine(model_folders[cfg], dtype="float32", num_pages=3, max_running_reqs=4, max_seq_len=128)
    assert tight.generate(prompts, sp) == alone
    assert tight.scheduler.counters["preemptions"] > 0
    assert tight.requests[1].preemptions > 0 and tight.requests[0].preemptions == 0
    assert sum(tight.runner.cache.held_pages()) == 0


def test_tight_engine_with_arrivals_gives_each_request_what_it_gets_alone(model_folders):
    """Ten to thirty requests arrive while the engine runs, with few pages, few live requests, short portions and a
    small token budget, so that prompts are cut, mixed with decoding, and requests are preempted and recomputed.
    In float32 with temperature sampling every request gets exactly the tokens it gets alone, and no page is left."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    preemptions = 0
    for trial, cfg in [(0, "A"), (1, "B"), (2, "W")]:
        rs = np.random.RandomState(trial)
        n = int(rs.randint(10, 30))
        prompts = [rs.randint(0, TINY[cfg]["vocab_size"], size=int(rs.randint(1, 120))).tolist() for _ in range(n)]
        sps = [SamplingParams(temperature=0.8, top_k=int(rs.choice([-1, 5])), max_tokens=int(rs.randint(1, 40)), ignore_eos=True,
                              seed=100 + i) for i in range(n)]
        one = Engine(model_folders[cfg], dtype="float32", num_pages=64, max_running_reqs=1, max_seq_len=256)
        alone = [one.generate([p], [sp])[0] for p, sp in zip(prompts, sps)]
        eng = Engine(model_folders[cfg], dtype="float32", num_pages=int(rs.randint(11, 15)), max_running_reqs=int(rs.randint(4, 9)),
                     max_seq_len=256, chunk_size=int(rs.choice([8, 16, 32, 64])), max_extend_tokens=int(rs.choice([16, 48, 128])))
        pending, steps = list(range(n)), 0
        while pending or eng.has_work():
            for _ in range(int(rs.randint(0, 4))):
                if pending:
                    i = pending.pop(0)
                    eng.add_request(prompts[i], sps[i], uid=i)
            if eng.has_work():
                eng.step()
                steps += 1
            assert steps < 5000, "the engine does not finish"
        assert [eng.requests[i].output for i in range(n)] == alone, (trial, cfg)
        assert sum(eng.runner.cache.held_pages()) == 0
        preemptions += eng.scheduler.counters["preemptions"]
    assert preemptions > 0      # the draws above leave too few pages for the live requests


@pytest.mark.parametrize("cfg", ["A", "W"])
def test_decoding_ahead_of_the_host_gives_the_same_tokens(cfg, tmp_path):
    """The engine starts the next decoding step before this one's tokens have reached the host.  With requests
    that end at different times (end-of-sequence tokens, output limits of their own), with temperature and without,
    it produces exactly the tokens and finish reasons of the engine that waits for every step."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    from vt_transformer_amd.weights import write_random_model
    vocab = TINY[cfg]["vocab_size"]
    d = dict(TINY[cfg], eos_token_id=list(range(3, vocab, 9)))          # one token in nine ends a request
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(d), folder, seed=17)
    rs = np.random.RandomState(5)
    prompts = [rs.randint(0, vocab, size=int(rs.randint(3, 40))).tolist() for _ in range(12)]
    sps = [SamplingParams(temperature=float(rs.choice([0.0, 0.9])), top_k=int(rs.choice([-1, 8])),
                          max_tokens=int(rs.randint(2, 40)), ignore_eos=bool(i % 4 == 0), seed=300 + i) for i in range(12)]
    outs = []
    for ahead in (False, True):
        eng = Engine(folder, dtype="bfloat16", num_pages=64, max_running_reqs=12, max_seq_len=128)
        eng.pipeline_decode = ahead
        launched = []
        orig = eng._launch
        eng._launch = lambda plan, ids, orig=orig: (launched.append(ids is not None), orig(plan, ids))[1]
        toks = eng.generate(prompts, sps)
        outs.append((toks, [eng.finish_reason(i) for i in range(12)]))
        assert any(launched) == ahead                                   # steps were started ahead, or none was
        assert sum(eng.runner.cache.held_pages()) == 0 and not eng.has_work()
    assert outs[0] == outs[1]
    reasons = set(outs[0][1])
    assert "eos" in reasons and "max_tokens" in reasons                 # both ways of ending happened


def test_decoding_ahead_stops_at_a_page_edge_when_no_page_is_free(model_folders):
    """The only running request decodes ahead of the host with every page taken and crosses a page's edge: the step
    ahead is not launched, and the request ends for want of pages (alone) or its neighbour is preempted (two of
    them); Engine.step never raises."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    cfg = "A"
    rs = np.random.RandomState(21)
    vocab = TINY[cfg]["vocab_size"]
    # alone: 2 pages of 16 tokens, a prompt of 23: token 33 has no page
    eng = Engine(model_folders[cfg], dtype="bfloat16", num_pages=2, max_running_reqs=2, max_seq_len=128)
    ahead = []
    orig = eng._launch
    eng._launch = lambda plan, ids: (ahead.append(ids is not None), orig(plan, ids))[1]
    out = eng.generate([rs.randint(0, vocab, size=23).tolist()], SamplingParams(max_tokens=40, ignore_eos=True))
    assert any(ahead) and eng.finish_reason(0) == "out_of_pages" and len(out[0]) == 10
    assert sum(eng.runner.cache.held_pages()) == 0 and not eng.has_work()
    # two requests and three pages: both stand at a page's edge with one page free; the younger gives way
    eng = Engine(model_folders[cfg], dtype="bfloat16", num_pages=3, max_running_reqs=2, max_seq_len=128)
    eng.pipeline_decode = True
    prompts = [rs.randint(0, vocab, size=9).tolist() for _ in range(2)]
    sp = SamplingParams(max_tokens=12, ignore_eos=True)
    outs = eng.generate(prompts, sp)
    assert [eng.finish_reason(i) for i in (0, 1)] == ["max_tokens"] * 2 and eng.requests[1].preemptions >= 1
    one = Engine(model_folders[cfg], dtype="bfloat16", num_pages=4, max_running_reqs=1, max_seq_len=128)
    # (the request that was never disturbed has the tokens it gets alone; the other was recomputed through the
    # prompt kernels, whose rounding may break a near-tie the other way)
    assert outs[0] == one.generate(prompts[0], sp)[0] and len(outs[1]) == 12


def test_decoding_ahead_with_arrivals_aborts_and_few_pages(model_folders):
    """Steps started ahead while requests arrive, are aborted and are preempted for want of pages: every request
    ends with a reason, within its limit, no page or slot stays held, and requests that were never disturbed
    (no preemption) have the tokens they get alone."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    cfg = "B"
    rs = np.random.RandomState(9)
    n = 24
    prompts = [rs.randint(0, TINY[cfg]["vocab_size"], size=int(rs.randint(1, 60))).tolist() for _ in range(n)]
    sps = [SamplingParams(temperature=0.0, max_tokens=int(rs.randint(1, 50)), ignore_eos=True, seed=i) for i in range(n)]
    eng = Engine(model_folders[cfg], dtype="bfloat16", num_pages=8, max_running_reqs=6, max_seq_len=128, chunk_size=32,
                 max_extend_tokens=64)
    ahead = []
    orig = eng._launch
    eng._launch = lambda plan, ids: (ahead.append(ids is not None), orig(plan, ids))[1]
    pending, aborted, steps = list(range(n)), set(), 0
    while pending or eng.has_work():
        for _ in range(int(rs.randint(0, 3))):
            if pending:
                i = pending.pop(0)
                eng.add_request(prompts[i], sps[i], uid=i)
        if steps % 7 == 3:
            live = [u for u, r in eng.requests.items() if r.state == "running" and u not in aborted]
            if live:
                u = live[int(rs.randint(0, len(live)))]
                assert eng.abort_request(u)
                aborted.add(u)
        eng.step()
        steps += 1
        assert steps < 5000, "the engine does not finish"
    assert any(ahead) and sum(eng.runner.cache.held_pages()) == 0
    assert eng.runner.cache.slots.available == 6
    one = Engine(model_folders[cfg], dtype="bfloat16", num_pages=16, max_running_reqs=1, max_seq_len=128, chunk_size=32,
                 max_extend_tokens=64)
    one.pipeline_decode = False
    pcfg, pw = plain_model.read_folder(model_folders[cfg])
    checked = 0
    for i in range(n):
        r = eng.requests[i]
        assert r.state == "finished" and r.finish_reason in ("max_tokens", "abort", "max_seq_len")
        assert len(r.output) <= sps[i].max_tokens
        if r.finish_reason == "max_tokens":
            assert len(r.output) == sps[i].max_tokens
            if r.preemptions == 0:
                # alone it goes through other kernels where it shared steps with others (rows per product), so a
                # near tie may fall the other way: where the tokens part, the two candidates' logits are close
                alone = one.generate([prompts[i]], [sps[i]])[0]
                if alone != r.output:
                    j = next(k for k in range(len(alone)) if alone[k] != r.output[k])
                    lg = plain_model.forward(pcfg, pw, prompts[i] + alone[:j])[-1]
                    assert float(abs(lg[alone[j]] - lg[r.output[j]]) / lg.abs().max()) < 2e-2, (i, j)
                    assert float((lg.max() - max(lg[alone[j]], lg[r.output[j]])) / lg.abs().max()) < 2e-2, (i, j)
                checked += 1
    assert checked >= 3 and eng.scheduler.counters["preemptions"] > 0 and aborted


def test_decode_graph_replays_match_eager(model_folders):
    """Captured decoding steps against the same steps launched one by one: several replays, with eager work
    (prompt portions of other requests, synchronisations) between them, all equal."""
    from vt_transformer_amd.engine import StepEntry
    model = get_model(model_folders, "A", "bfloat16")
    reqs = random_requests(TINY["A"]["vocab_size"], [60, 45, 30], seed=22)
    eager, graph = runner_for(model, 512), runner_for(model, 512)
    graph.decode_graphs = True
    for r in (eager, graph):
        for rid, toks in reqs.items():
            r.admit(rid)
            r.step([StepEntry(rid, toks[:20], [])])
    for i in range(20, 30):
        entries = [StepEntry(rid, toks[i:i + 1], [0]) for rid, toks in reqs.items()]
        a = eager.step(entries).clone()
        b = graph.step(entries).clone()
        torch.cuda.synchronize()
        assert torch.equal(a, b), f"decode step {i}"
        if i % 3 == 0:   # eager work between replays: another request's portion through both runners
            for r in (eager, graph):
                r.admit(f"x{i}")
                r.step([StepEntry(f"x{i}", reqs["r0"][:17], [16])])
                r.release(f"x{i}")
    # fewer entries than the captured batch: the padding entries must not disturb the real ones
    e2 = [StepEntry("r0", reqs["r0"][30:31], [0]), StepEntry("r1", reqs["r1"][30:31], [0])]
    e3 = e2 + [StepEntry("r2", reqs["r2"][29:30] if False else [reqs["r2"][29]], [0])]
    a = eager.step(e3).clone()
    b = graph.step(e3).clone()
    assert torch.equal(a, b)
    assert len(graph._graphs) >= 1


def test_a_request_name_used_again_does_not_decode_against_the_old_requests_pages(model_folders):
    """A captured decoding step's metadata is patched from one step to the next when the same requests go on.  A
    request that ended and a new one admitted under its name are not the same request, even if the new one is just
    as long as the old one was: its pages are others (the pool hands them out last-in-first-out)."""
    from vt_transformer_amd.engine import StepEntry
    cfg = "B"
    model = get_model(model_folders, cfg, "bfloat16")
    pc, pw = plain_model.read_folder(model_folders[cfg])
    runner = runner_for(model, 256, max_requests=2)
    runner.decode_graphs = True
    first = random_requests(TINY[cfg]["vocab_size"], [41], seed=51)["r0"]
    second = random_requests(TINY[cfg]["vocab_size"], [42], seed=52)["r0"]
    assert runner.admit("r")
    runner.step([StepEntry("r", first[:40], [])])
    got1 = runner.step([StepEntry("r", first[40:41], [0])]).float().cpu()
    runner.release("r")
    assert runner.admit("r")
    runner.step([StepEntry("r", second[:41], [])])
    assert runner.cache.get("r").tables[0] != [0, 1, 2]         # (other pages than the first request had)
    got2 = runner.step([StepEntry("r", second[41:42], [0])]).float().cpu()
    assert len(runner._graphs) == 1
    for toks, got in ((first, got1), (second, got2)):
        ref = plain_model.forward(pc, pw, toks)[-1]
        assert float((got[0].double() - ref).abs().max() / ref.abs().max()) < TOL_BF16


def test_prompts_that_fit_alone_but_not_together_finish_with_their_own_tokens(model_folders):
    """Four pages of four tokens, portions of four, two prompts of twelve: admitted together they would hold every
    page half-way through.  Both finish, with the tokens each gets alone."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    cfg = "B"
    prompts = list(random_requests(TINY[cfg]["vocab_size"], [12, 12], seed=53).values())
    sp = [SamplingParams(temperature=0.8, max_tokens=3, ignore_eos=True, seed=3000 + i) for i in range(2)]
    alone = []
    for i, p in enumerate(prompts):
        eng = Engine(model_folders[cfg], dtype="float32", num_pages=4, page_size=4, max_running_reqs=1, max_seq_len=16)
        alone.append(eng.generate([p], [sp[i]])[0])
    eng = Engine(model_folders[cfg], dtype="float32", num_pages=4, page_size=4, chunk_size=4, max_extend_tokens=8,
                 max_running_reqs=4, max_seq_len=16)
    steps = 0
    for p, s in zip(prompts, sp):
        eng.add_request(p, s)
    while eng.has_work():
        eng.step()
        steps += 1
        assert steps < 100, "the engine does not finish"
    assert [eng.requests[i].output for i in range(2)] == alone
    assert [eng.requests[i].finish_reason for i in range(2)] == ["max_tokens"] * 2
    assert sum(eng.runner.cache.held_pages()) == 0


def test_group_of_17_query_heads_is_not_replayed_and_right(tmp_path):
    """More query heads per kv head than the decoding kernels' one tile of 16 rows: the model says that its steps
    cannot be replayed, decoding goes through the planned kernel step by step, and the logits are those of the
    plain implementation."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.engine import StepEntry, load_model
    from vt_transformer_amd.weights import write_random_model
    d = dict(TINY["A"], num_attention_heads=17, num_key_value_heads=1, head_dim=16, hidden_size=48, num_hidden_layers=2)
    folder = str(tmp_path / "g17")
    write_random_model(config_from_dict(d), folder, seed=9)
    cfg, w = plain_model.read_folder(folder)
    toks = random_requests(d["vocab_size"], [40], seed=3)["r0"]
    ref = plain_model.forward(cfg, w, toks)
    for dtype, tol in (("float32", 2e-5), ("bfloat16", TOL_BF16)):
        runner = runner_for(load_model(folder, dtype), 128)
        runner.decode_graphs = True
        assert not runner._replayable
        runner.admit("r")
        got = [runner.step([StepEntry("r", toks[:25], list(range(25)))]).cpu()]
        for i in range(25, 40):
            got.append(runner.step([StepEntry("r", toks[i:i + 1], [0])]).cpu())
        assert not runner._graphs
        got = torch.cat(got).double()
        assert float((got - ref).abs().max() / ref.abs().max()) < tol, dtype


def test_single_weight_copy_gives_the_same_logits(model_folders):
    """With the matrices kept once (packed) instead of twice, portions of up to 255 rows go through the few-row kernels
    64 rows at a time, longer ones unpack each matrix into scratch memory for the GEMM library: the same logits to
    rounding as with two copies, no row-major matrix left on the device."""
    from vt_transformer_amd.engine import Engine, StepEntry
    toks = random_requests(TINY["W"]["vocab_size"], [480], seed=31)["r0"]
    logits = []
    for single in (False, True):
        eng = Engine(model_folders["W"], dtype="bfloat16", num_pages=40, max_running_reqs=2, max_seq_len=512,
                     single_weight_copy=single)
        mixer = eng.model.layers[0].mixer
        assert (mixer.w_qkv is None) == single and mixer.p_qkv is not None
        assert (eng.model.layers[0].feed_forward.w_down is None) == single
        eng.runner.admit("x")
        out = [eng.runner.step([StepEntry("x", toks[:150], list(range(150)))]).float().cpu()]               # few-row kernels
        out += [eng.runner.step([StepEntry("x", toks[150:450], list(range(0, 300, 3)))]).float().cpu()]     # unpacked
        out += [eng.runner.step([StepEntry("x", toks[i:i + 1], [0])]).float().cpu() for i in range(450, 460)]
        logits.append(torch.cat(out))
        assert ("linear.unpacked" in eng.model.rt._buffers) == single
    assert float((logits[0] - logits[1]).abs().max() / logits[0].abs().max()) < 2e-2
    cfg, w = plain_model.read_folder(model_folders["W"])
    ref = plain_model.forward(cfg, w, toks[:460])
    rows = list(range(150)) + list(range(150, 450, 3)) + list(range(450, 460))
    assert float((logits[1].double() - ref[rows]).abs().max() / ref.abs().max()) < TOL_BF16


def test_library_algorithm_search_keeps_results(model_folders):
    """With the GEMM library's algorithm search on, a long portion gives the plain implementation's logits, as
    without it."""
    from vt_transformer_amd.engine import Engine, StepEntry
    toks = random_requests(TINY["B"]["vocab_size"], [150], seed=30)["r0"]
    pc, pw = plain_model.read_folder(model_folders["B"])
    ref = plain_model.forward(pc, pw, toks)[[149, 70]]
    for tune in (False, True):
        eng = Engine(model_folders["B"], dtype="bfloat16", num_pages=32, max_running_reqs=2, max_seq_len=256,
                     chunk_size=128, tune_gemm=tune)
        eng.runner.admit("x")
        got = eng.runner.step([StepEntry("x", toks, [149, 70])]).float().cpu().double()
        assert sum(eng.runner.cache.held_pages()) == 10
        assert float((got - ref).abs().max() / ref.abs().max()) < TOL_BF16, tune


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_long_prompt_whole_and_in_two_portions(model_folders, dtype):
    """1,800 tokens: in bfloat16 the last rows' keys are cut into ranges that are merged afterwards (whole: a fresh
    portion; in two portions: the second one has 1,000 keys in the cache in front of it)."""
    from vt_transformer_amd.engine import StepEntry, load_model
    cfg = "B"
    toks = random_requests(TINY[cfg]["vocab_size"], [1800], seed=41)["r0"]
    pc, pw = plain_model.read_folder(model_folders[cfg])
    rows = list(range(0, 1800, 37)) + [1799]
    ref = plain_model.forward(pc, pw, toks)[rows]
    model = load_model(model_folders[cfg], dtype)
    tol = 3e-5 if dtype == "float32" else TOL_BF16
    for cuts in ([(0, 1800)], [(0, 1000), (1000, 1800)]):
        r = runner_for(model, 1856, max_requests=2)
        r.admit("x")
        got = torch.cat([r.step([StepEntry("x", toks[a:b], [i - a for i in rows if a <= i < b])]).float().cpu() for a, b in cuts])
        err = float((got.double() - ref).abs().max() / ref.abs().max())
        assert err < tol, (cuts, err)
    # (the planner does cut this shape: three kv heads, one query head each, head size 32)
    from vt_transformer_amd.parts.attention_plan import plan_tile_items
    for pos0, n in ((0, 1800), (1000, 800)):
        _, _, citems, n_parts = plan_tile_items(np.array([0, n], np.int32), np.array([pos0], np.int32), 1, 0, 3,
                                                np.arange(1), head_dim=32)
        assert n_parts > 0 and len(citems) > 0


@pytest.mark.parametrize("dtype", ["float16", "bfloat16"])
@pytest.mark.parametrize("stream,gain", [(3000.0, 12.0), (1e-4, 0.05)])
def test_streams_and_gains_far_from_one(tmp_path, dtype, stream, gain):
    """A residual stream of thousands under norm gains above ten (massive activations of a real checkpoint), and one
    of 1e-4 under gains of 0.05: the stream times the gains leaves float16's range (65,504) or its normal numbers
    (6e-5), while the normalised value that the reference rounds ((w * x) * r, v1/tensortype/hip_kernels/rmsnorm.cpp:28-41)
    does not.  Whole prompts, decoding one by one (up to 16 rows) and a portion of 40 rows (17 to 64), against the
    float64 model."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights import write_random_model
    from vt_transformer_amd.weights.safetensors_io import WeightStore, write_safetensors
    from vt_transformer_amd.engine import load_model
    cfg = dict(TINY["B"], hidden_size=256, intermediate_size=384, num_attention_heads=4, num_key_value_heads=2,
               head_dim=64, num_hidden_layers=2)
    folder = str(tmp_path / "m")
    write_random_model(config_from_dict(cfg), folder, seed=31)
    store = WeightStore(folder)
    g = torch.Generator().manual_seed(3)
    tensors = []
    for name in store.names():
        t = store.get(name).float()
        if name.endswith("embed_tokens.weight"):
            t = torch.randn(t.shape, generator=g) * stream
        elif "norm" in name:
            t = gain * (1.0 + 0.3 * torch.rand(t.shape, generator=g))
        tensors.append((name, t.to(torch.bfloat16)))
    store.close()
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    vocab = cfg["vocab_size"]
    reqs = random_requests(vocab, [60, 45], seed=8)
    portions = {"r0": [(0, 40)] + [(i, i + 1) for i in range(40, 60)], "r1": [(0, 45)]}
    steps = trace_alone(reqs, portions)
    runner = runner_for(load_model(folder, dtype), 128)
    got = run_in_process(runner, steps)
    worst = check_against_plain(folder, reqs, steps, got, dtype, {})
    report(f"stream {stream:g} gain {gain:g} {dtype}", worst)
