"""Host-side pieces of the step: the attention work planner, the decode chunk, the sampler's uniform numbers."""
import numpy as np
import pytest

from vt_transformer_amd.parts.attention_plan import decode_chunk, plan_attention_items, plan_tile_items, split_entries
from vt_transformer_amd.sampling import SamplingParams, request_seed, uniform


@pytest.mark.parametrize("group,window", [(1, 0), (7, 0), (2, 5), (5, 40), (3, 16)])
@pytest.mark.parametrize("target", [0, 2048, 10 ** 9])
@pytest.mark.parametrize("rt", [1, 2])
def test_every_row_gets_every_key_it_may_see_exactly_once(group, window, target, rt):
    lens = np.array([1, 37, 1, 2, 19, 130])
    pos0 = np.array([300, 0, 0, 16, 45, 7])
    start = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    items, citems, n_parts = plan_attention_items(start, pos0.astype(np.int32), group, window, 2, target_waves=target,
                                                  min_chunk=16, rt=rt)
    covered = {}
    for entry, q_tok0, q_len, p0, row0, lo, hi, part in items.tolist():
        assert q_tok0 == start[entry] and q_len == lens[entry] and p0 == pos0[entry]
        assert lo % 16 == 0 and lo < hi
        for r in range(row0, min(row0 + 16 * rt, q_len * group)):
            p = p0 + r // group
            first = max(0, p - window + 1) if window else 0
            keys = covered.setdefault((entry, r), [])
            keys.extend(j for j in range(lo, hi) if first <= j <= p)
    for e in range(len(lens)):
        for r in range(lens[e] * group):
            p = pos0[e] + r // group
            first = max(0, p - window + 1) if window else 0
            assert sorted(covered[(e, r)]) == list(range(first, p + 1)), (e, r)
    # partial indices: each used by one item; every 16-row tile of a split item is merged once over exactly its items
    parts = [it[7] for it in items.tolist() if it[7] >= 0]
    assert len(parts) == len(set(parts)) and all(p < n_parts for p in parts)
    by_part = {it[7]: it for it in items.tolist() if it[7] >= 0}
    merged = {}
    for q_tok0, q_len, r0, part0, n, sub in citems.tolist():
        assert 2 <= n <= 128 and 0 <= sub < rt
        for pi in range(part0, part0 + n):
            it = by_part[pi]
            assert it[1] == q_tok0 and it[4] + 16 * sub == r0 and r0 < q_len * group
            merged.setdefault(pi, []).append(sub)
    for pi, it in by_part.items():
        tiles = [s_ for s_ in range(rt) if it[4] + 16 * s_ < it[2] * group]
        assert sorted(merged[pi]) == tiles
    if target == 0:
        assert len(citems) == 0


@pytest.mark.parametrize("group,window", [(1, 0), (7, 0), (5, 40)])
@pytest.mark.parametrize("rt", [1, 2])
@pytest.mark.parametrize("split", [0., 0.5, 1.4, None])
@pytest.mark.parametrize("direct", [False, True])
def test_tile_items_cover_the_long_entries(group, window, rt, split, direct):
    """Every row of a long entry meets every key it may see exactly once, whether or not the keys of the longest
    items are cut into ranges; the ranges of an item have consecutive partial indices and one merge per 16-row tile."""
    lens = np.array([1, 300, 40, 2048, 260])
    pos0 = np.array([300, 0, 10, 77, 5000])
    start = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    short, long = split_entries(start, group)
    assert sorted(list(short) + list(long)) == list(range(5))
    assert all(lens[e] * group >= 256 for e in long) and all(lens[e] * group < 256 for e in short)
    items, got_rt, citems, n_parts = plan_tile_items(start, pos0.astype(np.int32), group, window, 4, long,
                                                     rt=rt if split is not None else None, split=split, direct=direct)
    if split is not None:
        assert got_rt == rt
    rt = got_rt
    spans = [it[6] - it[5] for it in items.tolist()]
    assert spans == sorted(spans, reverse=True)                       # the longest first
    if split == 0.:
        assert n_parts == 0 and len(citems) == 0 and all(it[7] == -1 for it in items.tolist())
    if split == 0.5 and window == 0:
        assert n_parts > 0                      # (under a window of 40 no row sees keys enough to cut)
    seen = {}            # (entry, row) -> key ranges
    by_item = {}         # (entry, row0) -> [(lo, hi, part)]
    for entry, q_tok0, q_len, p0, row0, lo, hi, part in items.tolist():
        assert lo % 16 == 0 and q_tok0 == start[entry] and hi > lo and -1 <= part < n_parts
        by_item.setdefault((entry, row0), []).append((lo, hi, part))
    for (entry, row0), ranges in by_item.items():
        ranges.sort()
        assert all(a[1] == b[0] for a, b in zip(ranges, ranges[1:]))         # the ranges follow each other
        if len(ranges) == 1:
            assert ranges[0][2] == -1
        else:
            assert [r_[2] for r_ in ranges] == list(range(ranges[0][2], ranges[0][2] + len(ranges)))
        lo, hi = ranges[0][0], ranges[-1][1]
        for r_ in range(row0, min(row0 + 64 * rt, lens[entry] * group)):
            p = pos0[entry] + r_ // group
            first = max(0, p - window + 1) if window else 0
            assert lo <= first and p < hi                               # all the keys the row may see are inside
            assert (entry, r_) not in seen
            seen[(entry, r_)] = True
    assert set(seen) == {(e, r_) for e in long for r_ in range(lens[e] * group)}
    # merges: one per existing 16-row tile of every cut item, naming its first partial index and number of ranges
    want = set()
    for (entry, row0), ranges in by_item.items():
        if len(ranges) > 1:
            for t in range(4 * rt):
                if row0 + 16 * t < lens[entry] * group:
                    want.add((int(start[entry]), int(lens[entry]), row0 + 16 * t, ranges[0][2], len(ranges), t))
    assert {tuple(c) for c in citems.tolist()} == want and len(citems) == len(want)
    used = sorted(p for rs in by_item.values() for _, _, p in rs if p >= 0)
    assert len(set(used)) == len(used) and all(p < n_parts for p in used)


def test_decode_chunk():
    from vt_transformer_amd.parts.attention_plan import decode_parts_max
    assert decode_chunk(np.array([1]), 16) == 64
    c = decode_chunk(np.array([8192]), 16, n_kv=4)             # one entry: cut into as many items as allowed
    assert c % 64 == 0 and -(-8192 // c) <= 16
    assert decode_chunk(np.full(256, 1024), 16, n_kv=4) == 1024  # many entries: one item each
    c = decode_chunk(np.full(8, 1040), 16, n_kv=4)
    assert c % 64 == 0 and -(-1040 // c) * 8 * 4 >= 64
    assert [decode_parts_max(n) for n in (1, 64, 65, 1000, 1024, 100000)] == [1, 1, 2, 16, 16, 16]


def test_the_step_function_knows_no_kernel():
    """The step function builds tokens, positions, entries, slots and block tables; what a mixer's kernels need
    beyond that is the mixer's to plan (prepare_step)."""
    import ast
    import os
    import vt_transformer_amd.engine.step as step
    tree = ast.parse(open(step.__file__).read())
    imported = set()
    for node in ast.walk(tree):
        if isinstance(node, ast.ImportFrom) and node.module:
            imported.add(node.module)
    assert not any("kernels" in m or "attention" in m for m in imported), imported
    assert os.path.basename(step.__file__) == "step.py"


def test_uniform_numbers_depend_only_on_seed_and_counter():
    a = [uniform(5, i) for i in range(2000)]
    assert a == [uniform(5, i) for i in range(2000)]
    assert all(0.0 <= x < 1.0 for x in a)
    assert abs(np.mean(a) - 0.5) < 0.03 and abs(np.var(a) - 1 / 12) < 0.01
    assert np.float32(a[7]) == a[7]                       # exact in float32
    assert uniform(6, 0) != uniform(5, 0)
    assert request_seed(1, "a") != request_seed(1, "b") and request_seed(1, "a") == request_seed(1, "a")


def test_sampling_params_follow_the_front_end():
    """sglfront/sglfront/core.py:6-16."""
    p = SamplingParams()
    assert (p.temperature, p.top_k, p.top_p, p.ignore_eos, p.max_tokens) == (0.0, -1, 1.0, False, 1024)
    assert p.is_greedy and SamplingParams(temperature=0.7, top_k=1).is_greedy
    assert not SamplingParams(temperature=0.7).is_greedy and not SamplingParams(top_p=0.9).is_greedy
    for bad in (dict(top_p=0.0), dict(top_k=0), dict(max_tokens=0)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)


def test_the_direct_kernels_launch_model_picks_what_was_measured():
    """A fresh 2,048-token prompt on 28 / 4 heads runs fastest as whole items of one row tile per wave (its longest
    item is what the launch lasts), the same portion behind 2,048 earlier tokens with two row tiles (every block
    of keys read serves twice the rows); eight 1,024-token prompts fill the GPU with two row tiles and no cuts."""
    def pick(lens, pos0, nh=28, nkv=4):
        start = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        items, rt, citems, n_parts = plan_tile_items(start, np.array(pos0, np.int32), nh // nkv, 0, nkv,
                                                     np.arange(len(lens)), head_dim=128, direct=True)
        return rt, n_parts
    assert pick([2048], [0]) == (1, 0)
    assert pick([2048], [2048])[0] == 2
    assert pick([2048], [2048])[1] == 0            # (cutting these costs a fifth: 112 -> 127 to 138 us)
    assert pick([1024] * 8, [0] * 8) == (2, 0)
    # A 2,048-token portion behind 30,720 earlier tokens on 12 / 2 heads is 192 blocks of 500 steps: two key ranges
    # each would leave a quarter of the 512 slots empty, four fill them (476 -> 427 us).
    rt, n_parts = pick([2048], [30720], nh=12, nkv=2)
    assert rt == 2 and n_parts == 4 * 96
