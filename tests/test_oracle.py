"""Pins the CPU oracle (oracle/) before anything is compared with it: golden vectors written from the reference's host code,
the literal answers of the reference's own tests, and closed forms / library reductions for the arithmetic."""

import gzip
import json
import os

import numpy as np
import pytest

from oracle import attention as oattn
from oracle import gdn as ogdn
from oracle import mask as omask
from oracle import plan as oplan
from oracle.layout import Job, pack_stream

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def golden():
    with gzip.open(os.path.join(HERE, "golden", "packer_golden.json.gz"), "rt") as f:
        return json.load(f)


def _jobs_of_batch(case, batch):
    trees = case["trees"]
    return [Job(trees[o[0]]["prefix"], trees[o[0]]["branches"], trees[o[0]]["parents"], tuple(trees[o[0]]["aligned"])) for o in batch["owners"]]


def test_layout_matches_reference_streams(golden):
    """oracle.layout.pack_stream == Packer._pack of the reference (spinf_serve/packer.py:352-423) on every golden batch"""
    n = 0
    for case in golden["cases"]:
        for b in case["batches"]:
            s = pack_stream(_jobs_of_batch(case, b), align=case["align"], length=len(b["ids"]))
            for key in ("ids", "pos", "seg", "art", "end", "prev"):
                assert getattr(s, key).tolist() == b[key], (key, n)
            assert s.n_real == b["n_tokens"]
            assert [sp[0] for sp in s.starts] == [o[1] for o in b["owners"]]
            n += 1
    assert n >= 8


def test_layout_literals_of_the_reference_tests():
    # tests/test_packer.py:191-199: trie of two template combinations and a prompt with a lead-in
    j = Job([1, 2], [[5, 6, 7], [8], [9], [4, 21]], [-1, 0, 0, -1])
    s = pack_stream([j])
    assert s.pos[:9].tolist() == [0, 1, 2, 3, 4, 5, 5, 2, 3]
    assert s.end[:9].tolist() == [9, 9, 7, 7, 7, 6, 7, 9, 9]
    assert s.prev[:9].tolist() == [-1, 0, 1, 2, 3, 4, 4, 1, 7]
    assert j.n_tokens == 2 + 3 + 1 + 1 + 2


def test_dense_mask_is_the_ancestor_relation(golden):
    """the predicate of spinf_serve/scorer.py:173-177 == 'k lies on q's path' derived independently from prev"""
    for case in golden["cases"][:4]:
        for b in case["batches"]:
            art, end, prev = np.array(b["art"]), np.array(b["end"]), np.array(b["prev"])
            n = min(len(art), 600)
            m = omask.dense_tree_mask(art[:n], np.minimum(end[:n], n))
            assert (m == omask.ancestor_mask(prev[:n], art[:n] >= 0)).all()


def test_each_row_sees_its_path_positions(golden):
    """tests/test_packer.py:209-239: a token sees exactly one token per position 0 .. pos"""
    b = golden["cases"][2]["batches"][0]
    art, end, pos = np.array(b["art"]), np.array(b["end"]), np.array(b["pos"])
    m = omask.dense_tree_mask(art, end)
    for q in np.flatnonzero(art >= 0)[::7]:
        assert sorted(pos[m[q]].tolist()) == list(range(pos[q] + 1))


def test_block_classes_match_reference_tables(golden):
    """oracle.mask.block_classes == block_tables (spinf_serve/packer.py:426-491), global and sliding, on every golden batch"""
    for case in golden["cases"]:
        for b in case["batches"]:
            (full, part), slid = omask.block_classes(b["art"], b["end"], b["pos"], b["window"], always_window=True)
            nb = len(b["ids"]) // 128
            for i in range(nb):
                assert np.flatnonzero(full[i]).tolist() == sorted(b["tables_full"]["full"][i])
                assert np.flatnonzero(part[i]).tolist() == sorted(b["tables_full"]["partial"][i])
                assert np.flatnonzero(slid[1][i]).tolist() == sorted(b["tables_sliding"]["partial"][i])
                assert not slid[0][i].any() and b["tables_sliding"]["full"][i] == []


def test_block_class_literals():
    # tests/test_packer.py:182-188: 2000-token trunk, window 512: q block 14 sees kv blocks 10..14, none full
    s = pack_stream([Job([1] * 2000, [[2]])], length=2048)
    _, (full, part) = omask.block_classes(s.art, s.end, s.pos, 512)
    assert np.flatnonzero(part[14]).tolist() == [10, 11, 12, 13, 14] and not full.any()
    # tests/test_packer.py:251-259: the sibling's q block 5 skips block 2, lists 1,3,4,5, block 0 full
    s = pack_stream([Job([1] * 200, [[2] * 300, [3] * 300])], length=1024)
    (full, part), _ = omask.block_classes(s.art, s.end, s.pos, None)
    listed = set(np.flatnonzero(full[5] | part[5]).tolist())
    assert 2 not in listed and {1, 3, 4, 5} <= listed and full[5, 0]


# ------------------------------------------------------------------------------------------------ attention arithmetic
def _rand(rng, *shape):
    return rng.standard_normal(shape)


def test_attention_reduces_to_causal_sdpa():
    """a trunk alone is causal attention: torch's own scaled_dot_product_attention(is_causal=True, enable_gqa=True)"""
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(0)
    n, hq, hkv, d = 70, 4, 2, 16
    q, k, v = _rand(rng, n, hq, d), _rand(rng, n, hkv, d), _rand(rng, n, hkv, d)
    s = pack_stream([Job(list(range(n)), [])], length=n)
    got = oattn.tree_attention(q, k, v, s.art, s.end, scale=0.3)
    t = lambda x: torch.from_numpy(x).transpose(0, 1)[None]  # noqa: E731
    want = F.scaled_dot_product_attention(t(q), t(k), t(v), is_causal=True, scale=0.3, enable_gqa=True)[0].transpose(0, 1).numpy()
    assert np.abs(got - want).max() < 1e-12


def test_branches_are_independent_causal_runs():
    """B branches == B independent causal runs of trunk||branch (brute force), nothing leaks between siblings or jobs"""
    rng = np.random.default_rng(1)
    P, lens = 9, [3, 5, 2]
    jobs = [Job(list(range(P)), [list(range(L)) for L in lens]), Job([7] * 4, [[1, 2]])]
    s = pack_stream(jobs, align=False)
    n, hq, hkv, d = len(s.art), 2, 1, 8
    q, k, v = _rand(rng, n, hq, d), _rand(rng, n, hkv, d), _rand(rng, n, hkv, d)
    got = oattn.tree_attention(q, k, v, s.art, s.end, scale=0.5)
    start = P
    for L in lens:
        rows = list(range(P)) + list(range(start, start + L))
        flat = pack_stream([Job(list(range(len(rows))), [])], length=len(rows))
        want = oattn.tree_attention(q[rows], k[rows], v[rows], flat.art, flat.end, scale=0.5)
        assert np.abs(got[rows] - want).max() < 1e-12
        start += L


def test_sliding_window_is_banded_causal():
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(2)
    n, W = 50, 7
    q, k, v = _rand(rng, n, 2, 8), _rand(rng, n, 2, 8), _rand(rng, n, 2, 8)
    s = pack_stream([Job(list(range(n)), [])], length=n)
    got = oattn.tree_attention(q, k, v, s.art, s.end, s.pos, window=W, scale=0.4)
    i = np.arange(n)
    band = torch.from_numpy((i[None, :] <= i[:, None]) & (i[:, None] - i[None, :] < W))
    t = lambda x: torch.from_numpy(x).transpose(0, 1)[None]  # noqa: E731
    want = F.scaled_dot_product_attention(t(q), t(k), t(v), attn_mask=band, scale=0.4)[0].transpose(0, 1).numpy()
    assert np.abs(got - want).max() < 1e-12


def test_pads_return_their_own_value_and_spans_change_nothing():
    rng = np.random.default_rng(3)
    s = pack_stream([Job([1] * 30, [[2] * 5]), Job([3] * 10, [[4] * 3, [5] * 2])], align=True)
    n = len(s.art)
    q, k, v = _rand(rng, n, 4, 8), _rand(rng, n, 2, 8), _rand(rng, n, 2, 8)
    whole = oattn.tree_attention(q, k, v, s.art, s.end)
    split = oattn.tree_attention(q, k, v, s.art, s.end, spans=oattn.job_spans(s.art))
    assert np.abs(whole - split).max() < 1e-12
    pad = np.flatnonzero(s.art < 0)
    assert np.abs(whole[pad] - np.repeat(v[pad], 2, axis=1)).max() < 1e-12


# ------------------------------------------------------------------------------------------------ gated delta rule
def _gdn_inputs(rng, T, H=2, HV=4, K=16, V=8):
    q, k = _rand(rng, T, H, K), _rand(rng, T, H, K)
    q /= np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6)
    k /= np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    v = _rand(rng, T, HV, V)
    beta = 1 / (1 + np.exp(-_rand(rng, T, HV)))
    g = -np.log1p(np.exp(_rand(rng, T, HV)))
    return q, k, v, g, beta


def test_recurrence_closed_forms():
    rng = np.random.default_rng(4)
    q, k, v, g, beta = _gdn_inputs(rng, 12)
    h0 = _rand(rng, 4, 16, 8)
    # g = 0, beta = 0: the state never changes and o_t = S0^T (scale q_t)
    o, S = ogdn.recurrent(q, k, v, np.zeros_like(g), np.zeros_like(beta), scale=0.25, h0=h0)
    assert np.abs(S - h0).max() == 0
    want = np.einsum("hkv,thk->thv", h0, np.repeat(q, 2, axis=1) * 0.25)
    assert np.abs(o - want).max() < 1e-12
    # plain delta rule (g = 0, beta = 1) from zero with a unit key: after one token S^T k = v exactly
    k1 = k[:1] / np.linalg.norm(k[:1], axis=-1, keepdims=True)
    _, S = ogdn.recurrent(q[:1], k1, v[:1], np.zeros((1, 4)), np.ones((1, 4)))
    assert np.abs(np.einsum("hkv,hk->hv", S, np.repeat(k1[0], 2, axis=0)) - v[0]).max() < 1e-12
    # linear in v (and in the initial state)
    o1, _ = ogdn.recurrent(q, k, v, g, beta)
    o2, _ = ogdn.recurrent(q, k, 3.0 * v, g, beta)
    assert np.abs(o2 - 3.0 * o1).max() < 1e-11
    # pure decay: beta = 0 scales the state by exp(sum g)
    _, S = ogdn.recurrent(q, k, v, g, np.zeros_like(beta), h0=h0)
    assert np.abs(S - h0 * np.exp(g.sum(0))[:, None, None]).max() < 1e-12


@pytest.mark.parametrize("T", [1, 63, 64, 65, 200])
def test_chunked_equals_recurrent(T):
    rng = np.random.default_rng(T)
    q, k, v, g, beta = _gdn_inputs(rng, T)
    h0 = _rand(rng, 4, 16, 8) * 0.3
    o1, s1 = ogdn.recurrent(q, k, v, g, beta, h0=h0)
    o2, s2 = ogdn.chunked(q, k, v, g, beta, h0=h0)
    assert np.abs(o1 - o2).max() < 1e-10 and np.abs(s1 - s2).max() < 1e-10


def test_fork_identity_branch_from_trunk_state():
    """docs/QWEN.md:51-52: a branch run from its parent's final state == prefix||branch as one sequence"""
    rng = np.random.default_rng(6)
    s = pack_stream([Job([1] * 40, [[2] * 6, [3] * 9], [-1, -1])], align=False)
    n = len(s.art)
    q, k, v, g, beta = _gdn_inputs(rng, n)
    o = ogdn.tree_scan(q, k, v, g, beta, s.prev, s.art >= 0)
    start = 40
    for L in (6, 9):
        rows = list(range(40)) + list(range(start, start + L))
        want, _ = ogdn.recurrent(q[rows], k[rows], v[rows], g[rows], beta[rows])
        assert np.abs(o[rows] - want).max() < 1e-12
        start += L
    assert np.abs(o[s.art < 0]).max() == 0


# ------------------------------------------------------------------------------------------------ recurrent-layer plan
def test_plan_matches_reference_calls(golden):
    """oracle.plan.tree_plan == tree_plan(path='indexed') of the reference (qwen.py:158-276): calls, slots, kept states"""
    for case in golden["cases"]:
        for b in case["batches"]:
            prev, real = np.array(b["prev"]), np.array(b["art"]) >= 0
            for short, ct in ((64, 8192), (4, 300)):
                want = b[f"plan_short{short}_ct{ct}"]
                levels, n_keep, info = oplan.tree_plan(prev, real, short=short, call_tokens=ct)
                assert n_keep == want["n_keep"] and len(info["starts"]) == want["n_segments"]
                assert len(levels) == len(want["levels"])
                for lv, wl in zip(levels, want["levels"]):
                    assert len(lv) == len(wl)
                    for c, wc in zip(lv, wl):
                        assert c["kind"] == wc["kind"] and c["idx"].tolist() == wc["idx"] and c["cu"].tolist() == wc["cu"]
                        assert (None if c["h0_idx"] is None else c["h0_idx"].tolist()) == wc["h0_idx"]
                        assert (None if c["ht_idx"] is None else c["ht_idx"].tolist()) == wc["ht_idx"]


def test_plan_literal_and_toy_recurrence():
    # tests/test_stacks.py:67-75: prev = [-1, 0, 1, 1, 3] -> 3 segments
    starts, lens, parent, depth, kids, seg = oplan.segments(np.array([-1, 0, 1, 1, 3]), np.ones(5, bool))
    assert len(starts) == 3 and lens.tolist() == [2, 1, 2] and parent.tolist() == [-1, 0, 0]
    # tests/test_qwen_plan.py:27-48: a toy integer recurrence level by level == along the path
    rng = np.random.default_rng(0)
    job = Job(list(rng.integers(5, 50, 37)), [list(rng.integers(5, 50, n)) for n in (6, 70, 3, 2, 9)], [-1, 0, 0, 2, -1])
    s = pack_stream([job, Job([9] * 5, [[1], [2]])], align=True)
    real = s.art >= 0
    step = lambda h, t: (h * 1_000_003 + int(t) + 1) % (1 << 61)  # noqa: E731
    want = np.zeros(len(s.ids), np.int64)
    for i in np.flatnonzero(real):
        want[i] = step(int(want[s.prev[i]]) if s.prev[i] >= 0 else 0, s.ids[i])
    levels, n_keep, _ = oplan.tree_plan(s.prev, real, short=4)
    got = np.zeros(len(s.ids), np.int64)
    prev_states = None
    for calls, nk in zip(levels, n_keep):
        states = [None] * nk
        for c in calls:
            for sg in range(len(c["cu"]) - 1):
                h = 0 if c["h0_idx"] is None or c["h0_idx"][sg] < 0 else prev_states[c["h0_idx"][sg]]
                for i in c["idx"][c["cu"][sg] : c["cu"][sg + 1]]:
                    h = step(h, s.ids[i])
                    got[i] = h
                if c["ht_idx"] is not None and c["ht_idx"][sg] >= 0:
                    states[c["ht_idx"][sg]] = h
        assert all(x is not None for x in states)
        prev_states = states
    assert (got[real] == want[real]).all()
