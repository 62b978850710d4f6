"""The extraction decoder's attention step (spinf_serve/decode.py:71-104): the numpy oracle against torch's SDPA and against the
tree-attention oracle, the host side, and (gpu) the HIP kernel through the C ABI against the oracle."""

import ctypes as C

import numpy as np
import pytest
import torch

import spinf_serve_amd as sa
from oracle import attention as oattn
from oracle import xdecode as ox
from spinf_serve_amd import _lib, decode, synth

TOL = 2e-2   # max abs error of the bf16 kernel against the float64 oracle on the same bf16 inputs


def _np(t):
    return t.float().cpu().numpy()


def _oracle(query, c, scale, window=None, softcap=None, layer=0):
    return ox.x_attention(_np(query), _np(c.kp[layer]), _np(c.vp[layer]), c.pos_p[layer].cpu().numpy(), _np(c.kt[layer]), _np(c.vt[layer]),
                          c.pos_t.cpu().numpy(), c.own_t.cpu().numpy(), _np(c.gk[layer]), _np(c.gv[layer]), c.qpos.cpu().numpy(),
                          int(c.step_t.item()), c.beam, scale, window, softcap)


# ------------------------------------------------------------------------------------------------ oracle pins (CPU)
@pytest.mark.parametrize("window", [None, 12])
def test_oracle_is_sdpa_over_the_concatenated_keys(window):
    """the mask is rebuilt here key by key from the rule's words; torch's scaled_dot_product_attention does the arithmetic"""
    q, c = synth.xdecode_case(G=3, H=4, h=2, d=16, slots=3, beam=2, S=5, prefix=(9, 20), template=(2, 5), window=window, step=2, seed=1, device="cpu")
    G, H, Q, d = q.shape
    h, S, beam = 2, 5, 2
    want = _oracle(q, c, 0.3, window)
    pos_p, pos_t, own_t, qpos = (x.numpy() for x in (c.pos_p[0], c.pos_t, c.own_t, c.qpos))
    for g in range(G):
        for qi in range(Q):
            keys, vals = [], []
            for kv in range(h):
                ks, vs = [], []
                for j in range(pos_p.shape[1]):
                    if pos_p[g, j] >= 0 and (window is None or qpos[g, qi] - pos_p[g, j] < window):
                        ks.append(c.kp[0][g, kv, j]); vs.append(c.vp[0][g, kv, j])
                for j in range(pos_t.shape[1]):
                    if own_t[g, j] == qi // beam and (window is None or qpos[g, qi] - pos_t[g, j] < window):
                        ks.append(c.kt[0][g, kv, j]); vs.append(c.vt[0][g, kv, j])
                for s in range(3):
                    ks.append(c.gk[0][g, kv, qi, s]); vs.append(c.gv[0][g, kv, qi, s])
                keys.append(torch.stack(ks)); vals.append(torch.stack(vs))
            k, v = torch.stack(keys).double()[None], torch.stack(vals).double()[None]   # [1, h, L, d]
            got = torch.nn.functional.scaled_dot_product_attention(q[g : g + 1, :, qi : qi + 1].double(), k, v, scale=0.3, enable_gqa=True)
            assert np.abs(got[0, :, 0].numpy() - want[g, qi]).max() < 1e-10


def test_oracle_step_is_the_last_row_of_causal_attention_over_the_path():
    """prefix | own template | own generated tokens is a path of the tree: the decode step's output is the last row of the
    packed-prefill attention oracle over that path"""
    q, c = synth.xdecode_case(G=2, H=2, h=1, d=8, slots=2, beam=1, S=4, prefix=(5, 9), template=(2, 4), step=3, seed=2, device="cpu")
    want = _oracle(q, c, 0.5)
    pos_p, own_t = c.pos_p[0].numpy(), c.own_t.numpy()
    for g in range(2):
        for qi in range(2):
            k = np.concatenate([_np(c.kp[0][g])[:, pos_p[g] >= 0], _np(c.kt[0][g])[:, own_t[g] == qi], _np(c.gk[0][g, :, qi])], 1)   # [h, n, d]
            v = np.concatenate([_np(c.vp[0][g])[:, pos_p[g] >= 0], _np(c.vt[0][g])[:, own_t[g] == qi], _np(c.gv[0][g, :, qi])], 1)
            n = k.shape[1]
            qq = np.zeros((n, 2, 8), np.float32)
            qq[-1] = _np(q[g, :, qi])
            art, end = np.zeros(n, np.int32), np.full(n, n, np.int32)
            ref = oattn.tree_attention(qq, k.transpose(1, 0, 2), v.transpose(1, 0, 2), art, end, scale=0.5, spans=oattn.job_spans(art))
            assert np.abs(ref[-1] - want[g, qi]).max() < 1e-10


def test_oracle_softcap_and_masks():
    q, c = synth.xdecode_case(G=1, H=2, h=2, d=8, slots=2, beam=2, S=3, prefix=(4, 4), template=(2, 2), step=0, seed=3, device="cpu")
    # one key visible per range at most: zero the scores' influence with a huge soft cap -> same as no cap
    a = _oracle(q, c, 1.0, softcap=1e9)
    b = _oracle(q, c, 1.0)
    assert np.abs(a - b).max() < 1e-6
    # a tiny cap flattens the softmax: the output is the mean of the visible values
    flat = _oracle(q, c, 1.0, softcap=1e-9)
    vis = np.concatenate([_np(c.vp[0][0, 0]), _np(c.vt[0][0, 0])[c.own_t[0].numpy() == 1], _np(c.gv[0][0, 0, 3, :1])])
    assert np.abs(flat[0, 3, 0] - vis.mean(0)).max() < 1e-6


# ------------------------------------------------------------------------------------------------ host side (CPU)
def test_argument_checks_come_before_any_launch(lib):
    a = _lib.XdecArgs()
    a.G, a.H, a.h, a.Q, a.S, a.Lp, a.Tt, a.d, a.beam, a.nsplit = 1, 4, 2, 6, 4, 10, 4, 96, 3, 1
    assert lib.spinf_xdecode_attn_fwd(C.byref(a), None) == -1 and b"head dim" in lib.spinf_last_error()
    a.d, a.H = 64, 5
    assert lib.spinf_xdecode_attn_fwd(C.byref(a), None) == -1 and b"bad sizes" in lib.spinf_last_error()
    a.H = 4
    assert lib.spinf_xdecode_attn_fwd(C.byref(a), None) == -1 and b"null pointer" in lib.spinf_last_error()
    assert lib.spinf_xdecode_attn_fwd(None, None) == -1
    a.G = 0
    assert lib.spinf_xdecode_attn_fwd(C.byref(a), None) == 0   # nothing to do
    with pytest.raises(RuntimeError, match="no CPU path"):
        q, c = synth.xdecode_case(G=1, H=2, h=1, d=64, slots=1, beam=2, S=2, prefix=(4, 4), template=(2, 2), device="cpu")
        sa.xdecode_attn(q, c, 0, nsplit=1)


def test_split_suggestion():
    assert decode.plan_splits(64, 16, 8, 24, 17, 470, 40, 256, 6) == (1, 0)          # 512 workgroups already
    ns, wb = decode.plan_splits(4, 16, 8, 24, 17, 4096, 40, 256, 6)                  # 32 (group, kv head) pairs for 512 places
    assert ns == 16 and wb == 4 * 16 * 24 * ns * 258 * 4
    ns, _ = decode.plan_splits(4, 16, 8, 24, 17, 300, 40, 256, 6)                    # short stream: a split keeps 8 tiles
    assert 1 <= ns <= (300 + 40 + 24 * 17 + 31) // 32 // 8


def test_split_sizes_for_ragged_groups():
    """with the groups' own lengths known the split size comes from a simulated schedule: many groups fill the GPU unsplit, a
    few ragged ones are cut into pieces of about the same size; nsplit x tiles per split always covers the longest list"""
    rng = np.random.default_rng(0)
    for G in (64, 12, 3):
        P = [int(x) for x in rng.integers(1024, 4097, G)]
        ns, per = decode.plan_ragged(G, 16, 8, 48, 33, max(P), 100, 256, 6, tuple(P), (100,) * G)
        longest = decode._list_tiles(max(P), 100, 33, max(P), 100, 0, 47)
        assert ns * per >= longest and per >= 8
        assert (ns == 1) == (G == 64)
    # the host's tile count is the library's
    a = _lib.XdecArgs()
    a.G, a.H, a.h, a.Q, a.S, a.Lp, a.Tt, a.d, a.beam = 2, 16, 8, 48, 33, 1000, 77, 256, 6
    n = C.c_int32(0)
    assert _lib.load_library().spinf_xdecode_tiles(C.byref(a), C.byref(n)) == 0
    assert n.value == decode._list_tiles(1000, 77, 33, 1000, 77, 0, 47) == 84   # 96 rows: one chunk with all 48 queries


def test_longest_list_over_all_row_chunks():
    """the library's tile count is the maximum over the row chunks (a later chunk can hold more tiles than the first: where its
    generated entries begin and end inside their tiles), so that splits sized from it cover every list"""
    rng = np.random.default_rng(5)
    lib = _lib.load_library()
    later = 0
    for _ in range(300):
        H, h = [(16, 1), (16, 8), (24, 4), (8, 8), (6, 2)][int(rng.integers(5))]
        Q, S = int(rng.integers(1, 200)), int(rng.integers(1, 70))
        Lp, Tt = int(rng.integers(0, 3000)), int(rng.integers(0, 300))
        a = _lib.XdecArgs()
        a.G, a.H, a.h, a.Q, a.S, a.Lp, a.Tt, a.d, a.beam = 3, H, h, Q, S, Lp, Tt, 128, 3
        n = C.c_int32(0)
        assert lib.spinf_xdecode_tiles(C.byref(a), C.byref(n)) == 0
        r, R = H // h, Q * (H // h)
        per_chunk = [decode._list_tiles(Lp, Tt, S, Lp, Tt, c * 128 // r, (min(c * 128 + 128, R) - 1) // r) for c in range(-(-R // 128))]
        assert n.value == max(per_chunk)
        later += max(per_chunk) > per_chunk[0]
        ns, per = decode.plan_ragged(3, H, h, Q, S, Lp, Tt, 128, 3, (Lp,) * 3, (Tt,) * 3)
        assert ns * per >= max(per_chunk)
    assert later > 10   # the case exists


# ------------------------------------------------------------------------------------------------ kernel parity (GPU)
CASES = [
    # G, H, h, d, slots, beam, S, prefix, template, window, softcap, step, nsplit
    (2, 4, 2, 64, 2, 3, 5, (10, 20), (2, 4), None, None, 2, 1),
    (3, 16, 8, 256, 4, 6, 17, (300, 470), (6, 14), None, None, 16, None),
    (3, 16, 8, 256, 4, 6, 17, (300, 470), (6, 14), 128, None, 7, 1),
    (2, 8, 4, 128, 12, 6, 9, (100, 200), (3, 9), None, None, 0, 3),          # 144 rows: two row chunks
    (2, 24, 4, 256, 5, 6, 12, (500, 900), (4, 20), None, None, 5, 5),        # r = 6 (the Qwen geometry), 180 rows
    (2, 8, 8, 128, 3, 6, 33, (31, 33), (1, 2), None, 30.0, 20, 2),           # MHA, soft cap, keys end inside a tile
    (1, 4, 1, 64, 1, 1, 3, (1, 1), (1, 1), 1024, 50.0, 1, 1),                # one query, a handful of keys
    (5, 16, 8, 256, 2, 6, 65, (64, 1500), (10, 30), 512, None, 40, 4),       # ragged prefixes, window clips them
    (2, 16, 1, 512, 4, 6, 9, (200, 600), (4, 12), None, None, 5, None),      # head dim 512, one kv head (Gemma-4 global layers): 384 rows
    (2, 8, 2, 512, 2, 3, 5, (20, 90), (2, 6), 64, 25.0, 4, 2),               # head dim 512 with window, soft cap and splits
    (24, 16, 1, 512, 8, 6, 33, (470, 470), (8, 16), None, None, 32, None),   # six row chunks, the later ones with longer tile lists than the first
    (3, 16, 1, 256, 8, 6, 33, (470, 470), (8, 16), None, None, 32, 1),       # the same at head dim 256, one split
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[f"case{i}" for i in range(len(CASES))])
def test_kernel_matches_oracle(dev, case):
    G, H, h, d, slots, beam, S, prefix, template, window, softcap, step, nsplit = case
    q, c = synth.xdecode_case(G, H, h, d, slots, beam, S, prefix, template, window, step, seed=7, device=dev)
    scale = d**-0.5
    out = sa.xdecode_attn(q, c, 0, scale, window, softcap, nsplit=nsplit)
    torch.cuda.synchronize()
    assert out.shape == (G, slots * beam, H, d) and out.is_contiguous()
    err = np.abs(_np(out) - _oracle(q, c, scale, window, softcap)).max()
    assert err <= TOL, err


@pytest.mark.gpu
def test_padding_rows_and_empty_ranges(dev):
    """padding inside the prefix and template ranges (shorter groups), a group without template tokens for one slot, no prefix at all"""
    q, c = synth.xdecode_case(4, 8, 4, 128, 3, 2, 6, (5, 90), (1, 12), None, 3, seed=11, device=dev)
    c.own_t[1][c.own_t[1] == 2] = -1          # slot 2 of group 1 loses its template
    out = sa.xdecode_attn(q, c, 0, 0.1, nsplit=2)
    assert np.abs(_np(out) - _oracle(q, c, 0.1)).max() <= TOL
    c.pos_p[0][:] = -1                         # nothing of any prefix is visible
    out = sa.xdecode_attn(q, c, 0, 0.1, nsplit=1)
    assert np.abs(_np(out) - _oracle(q, c, 0.1)).max() <= TOL
    # no prefix and no template tensors at all: the queries see their own generated tokens only
    for name in ("kp", "vp", "kt", "vt"):
        t = getattr(c, name)[0]
        getattr(c, name)[0] = t[:, :, :0].contiguous()
    c.pos_p[0], c.pos_t, c.own_t = c.pos_p[0][:, :0].contiguous(), c.pos_t[:, :0].contiguous(), c.own_t[:, :0].contiguous()
    out = sa.xdecode_attn(q, c, 0, 0.1)
    assert np.abs(_np(out) - _oracle(q, c, 0.1)).max() <= TOL


@pytest.mark.gpu
@pytest.mark.parametrize("nsplit", [1, 3])
def test_a_group_alone_or_among_others_bit_for_bit(dev, nsplit):
    """a group's outputs do not depend on the other groups of the call (same tensors' extents, same split count)"""
    q, c = synth.xdecode_case(6, 16, 8, 256, 3, 6, 9, (100, 400), (4, 12), None, 8, seed=5, device=dev)
    full = sa.xdecode_attn(q, c, 0, 1 / 16, nsplit=nsplit)
    for g in (0, 4):
        one = decode.XCaches(beam=c.beam, pos_t=c.pos_t[g : g + 1].contiguous(), own_t=c.own_t[g : g + 1].contiguous(), qpos=c.qpos[g : g + 1].contiguous(), step_t=c.step_t)
        for name in ("kp", "vp", "kt", "vt", "gk", "gv", "pos_p"):
            getattr(one, name)[0] = getattr(c, name)[0][g : g + 1].contiguous()
        one.set_lengths()
        alone = sa.xdecode_attn(q[g : g + 1], one, 0, 1 / 16, nsplit=nsplit)
        assert torch.equal(alone[0], full[g])


@pytest.mark.gpu
def test_the_interface_callable_and_the_cache_update(dev):
    """GroupKV.update writes the step's K/V, x_attention reads the running decoder's caches (decode.py:51-104); steps 0, 1, 2 in a row"""
    q, c = synth.xdecode_case(2, 8, 4, 128, 2, 6, 4, (40, 80), (3, 6), None, 0, seed=9, device=dev)
    c.gk[0].zero_(); c.gv[0].zero_()
    cache = decode.GroupKV(c)
    decode._CURRENT[0] = c
    gen = torch.Generator().manual_seed(1)
    base = c.qpos.clone()
    try:
        for step in range(3):
            c.step_t.fill_(step)
            c.qpos.copy_(base + step)
            knew = (torch.randn(2, 4, 12, 128, generator=gen) * 0.5).to(torch.bfloat16).to(dev)
            vnew = (torch.randn(2, 4, 12, 128, generator=gen) * 0.5).to(torch.bfloat16).to(dev)
            qs = torch.randn(2, 12, 8, 128, generator=gen).to(torch.bfloat16).to(dev).transpose(1, 2)
            key, value = cache.update(knew, vnew, 0)
            out, none = decode.x_attention(None, qs, key, value, None, scaling=0.09, sliding_window=None)
            assert none is None and torch.equal(c.gk[0][:, :, :, step], knew)
            assert np.abs(_np(out) - _oracle(qs, c, 0.09)).max() <= TOL
    finally:
        decode._CURRENT[0] = None
    with pytest.raises(RuntimeError, match="outside a decoding step"):
        decode.x_attention(None, qs, ("x", 0), ("x", 0), None)


@pytest.mark.gpu
@pytest.mark.parametrize("nsplit", [1, 2])
def test_step_replayed_from_a_graph(dev, nsplit):
    """the reference replays a decoding step from a captured graph on static buffers (decode.py:82, 170-171): the step index, the
    query positions and the generated K/V change between replays, the launch does not.  Every replay against the eager result."""
    q, c = synth.xdecode_case(3, 8, 4, 128, 3, 6, 6, (50, 120), (3, 8), None, 0, seed=13, device=dev)
    static_q = q.clone()
    sa.xdecode_attn(static_q, c, 0, 0.09, nsplit=nsplit)   # the workspace exists before the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            static_out = sa.xdecode_attn(static_q, c, 0, 0.09, nsplit=nsplit)
    torch.cuda.current_stream().wait_stream(side)
    gen = torch.Generator().manual_seed(3)
    base = c.qpos.clone()
    for step in (0, 3, 5, 1):
        c.step_t.fill_(step)
        c.qpos.copy_(base + step)
        c.gk[0][:, :, :, step] = (torch.randn(3, 4, 18, 128, generator=gen) * 0.5).to(torch.bfloat16).to(dev)
        static_q.copy_(torch.randn(3, 8, 18, 128, generator=gen).to(torch.bfloat16).to(dev))
        graph.replay()
        torch.cuda.synchronize()
        eager = sa.xdecode_attn(static_q, c, 0, 0.09, nsplit=nsplit)
        torch.cuda.synchronize()
        assert torch.equal(static_out, eager)
        assert np.abs(_np(static_out) - _oracle(static_q, c, 0.09)).max() <= TOL


@pytest.mark.gpu
def test_seeded_random_shapes(dev):
    """random geometries: head dims, GQA ratios, slots x beams (one to nine row chunks), ragged prefixes shorter than a tile or
    thousands long, windows, soft caps, steps, forced split counts (more splits than some groups have tiles)"""
    rng = np.random.default_rng(2024)
    for case in range(60):
        d = int(rng.choice([64, 128, 256, 512]))
        h = int(rng.choice([1, 2, 4]))
        r = int(rng.choice([1, 2, 3, 6, 16]))
        slots, beam = int(rng.integers(1, 13)), int(rng.choice([1, 3, 6]))
        S = int(rng.integers(1, 40))
        G = int(rng.integers(1, 5))
        lo = int(rng.integers(1, 200))
        hi = lo + int(rng.choice([0, 30, 700, 2500]))
        tl = int(rng.integers(1, 6))
        window = int(rng.choice([0, 16, 300, 4096])) or None
        softcap = float(rng.choice([0.0, 20.0])) or None
        step = int(rng.integers(0, S))
        nsplit = int(rng.choice([0, 1, 2, 5])) or None
        print(f"case {case}: G={G} H={h * r} h={h} d={d} slots={slots} beam={beam} S={S} prefix=({lo},{hi}) window={window} softcap={softcap} step={step} nsplit={nsplit}", flush=True)
        q, c = synth.xdecode_case(G, h * r, h, d, slots, beam, S, (lo, hi), (tl, tl + 9), window, step, seed=100 + case, device=dev)
        scale = float(rng.choice([d**-0.5, 1 / 16]))
        out = sa.xdecode_attn(q, c, 0, scale, window, softcap, nsplit=nsplit)
        err = np.abs(_np(out) - _oracle(q, c, scale, window, softcap)).max()
        assert err <= TOL, (case, err)
