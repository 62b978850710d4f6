"""GPU parity of the tree-mask attention kernel (through the C ABI) against the CPU oracle.

Bars: max abs error <= 2e-2 for the bf16 kernel against the float64 oracle on the same seeded bf16 inputs; bit-exact
per-content output alone vs packed vs reversed pack order (the reference's protocol, docs/BATCH_INVARIANCE.md:71-72)."""

import numpy as np
import pytest
import torch

import spinf_serve_amd as sa
from oracle import attention as oattn
from oracle import mask as omask
from spinf_serve_amd import attention, synth
from spinf_serve_amd.layout import TokenTree

pytestmark = pytest.mark.gpu
TOL = 2e-2


def _oracle(q, k, v, b, scale, window=None):
    return oattn.tree_attention(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), b.art, b.end, b.pos,
                                window=window, scale=scale, spans=oattn.job_spans(b.art))


def _pads_selfattend(out, v, b, g):
    pad = np.flatnonzero(b.art < 0)
    if len(pad):
        want = v[pad].repeat_interleave(g, dim=1)
        assert torch.equal(out[pad], want), "a pad row attends to itself only: its output is its own V row"


def _check(cfg, b, dev, window=None, seed=0, variant=None):
    q, k, v = synth.qkv(cfg, b, seed=seed, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, window=window, device=dev)
    print(f"case {cfg.name} n={b.length} hq={cfg.hq} hkv={cfg.hkv} d={cfg.d} window={window} variant={variant}", flush=True)
    out = sa.tree_attn(q, k, v, mask, cfg.scale, variant=variant)
    torch.cuda.synchronize()
    ref = _oracle(q, k, v, b, cfg.scale, window)
    err = float(np.abs(out.float().cpu().numpy() - ref).max())
    assert np.isfinite(out.float().cpu().numpy()).all()
    assert err <= TOL, err
    _pads_selfattend(out, v, b, cfg.hq // cfg.hkv)
    return out, err


@pytest.mark.parametrize("name", ["C1", "smoke"])
def test_small_configs(dev, name):
    cfg = synth.attention_config(name)
    _check(cfg, cfg.batches[0], dev)


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_c2_shape_three_contents(dev, variant):
    cfg = synth.attention_config("C2", contents=3)
    _check(cfg, cfg.batches[0], dev, variant=variant)


def _ring_aborts():
    import ctypes

    total = ctypes.c_int64(-1)
    assert sa.load_library().spinf_attn_ring_aborts(ctypes.byref(total)) == 0
    return total.value


def _exact_items():
    import ctypes

    total = ctypes.c_int64(0)
    assert sa.load_library().spinf_attn_exact_items(ctypes.byref(total)) == 0
    return total.value


@pytest.mark.parametrize("d,hq,hkv", [(64, 4, 2), (128, 4, 2), (256, 2, 1), (128, 3, 3), (512, 4, 1)])
def test_wide_score_range_takes_the_exact_pass(dev, d, hq, hkv):
    """scores that grow by far more than the fast pass allows for (2^60 above a row's first block maximum) send the query tile
    to the exact pass, which rescales its accumulators like a classic online softmax; the result must still match"""
    rng = np.random.default_rng(11)
    trees = [synth._tree(rng, 300, [20, 9]), synth._tree(rng, 90, [7])]
    cfg = synth.AttnConfig("wide", hq, hkv, d, d ** -0.5, 1.0, None, trees)
    b = synth.pack(trees)[0]
    q, k, v = synth.qkv(cfg, b, seed=3, device=dev)
    k = k.clone()
    k[96:] *= 60.0        # keys from the fourth 32-key block on: scores 60 times wider than in the blocks before
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    before = _exact_items()
    out = sa.tree_attn(q, k, v, mask, cfg.scale)
    torch.cuda.synchronize()
    assert _exact_items() > before, "the exact pass did not run"
    ref = _oracle(q, k, v, b, cfg.scale)
    got = out.float().cpu().numpy()
    assert np.isfinite(got).all()
    assert float(np.abs(got - ref).max()) <= TOL
    _pads_selfattend(out, v, b, hq // hkv)
    # and an ordinary launch afterwards leaves the count alone
    k2 = synth.qkv(cfg, b, seed=3, device=dev)[1]
    mid = _exact_items()
    out2 = sa.tree_attn(q, k2, v, mask, cfg.scale)
    torch.cuda.synchronize()
    assert _exact_items() == mid
    assert float(np.abs(out2.float().cpu().numpy() - _oracle(q, k2, v, b, cfg.scale)).max()) <= TOL


@pytest.mark.parametrize("d,hq,hkv", [(128, 4, 2), (256, 4, 2), (512, 4, 1)])
@pytest.mark.parametrize("window", [None, 150])
def test_exact_recomputation_is_the_same_in_both_kernels(dev, d, hq, hkv, window, monkeypatch):
    """the kernel with decoupled waves recomputes the items with too wide a score range itself, after its list; the lockstep
    kernels leave them to a second kernel: the same arithmetic, so the same bits, on a stream where some items take it and
    others do not; each run counts its items"""
    from spinf_serve_amd import attention

    rng = np.random.default_rng(21)
    trees = [synth._tree(rng, 400, [30, 11, 64]), synth._tree(rng, 150, [9, 40]), synth._tree(rng, 260, [])]
    cfg = synth.AttnConfig("wide2", hq, hkv, d, d ** -0.5, 1.0, None, trees)
    b = synth.pack(trees)[0]
    q, k, v = synth.qkv(cfg, b, seed=6, device=dev)
    k = k.clone()
    k[200:330] *= 60.0      # a stretch in the middle of the first trunk: the tiles of the first content that see it are redone
    mask = sa.TreeMask.build(b.art, b.end, b.pos, window=window, device=dev)
    outs, counts = [], []
    for ring in (0, 1):
        monkeypatch.setattr(attention, "RING", ring)
        print(f"case wide d={d} ring={ring} window={window}", flush=True)
        before = _exact_items()
        outs.append(sa.tree_attn(q, k, v, mask, cfg.scale))
        torch.cuda.synchronize()
        counts.append(_exact_items() - before)
    assert counts[0] > 0 and counts[1] > 0, counts
    assert counts[0] == counts[1] * (2 if d == 512 else 1), counts   # (the lockstep kernels take head dim 512 in two launches)
    assert torch.equal(outs[0], outs[1])
    got = outs[1].float().cpu().numpy()
    assert np.isfinite(got).all()
    assert float(np.abs(got - _oracle(q, k, v, b, cfg.scale, window)).max()) <= TOL


def test_exact_recomputation_with_several_items_per_workgroup(dev, monkeypatch):
    """a stream with more work items than workgroups (some workgroups own two or three, of which one or more are redone after the
    list), wide scores in two of its contents: decoupled kernel == lockstep kernels + exact-pass kernel, bit for bit, and every
    content that has no wide scores is bit-identical to the same stream without any"""
    from spinf_serve_amd import attention

    cfg = synth.attention_config("C2", contents=9)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=8, device=dev)
    k_wide = k.clone()
    for slot in (1, 4):
        start, length, *_ = b.jobs[slot]
        k_wide[start + length // 3 : start + length // 2] *= 50.0
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    n_items = mask.for_head_dim(cfg.d, ring=True).plan.n_qtiles * (cfg.hq // 2)
    assert n_items > torch.cuda.get_device_properties(dev).multi_processor_count
    outs, counts = [], []
    for ring in (0, 1):
        monkeypatch.setattr(attention, "RING", ring)
        print(f"case several items per workgroup ring={ring}", flush=True)
        before = _exact_items()
        outs.append(sa.tree_attn(q, k_wide, v, mask, cfg.scale))
        torch.cuda.synchronize()
        counts.append(_exact_items() - before)
    assert counts[0] == counts[1] and counts[1] >= 4, counts
    assert torch.equal(outs[0], outs[1])
    assert torch.isfinite(outs[1].float()).all()
    plain = sa.tree_attn(q, k, v, mask, cfg.scale)
    for slot in range(len(b.jobs)):
        if slot in (1, 4):
            continue
        start, length, *_ = b.jobs[slot]
        assert torch.equal(plain[start : start + length], outs[1][start : start + length]), slot
    start, length, *_ = b.jobs[1]
    sl = slice(start, start + length)
    dense = omask.dense_tree_mask(b.art[sl], b.end[sl] - start, b.pos[sl], None)
    ref = oattn.masked_attention(q[sl].float().cpu().numpy(), k_wide[sl].float().cpu().numpy(), v[sl].float().cpu().numpy(), dense, cfg.scale)
    assert float(np.abs(outs[1][sl].float().cpu().numpy() - ref).max()) <= TOL


@pytest.mark.parametrize("variant", [0, 1, 2])
def test_c4_shape_two_level_tree(dev, variant):
    """variant 0: eight waves, heads of a pair on different waves; 1: one head per item; 2: four waves with two heads each"""
    rng = np.random.default_rng(5)
    lens, parents = [], []
    for _ in range(4):
        node = len(lens)
        lens.append(32); parents.append(-1)
        for _ in range(5):
            lens.append(int(rng.integers(6, 11))); parents.append(node)
    trees = [synth._tree(rng, 700, lens, parents), synth._tree(rng, 130, lens[:7], parents[:7])]
    cfg = synth.AttnConfig("C4-small", 32, 16, 128, 128 ** -0.5, 0.5, None, trees)
    cfg.batches = synth.pack(trees)
    _check(cfg, cfg.batches[0], dev, variant=variant)


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("window", [64, 200, 1024])
def test_sliding_window(dev, window, variant):
    rng = np.random.default_rng(11)
    trees = [synth._tree(rng, 1500, rng.integers(4, 25, 12)), synth._tree(rng, 90, [7, 9])]
    cfg = synth.AttnConfig("C3-small", 16, 8, 256, 1.0 / 16, 0.5, window, trees)
    cfg.batches = synth.pack(trees)
    _check(cfg, cfg.batches[0], dev, window=window, variant=variant)


def test_odd_group_and_mha(dev):
    """groups of 3 and 1 heads run one head per item; groups of 4 and 8 are split into pairs that share an item"""
    rng = np.random.default_rng(2)
    trees = [synth._tree(rng, 200, [9, 17, 4])]
    for hq, hkv, d in ((6, 2, 128), (4, 4, 128), (3, 1, 128), (8, 2, 128), (8, 1, 64), (4, 1, 256), (3, 3, 256)):
        cfg = synth.AttnConfig("odd", hq, hkv, d, d ** -0.5, 1.0, None, trees)
        cfg.batches = synth.pack(trees)
        _check(cfg, cfg.batches[0], dev)


def test_unaligned_packing_and_ragged_length(dev):
    """jobs packed densely (align off) share tiles; the stream length need not be a multiple of the tile"""
    rng = np.random.default_rng(3)
    trees = [synth._tree(rng, 100, [5, 6]), synth._tree(rng, 37, [3]), synth._tree(rng, 260, [11] * 6)]
    cfg = synth.AttnConfig("dense", 4, 2, 64, 0.125, 1.0, None, trees)
    b = synth.pack(trees, align=False)[0]
    _check(cfg, b, dev)
    # ragged: cut the stream after the last real token
    n = int(np.flatnonzero(b.art >= 0)[-1]) + 1
    q, k, v = synth.qkv(cfg, b, device=dev)
    mask = sa.TreeMask.build(b.art[:n], b.end[:n], b.pos[:n], device=dev)
    out = sa.tree_attn(q[:n], k[:n], v[:n], mask, cfg.scale)
    ref = oattn.tree_attention(q[:n].float().cpu().numpy(), k[:n].float().cpu().numpy(), v[:n].float().cpu().numpy(), b.art[:n], b.end[:n], scale=cfg.scale)
    assert np.abs(out.float().cpu().numpy() - ref).max() <= TOL


def test_aligned_query_groups_leave_gaps(dev):
    """a branch group that starts on a block boundary leaves pads inside the job (spinf_serve/packer.py:390-391)"""
    rng = np.random.default_rng(4)
    t = TokenTree(rng.integers(5, 99, 300).tolist(), [rng.integers(5, 99, n).tolist() for n in (9, 12, 7, 30)], [-1, -1, -1, -1], aligned=(2,))
    cfg = synth.AttnConfig("gaps", 8, 4, 128, 128 ** -0.5, 1.0, None, [t])
    b = synth.pack([t])[0]
    assert (b.art[300:] == -1).any()
    _check(cfg, b, dev)


def test_batch_invariance_bit_exact(dev):
    """each content's rows are bit-identical alone, packed with the others, and packed in reverse order"""
    cfg = synth.attention_config("C2", contents=4)
    trees = cfg.trees
    rng = np.random.default_rng(0)
    qs = [torch.from_numpy(rng.standard_normal((t.n_tokens, cfg.hq, cfg.d)).astype(np.float32) * 0.5).to(torch.bfloat16) for t in trees]
    ks = [torch.from_numpy(rng.standard_normal((t.n_tokens, cfg.hkv, cfg.d)).astype(np.float32) * 0.5).to(torch.bfloat16) for t in trees]
    vs = [torch.from_numpy(rng.standard_normal((t.n_tokens, cfg.hkv, cfg.d)).astype(np.float32) * 0.5).to(torch.bfloat16) for t in trees]

    def run(order, window=None):
        b = synth.pack([trees[i] for i in order])[0]
        n = b.length
        q = torch.zeros((n, cfg.hq, cfg.d), dtype=torch.bfloat16)
        k = torch.zeros((n, cfg.hkv, cfg.d), dtype=torch.bfloat16)
        v = torch.zeros((n, cfg.hkv, cfg.d), dtype=torch.bfloat16)
        for slot, i in enumerate(order):
            s0 = b.jobs[slot][0]
            q[s0 : s0 + trees[i].n_tokens] = qs[i]
            k[s0 : s0 + trees[i].n_tokens] = ks[i]
            v[s0 : s0 + trees[i].n_tokens] = vs[i]
        mask = sa.TreeMask.build(b.art, b.end, b.pos, window=window, device=dev)
        out = sa.tree_attn(q.to(dev), k.to(dev), v.to(dev), mask, cfg.scale).cpu()
        return {i: out[b.jobs[slot][0] : b.jobs[slot][0] + trees[i].n_tokens] for slot, i in enumerate(order)}

    for window in (None, 256):
        packed = run([0, 1, 2, 3], window)
        rev = run([3, 2, 1, 0], window)
        for i in range(4):
            alone = run([i], window)[i]
            assert torch.equal(alone, packed[i]), (i, window)
            assert torch.equal(alone, rev[i]), (i, window)


def test_reference_call_signatures(dev):
    """tree_flex_forward (gemma4.py:98-119) and tree_attention (qwen.py:604-623) give the op's result in their layouts"""
    cfg = synth.attention_config("smoke")
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, device=dev)
    masks = sa.block_masks(b, sliding_window=None, device=dev)
    base = sa.tree_attn(q, k, v, masks["full_attention"], cfg.scale)
    out, none = sa.tree_flex_forward(None, q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], masks["full_attention"], scaling=cfg.scale)
    assert none is None and out.shape == (1, b.length, cfg.hq, cfg.d) and out.is_contiguous()
    assert torch.equal(out[0], base)
    o2 = sa.tree_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], masks["full_attention"], cfg.scale)
    assert o2.shape == (1, cfg.hq, b.length, cfg.d) and torch.equal(o2[0].transpose(0, 1), base)
    # compact rows: real rows first, then zero rows
    real = np.flatnonzero(b.art >= 0)
    sidx = torch.from_numpy(real).to(dev)
    rows = (len(real) + 127) // 128 * 128

    def compact(t):
        c = t.new_zeros(rows, t.shape[1], t.shape[2])
        c[: len(real)] = t[sidx]
        return c.transpose(0, 1)[None]

    o3 = sa.tree_attention(compact(q), compact(k), compact(v), masks["full_attention"], cfg.scale, sidx=sidx)
    assert torch.equal(o3[0, :, : len(real)].transpose(0, 1), base[sidx])
    assert (o3[0, :, len(real):] == 0).all()


def _compact_case(name):
    """-> (cfg, batch, window): streams with pads in different places"""
    rng = np.random.default_rng(21)
    if name == "c2":          # head dim 256, eight-wave kernel; alignment pads after every job
        cfg = synth.attention_config("C2", contents=3)
        return cfg, cfg.batches[0], None
    if name == "gaps":        # pads INSIDE a job (aligned branch group), head dim 128
        t = TokenTree(rng.integers(5, 99, 300).tolist(), [rng.integers(5, 99, n).tolist() for n in (9, 12, 7, 30)], [-1, -1, -1, -1], aligned=(2,))
        cfg = synth.AttnConfig("gaps", 8, 4, 128, 128 ** -0.5, 1.0, None, [t])
        return cfg, synth.pack([t])[0], None
    if name == "dense":       # no alignment: pads only at the end of the stream, head dim 64
        trees = [synth._tree(rng, 100, [5, 6]), synth._tree(rng, 37, [3]), synth._tree(rng, 260, [11] * 6)]
        cfg = synth.AttnConfig("dense", 4, 2, 64, 0.125, 1.0, None, trees)
        return cfg, synth.pack(trees, align=False)[0], None
    if name == "window":      # sliding layer
        trees = [synth._tree(rng, 700, [9, 14, 30]), synth._tree(rng, 150, [8])]
        cfg = synth.AttnConfig("window", 4, 2, 256, 1.0 / 16, 0.5, 200, trees)
        return cfg, synth.pack(trees)[0], 200
    trees = [synth._tree(rng, 200, [20, 9]), synth._tree(rng, 90, [7])]   # "mha": three heads, one head per work item
    cfg = synth.AttnConfig("mha", 3, 3, 128, 128 ** -0.5, 1.0, None, trees)
    return cfg, synth.pack(trees)[0], None


@pytest.mark.parametrize("name", ["c2", "gaps", "dense", "window", "mha"])
def test_compact_rows_equal_the_stream_layout_call(dev, name):
    """tree_attention with sidx (spinf_serve/models/qwen35/qwen.py:613-622): q, k, v hold the real rows only.  The reference
    scatters them into the stream layout (zero rows for pads) and gathers the output back; the kernel's row map must give the
    same bits for every real row, zero for the rows after them, and must not touch memory of other rows."""
    cfg, b, window = _compact_case(name)
    q, k, v = synth.qkv(cfg, b, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, window, device=dev)
    real = np.flatnonzero(b.art >= 0)
    sidx = torch.from_numpy(real).to(dev)
    R = len(real)
    rows = R + 37   # a few spare rows, as the reference's row buckets have
    # the reference's way: zero rows at the pad positions of the stream layout
    zq, zk, zv = (torch.zeros_like(t).index_copy_(0, sidx, t[sidx]) for t in (q, k, v))
    want = sa.tree_attn(zq, zk, zv, mask, cfg.scale)[sidx]
    ref = _oracle(zq, zk, zv, b, cfg.scale, window)
    assert float(np.abs(want.float().cpu().numpy() - ref[real]).max()) <= TOL

    def compact(t):
        c = torch.full((rows, t.shape[1], t.shape[2]), 7.0, dtype=t.dtype, device=dev)   # spare rows hold junk on purpose
        c[:R] = t[sidx]
        return c

    cq, ck, cv = compact(q), compact(k), compact(v)
    got = sa.tree_attn(cq, ck, cv, mask, cfg.scale, sidx=sidx)
    assert got.shape == (rows, cfg.hq, cfg.d)
    assert torch.equal(got[:R], want)
    assert (got[R:] == 0).all()
    # through the Qwen stack's function, [1, heads, rows, d] views
    o = sa.tree_attention(cq.transpose(0, 1)[None], ck.transpose(0, 1)[None], cv.transpose(0, 1)[None], mask, cfg.scale, sidx=sidx)
    assert o.shape == (1, cfg.hq, rows, cfg.d) and torch.equal(o[0].transpose(0, 1), got)


def test_compact_rows_through_the_exact_pass(dev):
    """the rescaling pass reads and writes through the same row map"""
    rng = np.random.default_rng(11)
    trees = [synth._tree(rng, 300, [20, 9]), synth._tree(rng, 90, [7])]
    cfg = synth.AttnConfig("wide", 4, 2, 128, 128 ** -0.5, 1.0, None, trees)
    b = synth.pack(trees)[0]
    q, k, v = synth.qkv(cfg, b, seed=3, device=dev)
    k = k.clone()
    k[96:] *= 60.0
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    real = np.flatnonzero(b.art >= 0)
    sidx = torch.from_numpy(real).to(dev)
    want = sa.tree_attn(q, k, v, mask, cfg.scale)[sidx]
    before = _exact_items()
    got = sa.tree_attn(q[sidx].contiguous(), k[sidx].contiguous(), v[sidx].contiguous(), mask, cfg.scale, sidx=sidx)
    torch.cuda.synchronize()
    assert _exact_items() > before, "the exact pass did not run"
    assert torch.equal(got, want)


def _image_stream(seed=8):
    """two jobs with image placeholders: groups that straddle tile borders, two in one block, one inside a branch"""
    rng = np.random.default_rng(seed)
    t1 = TokenTree(rng.integers(5, 99, 700).tolist(), [rng.integers(5, 99, n).tolist() for n in (40, 9, 70)], [-1, -1, -1])
    t2 = synth._tree(rng, 150, [20])
    trees = [t1, t2]
    b = synth.pack(trees)[0]
    grp = np.full(b.length, -1, np.int32)
    for gid, (a, e) in enumerate([(10, 22), (24, 30), (100, 356), (500, 530), (705, 735), (768 + 128 + 5, 768 + 128 + 40)]):
        grp[a:e] = gid
    grp[b.art < 0] = -1
    return trees, b, grp


@pytest.mark.parametrize("hq,hkv,d", [(4, 2, 256), (3, 3, 128), (4, 1, 64)])
@pytest.mark.parametrize("window,windowed", [(None, False), (64, False), (64, True)])
def test_image_groups_see_each_other_both_ways(dev, hq, hkv, d, window, windowed):
    """spinf_serve/scorer.py:184-198: the placeholders of an image attend to each other both ways (later keys too), on the
    global layers, on the sliding layers past the window, or on the sliding layers within it"""
    trees, b, grp = _image_stream()
    cfg = synth.AttnConfig("img", hq, hkv, d, d ** -0.5, 1.0, window, trees)
    q, k, v = synth.qkv(cfg, b, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, window, device=dev, grp=grp, grp_windowed=windowed)
    out = sa.tree_attn(q, k, v, mask, cfg.scale)
    dense = omask.dense_tree_mask(b.art, b.end, b.pos, window, grp, windowed)
    ref = oattn.masked_attention(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), dense, cfg.scale)
    got = out.float().cpu().numpy()
    assert float(np.abs(got - ref).max()) <= TOL
    # the groups matter: without them the same rows come out differently
    plain = sa.tree_attn(q, k, v, sa.TreeMask.build(b.art, b.end, b.pos, window, device=dev), cfg.scale).float().cpu().numpy()
    assert np.abs(plain[grp >= 0] - ref[grp >= 0]).max() > 10 * TOL
    assert np.array_equal(plain[(grp < 0) & (b.art < 0)], got[(grp < 0) & (b.art < 0)])      # pads: their own V row either way


def test_block_masks_with_images(dev):
    """bidir_all (the unified checkpoint): groups on both masks; otherwise the global mask stays causal and the sliding one
    takes the groups within the window (scorer.py:186-198)"""
    trees, b, grp = _image_stream()
    cfg = synth.AttnConfig("img", 4, 2, 128, 128 ** -0.5, 1.0, 64, trees)
    q, k, v = synth.qkv(cfg, b, device=dev)
    qn, kn, vn = (t.float().cpu().numpy() for t in (q, k, v))
    for bidir_all in (True, False):
        masks = sa.block_masks(b, sliding_window=64, device=dev, grp=grp, bidir_all=bidir_all)
        want_full = omask.dense_tree_mask(b.art, b.end, b.pos, None, grp if bidir_all else None)
        want_slid = omask.dense_tree_mask(b.art, b.end, b.pos, 64, grp, not bidir_all)
        for name, dense in (("full_attention", want_full), ("sliding_attention", want_slid)):
            got = sa.tree_attn(q, k, v, masks[name], cfg.scale).float().cpu().numpy()
            assert float(np.abs(got - oattn.masked_attention(qn, kn, vn, dense, cfg.scale)).max()) <= TOL, (bidir_all, name)


def test_image_groups_through_the_exact_pass(dev):
    trees, b, grp = _image_stream()
    cfg = synth.AttnConfig("img", 4, 2, 128, 128 ** -0.5, 1.0, None, trees)
    q, k, v = synth.qkv(cfg, b, seed=3, device=dev)
    k = k.clone()
    k[96:] *= 60.0
    mask = sa.TreeMask.build(b.art, b.end, b.pos, None, device=dev, grp=grp)
    before = _exact_items()
    out = sa.tree_attn(q, k, v, mask, cfg.scale)
    torch.cuda.synchronize()
    assert _exact_items() > before, "the exact pass did not run"
    dense = omask.dense_tree_mask(b.art, b.end, b.pos, None, grp)
    ref = oattn.masked_attention(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), dense, cfg.scale)
    assert float(np.abs(out.float().cpu().numpy() - ref).max()) <= TOL


@pytest.mark.parametrize("hq,hkv", [(8, 1), (4, 2)])
def test_head_dim_512(dev, hq, hkv):
    """the full-attention layers of the Gemma-4 checkpoints: head dim 512, one key / value head (spinf_serve/models/gemma4.py:39-41)"""
    rng = np.random.default_rng(12)
    trees = [synth._tree(rng, 300, [20, 9, 14]), synth._tree(rng, 90, [7]), synth._tree(rng, 33, [])]
    cfg = synth.AttnConfig("d512", hq, hkv, 512, 512 ** -0.5, 0.5, None, trees)
    b = synth.pack(trees)[0]
    _check(cfg, b, dev)
    _check(cfg, b, dev, window=100)
    # bit-identical per job alone and packed
    q, k, v = synth.qkv(cfg, b, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    packed = sa.tree_attn(q, k, v, mask, cfg.scale)
    start, length, *_ = b.jobs[1]
    b1 = synth.pack([trees[1]])[0]
    m1 = sa.TreeMask.build(b1.art, b1.end, b1.pos, device=dev)
    sl = slice(start, start + length)
    pad = b1.length - length
    ext = lambda t: torch.cat([t[sl], t.new_zeros(pad, *t.shape[1:])])  # noqa: E731
    alone = sa.tree_attn(ext(q), ext(k), ext(v), m1, cfg.scale)
    assert torch.equal(alone[:length], packed[sl])
    # compact rows
    real = np.flatnonzero(b.art >= 0)
    sidx = torch.from_numpy(real).to(dev)
    got = sa.tree_attn(q[sidx].contiguous(), k[sidx].contiguous(), v[sidx].contiguous(), mask, cfg.scale, sidx=sidx)
    assert torch.equal(got, packed[sidx])


@pytest.mark.parametrize("seed", range(12))
def test_random_forests_against_the_oracle(dev, seed):
    """seeded random cases over everything at once: forest shape, packing, head geometry, window, image groups or compact rows"""
    rng = np.random.default_rng(1000 + seed)
    trees = []
    for _ in range(int(rng.integers(1, 4))):
        nb = int(rng.integers(0, 6))
        lens = [int(x) for x in rng.integers(1, 40, nb)]
        parents = [-1 if i == 0 or rng.random() < 0.5 else int(rng.integers(0, i)) for i in range(nb)]
        parents = [p_ if p_ < 0 or parents[p_] < 0 else -1 for p_ in parents]
        aligned = [i for i in range(nb) if parents[i] < 0 and rng.random() < 0.2]
        trunk = int(rng.integers(0 if nb else 1, 400))
        trees.append(TokenTree(rng.integers(5, 99, trunk).tolist(), [rng.integers(5, 99, n).tolist() for n in lens], parents, tuple(aligned)))
    b = synth.pack(trees, align=bool(rng.integers(0, 2)))[0]
    hq, hkv, d = [(4, 2, 64), (8, 2, 128), (3, 3, 128), (4, 2, 256), (2, 1, 256), (4, 1, 512)][int(rng.integers(0, 6))]
    window = [None, 23, 150][int(rng.integers(0, 3))]
    mode = int(rng.integers(0, 3))          # 0 plain, 1 image groups, 2 compact rows
    grp, windowed = None, False
    if mode == 1:
        grp = np.full(b.length, -1, np.int32)
        for gid in range(int(rng.integers(1, 4))):
            a = int(rng.integers(0, b.length))
            grp[a : a + int(rng.integers(1, 90))] = gid
        grp[b.art < 0] = -1
        windowed = bool(rng.integers(0, 2)) and window is not None
    cfg = synth.AttnConfig("rand", hq, hkv, d, d ** -0.5, 1.0, window, trees)
    q, k, v = synth.qkv(cfg, b, seed=seed, device=dev)
    print(f"case seed={seed} n={b.length} heads={hq}/{hkv} d={d} window={window} mode={mode}", flush=True)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, window, device=dev, grp=grp, grp_windowed=windowed)
    dense = omask.dense_tree_mask(b.art, b.end, b.pos, window, grp, windowed)
    ref = oattn.masked_attention(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), dense, cfg.scale)
    if mode == 2:
        real = np.flatnonzero(b.art >= 0)
        sidx = torch.from_numpy(real).to(dev)
        got = sa.tree_attn(q[sidx].contiguous(), k[sidx].contiguous(), v[sidx].contiguous(), mask, cfg.scale, sidx=sidx).float().cpu().numpy()
        assert float(np.abs(got - ref[real]).max()) <= TOL
    else:
        got = sa.tree_attn(q, k, v, mask, cfg.scale).float().cpu().numpy()
        assert float(np.abs(got - ref).max()) <= TOL


def test_argument_errors(dev):
    cfg = synth.attention_config("smoke")
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    with pytest.raises(ValueError):
        sa.tree_attn(q[:, :3], k, v, mask, cfg.scale)            # 3 query heads over 2 kv heads
    with pytest.raises(ValueError):
        sa.tree_attn(q[:100], k[:100], v[:100], mask, cfg.scale)  # mask of another length
    with pytest.raises(ValueError):
        sa.tree_attn(q.float(), k, v, mask, cfg.scale)
    with pytest.raises(RuntimeError):
        sa.tree_attn(q.cpu(), k.cpu(), v.cpu(), mask, cfg.scale)  # no CPU path
    with pytest.raises(Exception, match="variant 3"):
        sa.tree_attn(q, k, v, mask, cfg.scale, variant=3)         # the decoupled kernel at head dim 128 wants a static schedule


@pytest.mark.parametrize("window", [None, 256])
def test_kernel_and_schedule_choices_give_the_same_bits(dev, window, monkeypatch):
    """the lockstep kernel on its queue, the lockstep kernel on the static lists and the kernel with decoupled waves: one result,
    and no wave of the decoupled kernel gave up a wait"""
    import ctypes

    from spinf_serve_amd import attention

    cfg = synth.attention_config("C2", contents=5)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=4, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, window=window, device=dev)
    outs = []
    aborts0 = _ring_aborts()
    for ring, static in ((0, 0), (0, 1), (1, 0)):
        monkeypatch.setattr(attention, "RING", ring)
        monkeypatch.setattr(attention, "STATIC", static)
        print(f"case ring={ring} static={static} window={window}", flush=True)
        outs.append(sa.tree_attn(q, k, v, mask, cfg.scale))
        torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert _ring_aborts() == aborts0


@pytest.mark.parametrize("window", [None, 200])
def test_head_dim_128_decoupled_kernel_gives_the_lockstep_bits(dev, window, monkeypatch):
    """the kernel with decoupled waves at head dim 128 (the library's variant 3: 64-key tiles, two 32-key blocks per tile and wave;
    not the default there, the lockstep kernel is faster on long trunks): the same bits as the lockstep kernel on a two-level tree
    with a long trunk, on short ragged trees, and through the entry point that allocates nothing; no wave gives up a wait"""
    from spinf_serve_amd import attention

    rng = np.random.default_rng(31)
    cases = [synth.attention_config("C4", contents=1), synth.attention_config("smoke"),
             synth.AttnConfig("ragged", 8, 2, 128, 128 ** -0.5, 1.0, None, [synth._tree(rng, 333, [17, 5, 64, 9]), synth._tree(rng, 70, []), synth._tree(rng, 1, [3])])]
    cases[2].batches = synth.pack(cases[2].trees)
    for cfg in cases:
        b = cfg.batches[0]
        q, k, v = synth.qkv(cfg, b, seed=12, device=dev)
        mask = sa.TreeMask.build(b.art, b.end, b.pos, window=window, device=dev)
        monkeypatch.setattr(attention, "RING", 0)
        want = sa.tree_attn(q, k, v, mask, cfg.scale)
        torch.cuda.synchronize()
        monkeypatch.setattr(attention, "RING", 1)
        before = _ring_aborts()
        print(f"case d=128 decoupled kernel {cfg.name} n={b.length} window={window}", flush=True)
        got = sa.tree_attn(q, k, v, mask, cfg.scale)
        out = torch.full_like(want, float("nan"))
        sa.tree_attn_noalloc(q, k, v, mask, out, cfg.scale)
        torch.cuda.synchronize()
        assert _ring_aborts() == before
        assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
        assert torch.equal(out, want)


@pytest.mark.parametrize("window", [None, 300])
def test_head_dim_512_kernel_choices_give_the_same_bits(dev, window, monkeypatch):
    """head dim 512: the kernel with decoupled waves (one launch, the whole output row in accumulation registers) and the lockstep
    kernel (two launches of 256 value dims) give one result, on a stream long enough for several items per workgroup and with
    its last query tile cut off by the end of the stream; no wave of the decoupled kernel gave up a wait"""
    import ctypes

    from spinf_serve_amd import attention

    cfg = synth.attention_config("C2_512", contents=6)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=5, device=dev)
    n = b.length - 37   # a stream that ends inside a query tile and inside a key tile
    q, k, v = q[:n].contiguous(), k[:n].contiguous(), v[:n].contiguous()
    mask = sa.TreeMask.build(b.art[:n], b.end[:n], b.pos[:n], window=window, device=dev)
    outs = []
    aborts0 = _ring_aborts()
    for ring in (0, 1):
        monkeypatch.setattr(attention, "RING", ring)
        print(f"case d512 ring={ring} window={window} n={n}", flush=True)
        outs.append(sa.tree_attn(q, k, v, mask, cfg.scale))
        torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
    assert _ring_aborts() == aborts0
    # and both against the oracle on one content
    start, length, *_ = b.jobs[0]
    sl = slice(start, start + length)
    dense = omask.dense_tree_mask(b.art[sl], b.end[sl] - start, b.pos[sl], window)
    ref = oattn.masked_attention(q[sl].float().cpu().numpy(), k[sl].float().cpu().numpy(), v[sl].float().cpu().numpy(), dense, cfg.scale)
    assert float(np.abs(outs[1][sl].float().cpu().numpy() - ref).max()) <= TOL


def test_calls_on_two_streams_do_not_share_cursors(dev):
    """calls interleaved on two streams, not synchronised with each other, give the bits of the same calls one after the other"""
    cfgs = [synth.attention_config("C2", seed=s, contents=4 + 3 * s) for s in range(2)]
    work = []
    for cfg in cfgs:
        b = cfg.batches[0]
        work.append((synth.qkv(cfg, b, seed=9, device=dev), sa.TreeMask.build(b.art, b.end, b.pos, device=dev), cfg.scale))
    serial = [sa.tree_attn(*qkv, mask, scale) for qkv, mask, scale in work]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=dev) for _ in range(2)]
    outs = [[], []]
    for rep in range(6):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                qkv, mask, scale = work[i]
                outs[i].append(sa.tree_attn(*qkv, mask, scale))
    torch.cuda.synchronize()
    for i in range(2):
        assert all(torch.equal(o, serial[i]) for o in outs[i])


def test_groups_of_the_windowed_checkpoint_are_rejected_on_a_global_layer(dev):
    import ctypes as C

    from spinf_serve_amd import _lib

    cfg = synth.attention_config("smoke")
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    items, list_ptr, n_items = mask.schedule(cfg.hq // 2)
    grp = torch.full((b.length,), -1, dtype=torch.int32, device=dev)
    out = torch.empty_like(q)
    a = attention._attn_args(q, k, v, out, b.length, mask.art, mask.end, mask.pos, mask.kv_idx, mask.kv_bits, items, list_ptr, n_items, cfg.scale, 0, 0, None, None, grp, 2, 64)
    lib = sa.load_library()
    assert lib.spinf_tree_attn_fwd(C.byref(a), None) == -1 and b"global layer takes no groups" in lib.spinf_last_error()


def test_allocating_entry_point_under_graph_capture(dev):
    """a stream that has made one call can record the call into a graph: the stream's cursor block goes with the graph, replays give
    the eager result every time (with eager calls on the same stream in between, which take a new block), and a capture on a stream
    that never made a call is refused with a message instead of allocating"""
    cfg = synth.attention_config("C2", contents=3)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=12, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    want = sa.tree_attn(q, k, v, mask, cfg.scale)
    torch.cuda.synchronize()
    s = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(s):
        warm = sa.tree_attn(q, k, v, mask, cfg.scale)   # the stream's block exists from here on
    s.synchronize()
    assert torch.equal(warm, want)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        out = sa.tree_attn(q, k, v, mask, cfg.scale)
    for rep in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        with torch.cuda.stream(s):   # eager work on the same stream between the replays
            again = sa.tree_attn(q, k, v, mask, cfg.scale)
        s.synchronize()
        assert torch.equal(again, want)
    fresh = torch.cuda.Stream(device=dev)
    g2 = torch.cuda.CUDAGraph()
    with pytest.raises(ValueError, match="before the capture"):
        with torch.cuda.graph(g2, stream=fresh):
            sa.tree_attn(q, k, v, mask, cfg.scale)
    torch.cuda.synchronize()


@pytest.mark.parametrize("ring", [0, 1])
def test_several_calls_recorded_by_one_capture_share_the_streams_block(dev, ring, monkeypatch):
    """a layer stack records one attention call per layer into one graph: the calls of ONE capture on a stream share the stream's
    cursor block (the graph runs them in recorded order); a second graph on the same stream needs a block of its own, which an
    eager call between the captures provides.  Both kernels (lockstep with its cursors, decoupled with its redo list)."""
    from spinf_serve_amd import attention

    monkeypatch.setattr(attention, "RING", ring)
    cfg = synth.attention_config("C2", contents=3)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=13, device=dev)
    q2 = (q.float() * 0.5 + 0.25).to(torch.bfloat16)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    want1, want2 = sa.tree_attn(q, k, v, mask, cfg.scale), sa.tree_attn(q2, k, v, mask, cfg.scale)
    torch.cuda.synchronize()
    s = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(s):
        sa.tree_attn(q, k, v, mask, cfg.scale)
    s.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        out1 = sa.tree_attn(q, k, v, mask, cfg.scale)
        out2 = sa.tree_attn(q2, k, v, mask, cfg.scale)
        out3 = sa.tree_attn(out2, k, v, mask, cfg.scale)   # a call that depends on the one before it
    want3 = sa.tree_attn(want2, k, v, mask, cfg.scale)
    for rep in range(3):
        for o in (out1, out2, out3):
            o.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out1, want1) and torch.equal(out2, want2) and torch.equal(out3, want3), rep
    g2 = torch.cuda.CUDAGraph()
    with pytest.raises(ValueError, match="stays with that graph"):   # the stream's only block went with the first graph
        with torch.cuda.graph(g2, stream=s):
            sa.tree_attn(q, k, v, mask, cfg.scale)
    torch.cuda.synchronize()
    with torch.cuda.stream(s):
        sa.tree_attn(q, k, v, mask, cfg.scale)   # takes a new block for the stream
    s.synchronize()
    g3 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g3, stream=s):
        out4 = sa.tree_attn(q2, k, v, mask, cfg.scale)
    g3.replay()
    g.replay()
    torch.cuda.synchronize()
    assert torch.equal(out4, want2) and torch.equal(out1, want1) and torch.equal(out3, want3)


@pytest.mark.parametrize("d,limit,wide", [(128, 1, False), (128, 1, True), (256, 1, False), (256, 1, True), (256, 3, False), (512, 1, False), (512, 1, True)])
def test_a_wave_that_gives_up_a_wait_costs_time_not_rows(dev, d, limit, wide, monkeypatch):
    """the decoupled kernel's landing: the waves are told (from the host, spinf_attn_args.debug_expire) to give up a wait after
    `limit` polls instead of 2^18, so every wave that has to wait for a tile at all gives up, as after a real time-out; its
    workgroup leaves the ring and computes its list again before it ends, one tile at a time between barriers.
    Every kernel exits normally, the aborts are counted, and the output equals the lockstep kernel's bit for bit, also where items
    go on to the exact recomputation (wide) and with a window."""
    from spinf_serve_amd import attention

    cfg = synth.attention_config({128: "C4", 256: "C2", 512: "C2_512"}[d], contents={128: 1, 256: 12, 512: 6}[d])
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=9, device=dev)
    if wide:
        k = (k.float() * 60).to(torch.bfloat16)   # scores far above the first block's maximum: items go to the exact recomputation
    for window in (None, 200):
        mask = sa.TreeMask.build(b.art, b.end, b.pos, window=window, device=dev)
        monkeypatch.setattr(attention, "RING", 0)
        monkeypatch.setattr(attention, "DEBUG_EXPIRE", 0)
        want = sa.tree_attn(q, k, v, mask, cfg.scale)
        torch.cuda.synchronize()
        monkeypatch.setattr(attention, "RING", 1)
        before, exact0 = _ring_aborts(), _exact_items()
        print(f"case d={d} limit={limit} wide={wide} window={window}: plain ring pass", flush=True)
        plain = sa.tree_attn(q, k, v, mask, cfg.scale)
        torch.cuda.synchronize()
        assert _ring_aborts() == before
        exact_plain = _exact_items() - exact0
        monkeypatch.setattr(attention, "DEBUG_EXPIRE", limit)
        print(f"case d={d} limit={limit} wide={wide} window={window}: waits run out after {limit} polls", flush=True)
        got = sa.tree_attn(q, k, v, mask, cfg.scale)
        torch.cuda.synchronize()
        monkeypatch.setattr(attention, "DEBUG_EXPIRE", 0)
        assert _ring_aborts() > before, "no wave took the abort path"
        assert torch.equal(plain, want)
        assert torch.equal(got, want), float((got.float() - want.float()).abs().max())
        if wide:
            assert exact_plain > 0 and _exact_items() - exact0 == 2 * exact_plain   # the same items were recomputed exactly, once each
        again = sa.tree_attn(q, k, v, mask, cfg.scale)   # and the next launch starts clean
        torch.cuda.synchronize()
        assert torch.equal(again, want) and _ring_aborts() == before + (_ring_aborts() - before)
