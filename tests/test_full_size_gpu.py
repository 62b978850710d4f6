"""The benchmark configurations at their full sizes (C2: 24 contents in one pass; C3: the fullest pass of the 512 contents, global
and sliding; C4: 64 contents of 10 k tokens in one launch; C5: 128 contents, 311,296 tokens), checked through properties that do not need the oracle to process the whole stream: a content's rows are bit-identical alone and
inside the full pack, the delta rule is exactly linear under a power-of-two scaling of v, and one content of the pack is
compared with the float64 oracle."""

import numpy as np
import pytest
import torch

import spinf_serve_amd as sa
from oracle import attention as oattn
from oracle import gdn as ogdn
from spinf_serve_amd import synth

pytestmark = pytest.mark.gpu
TOL = 2e-2       # attention: bf16 outputs of up to ~4 in size against float64
GDN_TOL = 2e-3   # the delta-rule scan: outputs of unit scale (measured 3e-4)


def _np(t):
    return t.float().cpu().numpy()


def test_c2_full_pack_is_invariant_and_matches_the_oracle(dev):
    cfg = synth.attention_config("C2")
    assert len(cfg.trees) == 24 and len(cfg.batches) == 1
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=0, device=dev)
    masks = sa.block_masks(b, sliding_window=None, device=dev)
    out = sa.tree_attn(q, k, v, masks["full_attention"], cfg.scale)
    torch.cuda.synchronize()
    for slot in (0, 11, 23):
        s0, n = b.jobs[slot][0], cfg.trees[slot].n_tokens
        one = synth.pack([cfg.trees[slot]])[0]
        m1 = sa.TreeMask.build(one.art, one.end, one.pos, window=None, device=dev)
        pad = one.length - n

        def z(t):
            t = t[s0 : s0 + n]
            return torch.cat([t, torch.zeros((pad, *t.shape[1:]), dtype=t.dtype, device=dev)]) if pad else t.contiguous()

        alone = sa.tree_attn(z(q), z(k), z(v), m1, cfg.scale)
        assert torch.equal(alone[:n], out[s0 : s0 + n]), slot
    # one content against the dense float64 oracle
    s0 = b.jobs[5][0]
    one = synth.pack([cfg.trees[5]])[0]
    n = cfg.trees[5].n_tokens
    want = oattn.tree_attention(_np(q[s0 : s0 + n]), _np(k[s0 : s0 + n]), _np(v[s0 : s0 + n]), one.art[:n], one.end[:n], pos=one.pos[:n], scale=cfg.scale)
    real = one.art[:n] >= 0
    err = float(np.abs(_np(out[s0 : s0 + n])[real] - want[real]).max())
    print(f"C2 full pack, content 5: max abs err {err:.3e}", flush=True)
    assert err <= TOL, f"C2 full pack, content 5: max abs error {err:.3e} against the float64 oracle, tolerance {TOL:.0e}"


def test_c5_full_stream_properties(dev):
    cfg = synth.gdn_config("C5")
    assert len(cfg.trees) == 128
    t = synth.gdn_inputs(cfg, seed=0, device=dev)
    plan = cfg.plan(dev)
    o = sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], plan)
    # exact linearity in v under a power-of-two scale: every product and rounding commutes with it
    o2 = sa.gdn_tree(t["q"], t["k"], t["v"] * 2, t["g"], t["beta"], plan)
    torch.cuda.synchronize()
    assert torch.equal(o2, o * 2)
    del o2
    b = cfg.batch
    for slot in (0, 77, 127):
        s0 = b.jobs[slot][0]
        n = cfg.trees[slot].n_tokens
        one = synth.GdnConfig("one", cfg.h, cfg.hv, cfg.dk, cfg.dv, [cfg.trees[slot]])
        one.batch = synth.pack([cfg.trees[slot]])[0]
        pad = one.batch.length - n

        def z(x):
            x = x[s0 : s0 + n]
            return torch.cat([x, torch.zeros((pad, *x.shape[1:]), dtype=x.dtype, device=dev)]) if pad else x.contiguous()

        alone = sa.gdn_tree(z(t["q"]), z(t["k"]), z(t["v"]), z(t["g"]), z(t["beta"]), one.plan(dev))
        assert torch.equal(alone[:n], o[s0 : s0 + n]), slot
        if slot == 77:
            want = ogdn.tree_scan(*(_np(z(t[x])) for x in ("q", "k", "v", "g", "beta")), one.batch.prev, one.batch.art >= 0)
            err = float(np.abs(_np(alone) - want).max())
            print(f"C5 full stream, content 77: max abs err {err:.3e}", flush=True)
            assert err <= GDN_TOL, f"C5 full stream, content 77: max abs error {err:.3e} against the float64 recurrence, tolerance {GDN_TOL:.0e}"


def _device_qkv(cfg, n, dev, seed):
    """Q, K, V of the configuration's shape and value distribution, drawn on the device (the properties checked below do not
    depend on which generator made the values; the host generator of synth.qkv takes half a minute at these sizes)"""
    gen = torch.Generator(device=dev).manual_seed(seed)

    def mk(h):
        out = torch.empty((n, h, cfg.d), dtype=torch.bfloat16, device=dev)
        step = max(1, (1 << 26) // (h * cfg.d))
        for a in range(0, n, step):
            b = min(n, a + step)
            out[a:b] = (torch.randn((b - a, h, cfg.d), generator=gen, device=dev) * cfg.std).to(torch.bfloat16)
        return out

    return mk(cfg.hq), mk(cfg.hkv), mk(cfg.hkv)


def _check_pack(cfg, b, trees, slots, oracle_slot, oracle_heads, window, dev, seed):
    q, k, v = _device_qkv(cfg, b.length, dev, seed)
    masks = sa.block_masks(b, sliding_window=window, device=dev)
    out = sa.tree_attn(q, k, v, masks["sliding_attention" if window else "full_attention"], cfg.scale)
    torch.cuda.synchronize()
    for slot in slots:
        s0, n = b.jobs[slot][0], trees[slot].n_tokens
        one = synth.pack([trees[slot]])[0]
        m1 = sa.TreeMask.build(one.art, one.end, one.pos, window=window, device=dev)
        pad = one.length - n

        def z(t):
            t = t[s0 : s0 + n]
            return torch.cat([t, torch.zeros((pad, *t.shape[1:]), dtype=t.dtype, device=dev)]) if pad else t.contiguous()

        alone = sa.tree_attn(z(q), z(k), z(v), m1, cfg.scale)
        assert torch.equal(alone[:n], out[s0 : s0 + n]), (slot, window)
    # one content, the first `oracle_heads` query heads of it, against the dense float64 oracle
    s0, n = b.jobs[oracle_slot][0], trees[oracle_slot].n_tokens
    one = synth.pack([trees[oracle_slot]])[0]
    hk = max(1, oracle_heads * cfg.hkv // cfg.hq)
    want = oattn.tree_attention(_np(q[s0 : s0 + n, :oracle_heads]), _np(k[s0 : s0 + n, :hk]), _np(v[s0 : s0 + n, :hk]), one.art[:n], one.end[:n],
                                pos=one.pos[:n], window=window, scale=cfg.scale)
    real = one.art[:n] >= 0
    err = float(np.abs(_np(out[s0 : s0 + n, :oracle_heads])[real] - want[real]).max())
    what = f"{cfg.name} pack of {b.length} tokens, window {window}, content {oracle_slot} ({n} tokens, {oracle_heads} heads)"
    print(f"{what}: max abs err {err:.3e}", flush=True)
    assert err <= TOL, f"{what}: max abs error {err:.3e} against the float64 oracle, tolerance {TOL:.0e}"


@pytest.mark.parametrize("window", [None, 1024])
def test_c3_largest_pass_is_invariant_and_matches_the_oracle(dev, window):
    """C3's fullest pass (<= 65,536 tokens of the 512 contents), as a global and as a sliding-window (1,024) layer"""
    cfg = synth.attention_config("C3")
    assert len(cfg.trees) == 512 and len(cfg.batches) >= 12
    b = max(cfg.batches, key=lambda x: x.length)
    trees = [cfg.trees[k] for *_, k in b.jobs]
    small = min(range(len(trees)), key=lambda i: trees[i].n_tokens)
    _check_pack(cfg, b, trees, (0, len(trees) // 2, len(trees) - 1), small, cfg.hq, window, dev, seed=3)


def test_c4_full_pack_is_invariant_and_matches_the_oracle(dev):
    """C4 at its full size: 64 contents of 10 k tokens (two-level trees) in one launch, 32 / 16 heads, head dim 128"""
    cfg = synth.attention_config("C4")
    assert len(cfg.trees) == 64 and len(cfg.batches) == 1
    b = cfg.batches[0]
    _check_pack(cfg, b, [cfg.trees[k] for *_, k in b.jobs], (0, 37, 63), 5, 2, None, dev, seed=4)
