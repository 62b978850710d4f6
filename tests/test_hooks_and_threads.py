"""The pieces around the kernels that the forward pass of the reference touches: the capture hooks of the attention and the
recurrent-layer interfaces (spinf_serve/models/gemma4.py:98-119, spinf_serve/models/qwen35/qwen.py:514-623), the registration
with transformers (gemma4.py:121-122), the plan compilers under threads, and the CPU baseline's fp32 arithmetic against the
float64 oracle."""

import threading
import types

import numpy as np
import pytest
import torch

import spinf_serve_amd as sa
from oracle import attention as oattn
from oracle import cpu_baseline
from oracle import gdn as ogdn
from oracle import mask as omask
from spinf_serve_amd import attention, synth


# ----------------------------------------------------------------------------------------------------------------- CPU

def test_registration_with_transformers():
    from transformers import AttentionInterface

    sa.register_tree_attention("tree_flex_test")
    assert AttentionInterface()["tree_flex_test"] is sa.tree_flex_forward
    sa.register_tree_attention("tree_flex_test")   # a second call leaves it alone
    assert AttentionInterface()["tree_flex_test"] is sa.tree_flex_forward


def test_ops_are_registered_with_torch_library():
    """the kernels are opaque torch.library ops (inductor never traces into them); the scan mutates its output and state tensors"""
    for name in ("tree_attn", "gdn_scan", "lm_logprobs", "lm_head_logprobs"):
        assert hasattr(torch.ops.spinf, name), name
    schema = str(torch.ops.spinf.gdn_scan.default._schema)
    assert "Tensor(a" in schema and "o" in schema and "-> ()" in schema, schema
    with pytest.raises(RuntimeError):   # no CPU path
        sa.gdn.recurrent(torch.zeros(1, 4, 1, 128, dtype=torch.bfloat16), torch.zeros(1, 4, 1, 128, dtype=torch.bfloat16), torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16),
                         torch.zeros(1, 4, 2), torch.zeros(1, 4, 2, dtype=torch.bfloat16), 1.0, torch.tensor([0, 4]), 1)


def test_plan_compilers_from_two_threads():
    """tile plans, their schedules and recurrent-layer plans built at the same time on different streams equal the ones built
    one after the other"""
    cfgs = [synth.attention_config("C2", seed=s, contents=6 + s) for s in range(4)]

    def build(cfg, window):
        b = cfg.batches[0]
        p = sa.TilePlan.build(b.art, b.end, b.pos, window)
        items, ptr = p.schedule(8)
        sitems, sptr = p.schedule_static(8, 64)
        g = sa.qwen_plan._compile(np.ascontiguousarray(b.prev, np.int64), np.ascontiguousarray(b.art >= 0).view(np.uint8), "indexed", 64, 8192, 96, None, None)
        return [p.qt_ptr, p.kv_idx, p.kv_bits, p.order, items, ptr, sitems, sptr, g["idx"], g["h0_idx"], g["ht_idx"], g["conv"], g["seg_len"]]

    jobs = [(c, w) for c in cfgs for w in (None, 512)]
    serial = [build(c, w) for c, w in jobs]
    for _ in range(3):
        got = [None] * len(jobs)

        def run(i):
            got[i] = build(*jobs[i])

        threads = [threading.Thread(target=run, args=(i,)) for i in range(len(jobs))]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        for a, b in zip(serial, got):
            assert all(np.array_equal(np.asarray(x), np.asarray(y)) for x, y in zip(a, b))


def test_c1_in_fp32_on_the_cpu_against_the_oracle():
    """the CPU baseline leg (fp32 scaled_dot_product_attention under a dense tree mask per content) and torch's eager
    flex_attention under the same rule agree with the float64 oracle to 1e-5 on C1"""
    from torch.nn.attention.flex_attention import create_block_mask, flex_attention

    cfg = synth.attention_config("C1")
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=0, device="cpu")
    q, k, v = q.float(), k.float(), v.float()
    want = oattn.tree_attention(q.numpy(), k.numpy(), v.numpy(), b.art, b.end, b.pos, scale=cfg.scale, spans=oattn.job_spans(b.art))
    _, done, _, _, outs = cpu_baseline.attention_tokens_per_s(q, k, v, b.art, b.end, b.pos, cfg.scale)
    assert done == len(cfg.trees)
    for (a, e), o in outs.items():
        real = b.art[a:e] >= 0
        assert np.abs(o.numpy()[real] - want[a:e][real]).max() <= 1e-5
    art, end = torch.from_numpy(b.art), torch.from_numpy(b.end)

    def rule(_b, _h, qi, ki):   # spinf_serve/scorer.py:173-177
        return ((art[qi] >= 0) & (art[qi] == art[ki]) & (ki <= qi) & (end[ki] > qi)) | (qi == ki)

    n = b.length
    bm = create_block_mask(rule, None, None, n, n, device="cpu", BLOCK_SIZE=128)
    dense = omask.dense_tree_mask(b.art, b.end, b.pos)
    blocks = dense.reshape(n // 128, 128, n // 128, 128).any(axis=(1, 3))   # the oracle's view of which 128 x 128 blocks are live
    assert np.array_equal(bm.to_dense()[0, 0].bool().numpy(), blocks)
    o = flex_attention(q.transpose(0, 1)[None], k.transpose(0, 1)[None], v.transpose(0, 1)[None], block_mask=bm, scale=cfg.scale, enable_gqa=True)
    real = b.art >= 0
    assert np.abs(o[0].transpose(0, 1).numpy()[real] - want[real]).max() <= 1e-5


# ----------------------------------------------------------------------------------------------------------------- GPU

def _np(t):
    return t.float().cpu().numpy()


@pytest.mark.gpu
def test_attention_capture_keeps_the_named_ranges(dev):
    """gemma4.py:100-106: under CAPTURE a global layer keeps the keys / values of each range, a sliding layer their last window - 1"""
    cfg = synth.attention_config("C2", contents=2)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=2, device=dev)
    masks = sa.block_masks(b, sliding_window=64, device=dev)
    config = types.SimpleNamespace(layer_types=["sliding_attention", "full_attention"])
    ranges = [(0, 470, "trunk0"), (b.jobs[1][0], 30, "head1"), (5, 10, "short")]
    args = [t.transpose(0, 1)[None] for t in (q, k, v)]
    plain = [sa.tree_flex_forward(types.SimpleNamespace(config=config, layer_idx=i), *args, masks[config.layer_types[i]], scaling=cfg.scale)[0] for i in range(2)]
    attention.CAPTURE[dev] = {"window": 64, "ranges": ranges, "kv": {}}
    try:
        hooked = [sa.tree_flex_forward(types.SimpleNamespace(config=config, layer_idx=i), *args, masks[config.layer_types[i]], scaling=cfg.scale)[0] for i in range(2)]
        kept = attention.CAPTURE[dev]["kv"]
    finally:
        del attention.CAPTURE[dev]
    assert all(torch.equal(a, c) for a, c in zip(plain, hooked)) and plain[0].shape == (1, b.length, cfg.hq, cfg.d)
    for start, n, name in ranges:
        assert sorted(kept[name]) == [0, 1]
        for layer, first in ((0, start + max(0, n - 63)), (1, start)):
            kk, vv = kept[name][layer]
            assert torch.equal(kk[0], k[first : start + n].transpose(0, 1)) and torch.equal(vv[0], v[first : start + n].transpose(0, 1))
    assert dev not in attention.CAPTURE


@pytest.mark.gpu
@pytest.mark.parametrize("compact", [False, True])
def test_qwen_attention_capture_and_compact_rows(dev, compact):
    """qwen.py:604-623: plan.cap keeps the keys / values of the named row ranges per layer; with sidx the tensors hold the real
    rows only and every real row's output has the stream call's bits"""
    cfg = synth.attention_config("C2", contents=2)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=3, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    stream = sa.tree_attn(q, k, v, mask, cfg.scale)
    sidx = torch.from_numpy(np.flatnonzero(b.art >= 0)).to(dev) if compact else None
    if compact:
        q, k, v = (t[sidx].contiguous() for t in (q, k, v))
    plan = types.SimpleNamespace(cap={"ranges": [(3, 40, "a"), (500, 7, "b")], "out": {"kv": {}}})
    o = sa.tree_attention(*(t.transpose(0, 1)[None] for t in (q, k, v)), mask, cfg.scale, sidx=sidx, plan=plan, mod=types.SimpleNamespace(li=5))
    want = stream[sidx] if compact else stream
    assert torch.equal(o[0].transpose(0, 1), want)
    for r0, n, name in plan.cap["ranges"]:
        kk, vv = plan.cap["out"]["kv"][name][5]
        assert torch.equal(kk[0], k[r0 : r0 + n].transpose(0, 1)) and torch.equal(vv[0], v[r0 : r0 + n].transpose(0, 1))


@pytest.mark.gpu
def test_gdn_capture_keeps_inputs_and_final_states(dev):
    """qwen.py:520-526,558-565: plan.cap keeps the scan inputs of row ranges and the final state of the segment that holds a
    named row; the state equals the oracle's state after that segment's last token"""
    cfg = synth.gdn_config("C5", contents=2)
    b = cfg.batch
    t = synth.gdn_inputs(cfg, seed=4, device=dev)
    trunk_last = [s0 + P - 1 for s0, _, P, _ in b.jobs]
    leaf_row = int(np.flatnonzero(b.seg == 3)[2])                     # a row inside branch 2 of the first content
    leaf_last = int(np.flatnonzero((b.seg == 3) & (b.art == 0))[-1])
    keep = [trunk_last[0], trunk_last[1], leaf_last]
    plan = cfg.plan(dev, keep=keep)
    plain = sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], cfg.plan(dev))
    plan.cap = {"tok": [(10, 20, "rows")], "state": [(5, "trunk0"), (trunk_last[1], "trunk1"), (leaf_row, "leaf")], "out": {"gdn": {}, "state": {}}}
    o = sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], plan, mod=types.SimpleNamespace(li=7))
    torch.cuda.synchronize()
    assert torch.equal(o, plain)
    got = plan.cap["out"]["gdn"]["rows"][7]
    assert all(torch.equal(x, t[n][10:30]) for x, n in zip(got, ("q", "k", "v", "g", "beta")))
    _, states = ogdn.tree_scan(*(_np(t[x]) for x in ("q", "k", "v", "g", "beta")), b.prev, b.art >= 0, keep=keep)
    for name, pos in (("trunk0", trunk_last[0]), ("trunk1", trunk_last[1]), ("leaf", leaf_last)):
        s = _np(plan.cap["out"]["state"][name][7])
        assert s.shape == (cfg.hv, cfg.dk, cfg.dv)
        assert np.abs(s - states[pos]).max() <= 2e-2, name
    plan.cap = {"tok": [], "state": [(int(np.flatnonzero(b.seg == 5)[0]), "unkept")], "out": {"gdn": {}, "state": {}}}
    with pytest.raises(RuntimeError):
        sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], plan, mod=types.SimpleNamespace(li=7))


@pytest.mark.gpu
def test_every_c3_pass(dev):
    """all 13 passes of C3, sliding and global: pad rows come out as their own V row, and the smallest content of each pass
    matches the float64 oracle"""
    cfg = synth.attention_config("C3")
    assert len(cfg.batches) == 13
    for i, b in enumerate(cfg.batches):
        q, k, v = synth.qkv(cfg, b, seed=i, device=dev)
        masks = sa.block_masks(b, sliding_window=cfg.window, device=dev)
        s0, n, _, _ = min(b.jobs, key=lambda j: j[1])
        e0 = s0 + -(-n // 128) * 128
        sub = (q[s0:e0], k[s0:e0], v[s0:e0])
        pad = torch.from_numpy(np.flatnonzero(b.art < 0)).to(dev)
        for name, window in (("sliding_attention", cfg.window), ("full_attention", None)):
            print(f"case C3 pass {i} n={b.length} {name} content at {s0}+{n}", flush=True)
            out = sa.tree_attn(q, k, v, masks[name], cfg.scale)
            assert torch.equal(out[pad], v[pad].repeat_interleave(cfg.hq // cfg.hkv, dim=1))
            want = oattn.tree_attention(*(_np(x) for x in sub), b.art[s0:e0], b.end[s0:e0] - s0, b.pos[s0:e0], window=window, scale=cfg.scale)
            real = b.art[s0:e0] >= 0
            assert np.abs(_np(out[s0:e0])[real] - want[real]).max() <= 2e-2
