"""The attention entry point that allocates nothing (spinf_tree_attn_fwd_noalloc: cursors, counts and redo list in a file-scope
device array) against spinf_tree_attn_fwd, through the C ABI: the same bits, on two calls in a row, the second on a smaller
stream; then a tile that needs the exact pass, and the size limit."""

import ctypes

import numpy as np
import pytest
import torch

import spinf_serve_amd as sa
from spinf_serve_amd import synth

pytestmark = pytest.mark.gpu


def _pair(cfg, b, dev, seed, window=None, scale_keys=None):
    q, k, v = synth.qkv(cfg, b, seed=seed, device=dev)
    if scale_keys is not None:
        k = k.clone()
        k[scale_keys[0]:] *= scale_keys[1]
    mask = sa.TreeMask.build(b.art, b.end, b.pos, window=window, device=dev)
    want = sa.tree_attn(q, k, v, mask, cfg.scale)          # spinf_tree_attn_fwd (uploads the schedule, allocates its output)
    torch.cuda.synchronize()
    got = torch.full_like(want, float("nan"))
    print(f"no-alloc case {cfg.name} n={b.length} hq={cfg.hq} hkv={cfg.hkv} d={cfg.d} window={window}", flush=True)
    sa.tree_attn_noalloc(q, k, v, mask, got, cfg.scale)     # spinf_tree_attn_fwd_noalloc into the caller's tensor
    torch.cuda.synchronize()
    return want, got


def test_noalloc_equals_the_allocating_entry_point_twice_in_a_row(dev):
    big = synth.attention_config("C2", contents=5)
    want, got = _pair(big, big.batches[0], dev, seed=1)
    assert torch.equal(want, got)
    small = synth.attention_config("C2", contents=2)       # the second call: a smaller stream on the same scratch array
    want, got = _pair(small, small.batches[0], dev, seed=2)
    assert torch.equal(want, got)
    want, got = _pair(small, small.batches[0], dev, seed=3, window=200)
    assert torch.equal(want, got)


def test_noalloc_exact_pass_and_other_geometry(dev):
    rng = np.random.default_rng(11)
    trees = [synth._tree(rng, 300, [20, 9]), synth._tree(rng, 90, [7])]
    cfg = synth.AttnConfig("wide", 4, 2, 128, 128 ** -0.5, 1.0, None, trees)
    b = synth.pack(trees)[0]
    total = ctypes.c_int64(0)
    lib = sa.load_library()
    assert lib.spinf_attn_exact_items(ctypes.byref(total)) == 0
    before = total.value
    want, got = _pair(cfg, b, dev, seed=3, scale_keys=(96, 60.0))   # scores far wider than the fast pass allows: redo list in use
    assert torch.equal(want, got)
    assert lib.spinf_attn_exact_items(ctypes.byref(total)) == 0
    assert total.value >= before + 2, "both entry points hand the wide tiles to the exact pass"
    c1 = synth.attention_config("C1")
    want, got = _pair(c1, c1.batches[0], dev, seed=0)
    assert torch.equal(want, got)


def test_noalloc_head_dim_512_one_launch_and_graph_replay(dev):
    """head dim 512 through the entry point that allocates nothing: the kernel with decoupled waves, ONE launch per call (it takes
    no item from a shared list and redoes its wide-range items itself, their indices in the scratch array), so the call can be
    recorded into a graph as it is; replays, with eager calls in between, give the allocating entry point's bits every time"""
    cfg = synth.attention_config("C2_512", contents=3)
    b = cfg.batches[0]
    want, got = _pair(cfg, b, dev, seed=4)
    assert torch.equal(want, got)
    lib = sa.load_library()
    total = ctypes.c_int64(0)
    assert lib.spinf_attn_exact_items(ctypes.byref(total)) == 0
    before = total.value
    want_w, got_w = _pair(cfg, b, dev, seed=4, scale_keys=(200, 50.0))   # wide scores: items redone inside the launch
    assert torch.equal(want_w, got_w)
    assert lib.spinf_attn_exact_items(ctypes.byref(total)) == 0
    assert total.value > before
    q, k, v = synth.qkv(cfg, b, seed=4, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    sa.tree_attn(q, k, v, mask, cfg.scale)     # uploads the schedule of this mask
    torch.cuda.synchronize()
    out = torch.zeros_like(want)
    side = torch.cuda.Stream(device=dev)
    g = torch.cuda.CUDAGraph()
    print("no-alloc case d512 under capture", flush=True)
    with torch.cuda.graph(g, stream=side):
        sa.tree_attn_noalloc(q, k, v, mask, out, cfg.scale)
    for rep in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        again = sa.tree_attn(q, k, v, mask, cfg.scale)   # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(again, want)


@pytest.mark.parametrize("ring", [0, 1])
def test_noalloc_takes_no_device_memory_and_replays_with_cursors_and_wide_scores(dev, ring, monkeypatch):
    """head dim 256 through both kernels (ring 0: the lockstep kernel, whose cursors, counts and redo list are the scratch array's,
    cleared by a kernel in front of the pass; ring 1: the kernel with decoupled waves), on scores wide enough that items go to the
    exact recomputation: the device's free memory and the number of allocations torch has made are the same after the calls as before, and a
    graph that recorded the call replays to the allocating entry point's bits every time, with eager calls of both entry
    points in between"""
    from spinf_serve_amd import attention

    monkeypatch.setattr(attention, "RING", ring)
    cfg = synth.attention_config("C2", contents=3)
    b = cfg.batches[0]
    want, got = _pair(cfg, b, dev, seed=6, scale_keys=(200, 50.0))
    assert torch.equal(want, got)
    q, k, v = synth.qkv(cfg, b, seed=6, device=dev)
    k = k.clone()
    k[200:] *= 50.0
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    assert torch.equal(sa.tree_attn(q, k, v, mask, cfg.scale), want)     # uploads this mask's schedule
    out = torch.zeros_like(want)
    lib = sa.load_library()
    total = ctypes.c_int64(0)
    assert lib.spinf_attn_exact_items(ctypes.byref(total)) == 0          # (synchronises)
    before = total.value
    free0, made0 = torch.cuda.mem_get_info(dev)[0], torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    for _ in range(3):
        sa.tree_attn_noalloc(q, k, v, mask, out, cfg.scale)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free0, "device memory was taken"
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == made0, "torch's allocator was asked for memory"
    assert torch.equal(out, want)
    assert lib.spinf_attn_exact_items(ctypes.byref(total)) == 0
    assert total.value > before, "the wide items went through the exact recomputation"
    side = torch.cuda.Stream(device=dev)
    g = torch.cuda.CUDAGraph()
    print(f"no-alloc case d256 ring={ring} wide scores under capture", flush=True)
    with torch.cuda.graph(g, stream=side):
        sa.tree_attn_noalloc(q, k, v, mask, out, cfg.scale)
    for rep in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), rep
        again = sa.tree_attn(q, k, v, mask, cfg.scale)                     # eager work between the replays, both entry points
        eager = torch.zeros_like(want)
        sa.tree_attn_noalloc(q, k, v, mask, eager, cfg.scale)
        torch.cuda.synchronize()
        assert torch.equal(again, want) and torch.equal(eager, want)


def test_noalloc_rejects_more_items_than_its_array_holds(dev):
    a = sa._lib.AttnArgs()
    one = torch.zeros(8, dtype=torch.int32, device=dev)
    t = torch.zeros((128, 2, 64), dtype=torch.bfloat16, device=dev)
    for f in ("q", "k", "v", "out"):
        setattr(a, f, t.data_ptr())
    for f in ("art", "end", "pos", "kv_idx", "kv_bits", "items", "list_ptr"):
        setattr(a, f, one.data_ptr())
    a.q_tok = a.k_tok = a.v_tok = a.o_tok = 128
    a.q_head = a.k_head = a.v_head = a.o_head = 64
    a.n, a.hq, a.hkv, a.d, a.scale = 128, 2, 2, 64, 0.125
    a.n_items = 65537
    lib = sa.load_library()
    assert lib.spinf_tree_attn_fwd_noalloc(ctypes.byref(a), None) == -1
    assert b"at most" in lib.spinf_last_error()
