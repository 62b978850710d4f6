"""Host side of the path (no GPU): the stream layout, the tile-plan compiler (C ABI, host code), the recurrent-layer planner,
and that the shared library loads and exports every symbol include/spinf_tree.h declares."""

import ctypes
import gzip
import json
import os
import re

import numpy as np
import pytest

import spinf_serve_amd as sa
from oracle import mask as omask
from oracle import plan as oplan
from oracle.layout import Job, pack_stream
from spinf_serve_amd import synth
from spinf_serve_amd import layout as lay
from spinf_serve_amd.layout import TokenTree

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


@pytest.fixture(scope="module")
def golden():
    with gzip.open(os.path.join(HERE, "golden", "packer_golden.json.gz"), "rt") as f:
        return json.load(f)


# ------------------------------------------------------------------------------------------------ C ABI
def test_library_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "spinf_tree.h")).read()
    declared = set(re.findall(r"\b(spinf_[a-z0-9_]+)\s*\(", header))
    assert {"spinf_tileplan_build", "spinf_tree_attn_fwd", "spinf_gdn_fwd", "spinf_last_error"} <= declared
    raw = ctypes.CDLL(sa.library_path())
    for name in declared:
        assert hasattr(raw, name), name
    assert lib.spinf_version() >= 1


def test_c_abi_rejects_bad_arguments(lib):
    out = ctypes.c_void_p()
    assert lib.spinf_tileplan_build(None, None, None, 5, 0, ctypes.byref(out)) == -1
    assert b"null" in lib.spinf_last_error()
    assert lib.spinf_tileplan_build(None, None, None, 0, 0, None) == -1
    assert lib.spinf_tree_attn_fwd(None, None) == -1 and lib.spinf_gdn_fwd(None, None) == -1
    # an empty stream is a valid (empty) plan
    assert lib.spinf_tileplan_build(None, None, None, 0, 0, ctypes.byref(out)) == 0
    counts = (ctypes.c_int64 * 5)()
    assert lib.spinf_tileplan_counts(out, counts) == 0 and list(counts) == [0, 0, 0, 0, 0]
    lib.spinf_tileplan_free(out)
    # the yardsticks check their arguments before they touch the GPU
    buf = (ctypes.c_int64 * 32)()
    assert lib.spinf_diag_mfma_valu(3, 0, 2, 100, buf, None) == -1 and b"nv 3" in lib.spinf_last_error()
    assert lib.spinf_diag_mfma_valu(4, 3, 2, 100, buf, None) == -1 and b"kind 3" in lib.spinf_last_error()
    assert lib.spinf_diag_mfma_valu(4, 0, 3, 100, buf, None) == -1 and b"waves per SIMD" in lib.spinf_last_error()
    assert lib.spinf_diag_mfma_valu(4, 0, 2, 100, None, None) == -1


def test_heads_per_item_follows_the_kernel_choice(lib):
    """even GQA groups share an item between the heads of a pair (variant 0: across waves; variant 2: inside a wave, head
    dim <= 128 only); odd groups, MHA and variant 1 run one head per item; the schedule must be built for this count"""
    f = lib.spinf_attn_heads_per_item
    for d in (64, 128, 256):
        assert f(16, 8, d, 0) == 2 and f(8, 2, d, 0) == 2 and f(8, 1, d, 0) == 2
        assert f(6, 2, d, 0) == 1 and f(4, 4, d, 0) == 1 and f(3, 1, d, 0) == 1
        assert f(16, 8, d, 1) == 1
        assert f(16, 8, d, 2) == (2 if d <= 128 else 1)
        assert f(16, 8, d, 3) == 2 and f(6, 2, d, 3) == 1     # (variant 3, the decoupled kernel at head dim 128: items as for variant 0)
    assert f(0, 1, 128, 0) == 0 and f(5, 2, 128, 0) == 0      # not a head geometry


def test_gdn_argument_checks_come_before_any_launch(lib):
    """spinf_gdn_fwd validates shapes, strides and alignment on the host and reports what it rejects"""
    from spinf_serve_amd import _lib as L

    def args(**kw):
        a = L.GdnArgs()
        for name in ("q", "k", "v", "g", "beta", "o", "cu"):
            setattr(a, name, 0x1000)      # never dereferenced: every case below is rejected first
        a.q_tok, a.v_tok, a.g_tok, a.o_tok = 2048, 4096, 32, 4096
        a.h, a.hv, a.dk, a.dv, a.scale = 16, 32, 128, 128, 0.088
        a.n_seg, a.max_len, a.mode = 1, 0, 0
        for k_, v_ in kw.items():
            setattr(a, k_, v_)
        return a

    for kw, word in ((dict(dk=64), b"key head dim"), (dict(dv=48), b"value head dim"), (dict(hv=30), b"multiple of h"),
                     (dict(q_tok=2044), b"q/k row stride"), (dict(v_tok=4100), b"v/o row stride"), (dict(o_tok=1 << 31), b"below 2^31"),
                     (dict(mode=7), b"unknown mode")):
        assert lib.spinf_gdn_fwd(ctypes.byref(args(**kw)), None) == -1, kw
        assert word in lib.spinf_last_error(), (kw, lib.spinf_last_error())
    assert lib.spinf_gdn_fwd(ctypes.byref(args(n_seg=0)), None) == 0      # nothing to do is not an error


def test_missing_library_fails_loudly(monkeypatch):
    from spinf_serve_amd import _lib

    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setenv("SPINF_TREE_LIB", "/nonexistent/libspinf_tree.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load_library()


def test_ops_have_no_cpu_path(lib):
    import torch

    cfg = synth.attention_config("C1")
    b = cfg.batches[0]
    q = torch.zeros((b.length, cfg.hq, cfg.d), dtype=torch.bfloat16)
    k = torch.zeros((b.length, cfg.hkv, cfg.d), dtype=torch.bfloat16)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device="cpu")
    with pytest.raises(RuntimeError, match="ROCm"):
        sa.tree_attn(q, k, k, mask, cfg.scale)


@pytest.mark.parametrize("entry", ["tree_attn", "tree_attn_noalloc"])
def test_both_attention_entry_points_check_their_tensors_before_any_launch(lib, entry):
    """one shared check in front of spinf_tree_attn_fwd and spinf_tree_attn_fwd_noalloc: a wrong dtype, shape, head grouping,
    stride or row count raises ValueError on the host (the kernels index by these and would read out of bounds)"""
    import torch

    from spinf_serve_amd import attention

    cfg = synth.attention_config("C1")
    b = cfg.batches[0]
    n, hq, hkv, d = b.length, cfg.hq, cfg.hkv, cfg.d
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device="cpu")

    def call(q, k, v, out=None):
        if entry == "tree_attn":
            return sa.tree_attn(q, k, v, mask, cfg.scale)
        return attention.tree_attn_noalloc(q, k, v, mask, torch.empty_like(q) if out is None else out, cfg.scale)

    def z(rows, heads, dim, dtype=torch.bfloat16):
        return torch.zeros((rows, heads, dim), dtype=dtype)

    q, k = z(n, hq, d), z(n, hkv, d)
    with pytest.raises(ValueError, match="bf16"):
        call(z(n, hq, d, torch.float16), k, k)
    with pytest.raises(ValueError, match="bf16"):
        call(q, k, z(n, hkv, d, torch.float32))
    with pytest.raises(ValueError, match="heads, head dim"):
        call(q.reshape(n, hq * d), k, k)
    with pytest.raises(ValueError, match="do not match"):
        call(q, z(n - 1, hkv, d), k)
    with pytest.raises(ValueError, match="do not match"):
        call(q, k, z(n, hkv, d // 2))
    with pytest.raises(ValueError, match="do not match"):
        call(q, k, z(n, hkv + 1, d))
    with pytest.raises(ValueError, match="do not group"):
        call(z(n, 3, d), z(n, 2, d), z(n, 2, d))
    with pytest.raises(ValueError, match="contiguous"):
        call(z(n, hq, 2 * d)[:, :, ::2], k, k)
    with pytest.raises(ValueError, match="mask describes"):
        call(z(n + 64, hq, d), z(n + 64, hkv, d), z(n + 64, hkv, d))
    with pytest.raises(TypeError, match="TreeMask"):
        (sa.tree_attn if entry == "tree_attn" else attention.tree_attn_noalloc)(q, k, k, None, *(() if entry == "tree_attn" else (q,)))
    if entry == "tree_attn_noalloc":
        with pytest.raises(ValueError, match="out must be"):
            call(q, k, k, out=z(n, hq, d, torch.float32))
        with pytest.raises(ValueError, match="out must be"):
            call(q, k, k, out=z(n + 1, hq, d))
        with pytest.raises(ValueError, match="out must be"):
            call(q, k, k, out=z(n, 2 * hq, d)[:, ::2])
    with pytest.raises(RuntimeError, match="ROCm"):   # everything in order except the device: still no CPU path
        call(q, k, k)


def test_build_scan_of_the_ring_assembly_catches_what_it_is_there_for():
    """the scan build() runs over tree_attn_ring.s, on hand-made listings: a vector write of an MFMA operand in the issue cycle
    before an assembly MFMA (a wait on a memory counter in between does not count), a compiler-owned accumulation register,
    too many spills; and what it must let pass"""
    import __graft_entry__ as ge

    def listing(*body):
        return ["_Zkernel:", *("\t" + b for b in body)]

    mfma = ["\t;;#ASMSTART", "\tv_mfma_f32_32x32x16_bf16 a[0:15], v[0:3], v[4:7], a[0:15]", "\t;;#ASMEND"]
    ge._scan_ring_assembly(listing("v_cvt_pk_bf16_f32 v7, v14, v15", "ds_read_b64_tr_b16 v[0:1], v89") + mfma)
    ge._scan_ring_assembly(listing("v_cvt_pk_bf16_f32 v7, v14, v15", "s_nop 0") + mfma)
    ge._scan_ring_assembly(listing("v_cvt_pk_bf16_f32 v8, v14, v15", "s_waitcnt lgkmcnt(0)") + mfma)
    ge._scan_ring_assembly(listing("v_cvt_pk_bf16_f32 v7, v14, v15") + [".LBB0_1:"] + mfma)   # (a branch target: the writer is not the predecessor)
    with pytest.raises(RuntimeError, match="issue cycle before"):
        ge._scan_ring_assembly(listing("v_cvt_pk_bf16_f32 v7, v14, v15", "s_waitcnt lgkmcnt(0)") + mfma)
    with pytest.raises(RuntimeError, match="issue cycle before"):
        ge._scan_ring_assembly(listing("v_mov_b32_e32 v2, v9") + mfma)
    with pytest.raises(RuntimeError, match="accumulation register that the assembly owns"):
        ge._scan_ring_assembly(listing("v_accvgpr_write_b32 a130, v3"))
    k128 = "_ZN12_GLOBAL__N_121tree_attn_ring_kernelILi128ELb0EEEv10AttnParams: ; @kernel"
    ge._scan_ring_assembly([k128, "\tv_accvgpr_write_b32 a66, v3"])        # head dim 128: the assembly owns a[0:63] only
    with pytest.raises(RuntimeError, match="accumulation register that the assembly owns"):
        ge._scan_ring_assembly([k128, "\tv_accvgpr_read_b32 v3, a63"])
    reload = ["_ZN12_GLOBAL__N_121tree_attn_ring_kernelILi256ELb0EEEv10AttnParams: ; @kernel", ".LBB0_7:    ;   in Loop: Header=BB0_3 Depth=2",
              "\tscratch_load_dwordx4 v[4:7], off, off offset:16"]
    with pytest.raises(RuntimeError, match="16-byte reload"):
        ge._scan_ring_assembly(reload)
    ge._scan_ring_assembly([reload[0], ".LBB0_7:", reload[2]])                                  # outside any loop: tolerated
    ge._scan_ring_assembly([reload[0], reload[1], "\tscratch_load_dword v4, off, off offset:16"])   # a single register: tolerated
    meta = ["    .name:           _ZN12_GLOBAL__N_121tree_attn_ring_kernelILi256ELb0EEEv10AttnParams", "    .vgpr_spill_count: 16"]
    with pytest.raises(RuntimeError, match="spills 16"):
        ge._scan_ring_assembly(meta)
    ge._scan_ring_assembly([meta[0], "    .vgpr_spill_count: 2"])


# ------------------------------------------------------------------------------------------------ stream layout
def _golden_trees(case):
    return [TokenTree(t["prefix"], t["branches"], list(t["parents"]), tuple(t["aligned"])) for t in case["trees"]]


def test_layout_reproduces_reference_streams(golden):
    """the jobs the reference's packer put into a stream (its owners say which, in which order), laid out by pack_stream: the same
    ids / pos / seg / art / end / prev, field by field (Packer._pack, spinf_serve/packer.py:352-423)"""
    for case in golden["cases"]:
        trees = _golden_trees(case)
        for want in case["batches"]:
            members = [trees[job_id] for job_id, *_ in want["owners"]]
            b = lay.pack_stream(members, align=case["align"], length=len(want["ids"]))
            for key in ("ids", "pos", "seg", "art", "end", "prev"):
                assert getattr(b, key).tolist() == want[key], key
            assert b.n_tokens == want["n_tokens"]
            assert [[s0, n, P] for s0, n, P, _ in b.jobs] == [o[1:] for o in want["owners"]]


def test_layout_literals_and_invariants():
    # two-level tree (spinf_serve/packer.py:382-408): depth on the path, subtree ends, the path predecessor
    t = TokenTree([1, 2], [[5, 6, 7], [8], [9], [4, 21]], [-1, 0, 0, -1])
    b = lay.pack_stream([t], align=True)
    assert b.length == 128 and b.n_tokens == 9 and t.n_tokens == 9
    assert b.pos[:9].tolist() == [0, 1, 2, 3, 4, 5, 5, 2, 3] and b.seg[:9].tolist() == [0, 0, 1, 1, 1, 2, 3, 4, 4]
    assert b.end[:9].tolist() == [9, 9, 7, 7, 7, 6, 7, 9, 9] and b.prev[:9].tolist() == [-1, 0, 1, 2, 3, 4, 4, 1, 7]
    assert (b.art[9:] == -1).all() and (b.end[9:] == -1).all() and (b.prev[9:] == -1).all() and (b.pos[9:] == 0).all()
    # aligned branches start on a block boundary relative to the job, the gap is padding (packer.py:390-391)
    t = TokenTree(list(range(100)), [[1] * 10, [2] * 10], [-1, -1], aligned=(1,))
    b = lay.pack_stream([TokenTree([7] * 130, []), t], align=True)
    assert t.n_tokens == 138 and b.jobs == [(0, 130, 130, 0), (256, 138, 100, 1)]
    assert (b.art[256 + 110 : 256 + 128] == -1).all() and b.seg[256 + 128] == 2 and b.prev[256 + 128] == 256 + 99
    # unaligned packing, stream length, a job that does not fit
    b = lay.pack_stream([TokenTree([7] * 130, []), t], align=False, min_stream=512)
    assert b.length == 512 and b.jobs[1][0] == 130
    with pytest.raises(ValueError):
        lay.pack_stream([t], length=128)
    with pytest.raises(ValueError):
        TokenTree([1], [[2], [3]], [1, -1])
    # first-fit-decreasing streams: every job once, none over the budget
    rng = np.random.default_rng(3)
    trees = [TokenTree(rng.integers(1, 9, int(n)).tolist(), [[1, 2]]) for n in rng.integers(50, 900, 40)]
    streams = lay.pack_streams(trees, 2048)
    assert sorted(k for s in streams for *_, k in s.jobs) == list(range(40)) and all(s.length <= 2048 for s in streams)
    with pytest.raises(ValueError):
        lay.pack_streams([TokenTree([1] * 3000, [])], 2048)


def test_every_token_sees_exactly_its_path():
    """the invariant behind tests/test_packer.py:209-239: under the mask rule a token sees one token per position 0 .. pos, and they
    spell its root-to-leaf path"""
    rng = np.random.default_rng(0)
    for _ in range(10):
        nb = int(rng.integers(1, 9))
        parents = []
        for b in range(nb):   # pre-order: a branch hangs on the trunk, on the branch before it or on one of that branch's ancestors
            chain, a = [-1], b - 1
            while a >= 0:
                chain.append(a)
                a = parents[a]
            parents.append(int(rng.choice(chain)))
        t = TokenTree(rng.integers(2, 6, 4).tolist(), [rng.integers(2, 9, int(rng.integers(1, 6))).tolist() for _ in range(nb)], parents)
        b = lay.pack_stream([TokenTree([1, 7, 7, 2], [[9], [3, 9]]), t], align=bool(rng.integers(0, 2)))
        m = omask.dense_tree_mask(b.art, b.end)
        for q in np.flatnonzero(b.art >= 0):
            ks = np.flatnonzero(m[q])
            assert b.pos[ks].tolist() == list(range(b.pos[q] + 1))
            path, i = [], int(q)
            while i >= 0:
                path.append(i)
                i = int(b.prev[i])
            assert path[::-1] == ks.tolist()


# ------------------------------------------------------------------------------------------------ tile plan
def _check_plan(art, end, pos, window, grp=None, grp_windowed=False):
    """exactness of the compiled plan against the dense mask at 32 x 32 granularity: a set bit <=> some pair visible,
    a clear mask bit <=> every pair visible, unlisted tiles <=> nothing visible; key tiles ascending"""
    plan = sa.TilePlan.build(art, end, pos, window, grp, grp_windowed)
    n = len(art)
    m = omask.dense_tree_mask(art, end, pos, window, grp, grp_windowed)
    nqt = -(-n // 128)
    assert plan.n_qtiles == nqt and sorted(plan.order.tolist()) == list(range(nqt))
    active = masked = 0
    for t in range(nqt):
        ents = range(plan.qt_ptr[t], plan.qt_ptr[t + 1])
        kts = [int(plan.kv_idx[e]) for e in ents]
        assert kts == sorted(set(kts))
        listed = dict(zip(kts, (int(plan.kv_bits[e]) for e in ents)))
        for j in range(-(-n // 64)):
            bits = listed.get(j, 0)
            for w in range(4):
                for s in range(2):
                    blk = m[128 * t + 32 * w : 128 * t + 32 * w + 32, 64 * j + 32 * s : 64 * j + 32 * s + 32]
                    on = bool(bits >> (2 * w + s) & 1)
                    assert on == bool(blk.size and blk.any()), (t, j, w, s)
                    if on:
                        active += 1
                        need = bool(bits >> (8 + 2 * w + s) & 1)
                        assert need == (not (blk.all() and blk.shape == (32, 32))), (t, j, w, s)
                        masked += need
                    else:
                        assert not (bits >> (8 + 2 * w + s) & 1)
    assert (active, masked) == (plan.active_blocks, plan.masked_blocks)
    return plan


def _image_stream(seed=8):
    """two jobs with image placeholders: groups that straddle tile borders, two in one block, one in a branch"""
    rng = np.random.default_rng(seed)
    t1 = TokenTree(rng.integers(5, 99, 700).tolist(), [rng.integers(5, 99, n).tolist() for n in (40, 9, 70)], [-1, -1, -1])
    t2 = synth._tree(rng, 150, [20])
    b = synth.pack([t1, t2])[0]
    grp = np.full(b.length, -1, np.int32)
    for gid, (a, e) in enumerate([(10, 22), (24, 30), (100, 356), (500, 530), (705, 735), (768 + 128 + 5, 768 + 128 + 40)]):
        grp[a:e] = gid
    grp[b.art < 0] = -1
    return b, grp


def test_image_group_mask_literal():
    """scorer.py:184-198 on six tokens of one job, tokens 2..4 one image: they see each other both ways, the rest stays causal"""
    art, end = np.zeros(6, np.int32), np.full(6, 6, np.int32)
    grp = np.array([-1, -1, 0, 0, 0, -1], np.int32)
    want = np.array([[1, 0, 0, 0, 0, 0],
                     [1, 1, 0, 0, 0, 0],
                     [1, 1, 1, 1, 1, 0],
                     [1, 1, 1, 1, 1, 0],
                     [1, 1, 1, 1, 1, 0],
                     [1, 1, 1, 1, 1, 1]], bool)
    assert np.array_equal(omask.dense_tree_mask(art, end, grp=grp), want)
    pos = np.arange(6)
    # window 2, group term not windowed: the image still sees itself whole; windowed: only neighbours at distance < 2
    w_all = omask.dense_tree_mask(art, end, pos, 2, grp)
    assert w_all[2].tolist() == [0, 1, 1, 1, 1, 0] and w_all[4].tolist() == [0, 0, 1, 1, 1, 0] and w_all[5].tolist() == [0, 0, 0, 0, 1, 1]
    w_win = omask.dense_tree_mask(art, end, pos, 2, grp, grp_windowed=True)
    assert w_win[2].tolist() == [0, 1, 1, 1, 1, 0] and w_win[4].tolist() == [0, 0, 0, 1, 1, 0]   # later keys: pos[q] - pos[k] < 0 < W


def test_tileplan_with_image_groups_is_exact():
    b, grp = _image_stream()
    for window, windowed in ((None, False), (64, False), (64, True), (300, True)):
        plan = _check_plan(b.art, b.end, b.pos, window, grp, windowed)
    # a query tile lists the LATER key tiles of its images (packer.py:456-468)
    plan = sa.TilePlan.build(b.art, b.end, b.pos, None, grp)
    kts = plan.kv_idx[plan.qt_ptr[0] : plan.qt_ptr[1]].tolist()      # tile 0 holds the start of the image at 100 .. 355
    assert kts == [0, 1, 2, 3, 4, 5]
    # without groups the same stream lists nothing after the diagonal
    plain = sa.TilePlan.build(b.art, b.end, b.pos, None)
    assert plain.kv_idx[plain.qt_ptr[0] : plain.qt_ptr[1]].tolist() == [0, 1]


def test_tileplan_is_exact_on_golden_streams(golden):
    for case in golden["cases"]:
        for b in case["batches"]:
            art, end, pos = (np.array(b[k], np.int32) for k in ("art", "end", "pos"))
            _check_plan(art, end, pos, None)
            _check_plan(art, end, pos, b["window"])


def test_tileplan_edge_cases():
    # all pads; a single token; ragged length; dense (unaligned) packing with jobs sharing tiles
    _check_plan(np.full(130, -1, np.int32), np.full(130, -1, np.int32), np.zeros(130, np.int32), None)
    _check_plan(np.zeros(1, np.int32), np.ones(1, np.int32), np.zeros(1, np.int32), None)
    s = pack_stream([Job([1] * 100, [[2] * 5, [3] * 6]), Job([4] * 37, [[5] * 3]), Job([6] * 260, [[7] * 11] * 6)], align=False)
    n = int(np.flatnonzero(s.art >= 0)[-1]) + 1
    _check_plan(s.art[:n], np.minimum(s.end[:n], n), s.pos[:n], None)
    _check_plan(s.art[:n], np.minimum(s.end[:n], n), s.pos[:n], 50)
    # the reference's literal: 2000-token trunk at window 512, query block 14 needs exactly key blocks 10..14
    s = pack_stream([Job([1] * 2000, [[2]])], length=2048)
    plan = sa.TilePlan.build(s.art, s.end, s.pos, 512)
    assert sorted({int(k) // 2 for k in plan.kv_idx[plan.qt_ptr[14] : plan.qt_ptr[15]]}) == [10, 11, 12, 13, 14]
    # finished sibling branches are skipped (tests/test_packer.py:251-259)
    s = pack_stream([Job([1] * 200, [[2] * 300, [3] * 300])], length=1024)
    plan = sa.TilePlan.build(s.art, s.end, s.pos, None)
    blocks = {int(k) // 2 for k in plan.kv_idx[plan.qt_ptr[5] : plan.qt_ptr[6]]}
    assert 2 not in blocks and {0, 1, 3, 4, 5} <= blocks


def test_schedule_covers_every_tile_and_head_group_once():
    """the kernel's work lists: every (query tile, head group) appears in exactly one list, with its own entry range and
    first key tile; lists are contiguous and ordered job by job (items of one job and head group are neighbours, so that
    the workgroups that take them share K/V in one L2)"""
    cfg = synth.attention_config("C2", contents=5)
    b = cfg.batches[0]
    plan = sa.TilePlan.build(b.art, b.end, b.pos, None)
    for head_groups in (1, 3, 16):
        items, list_ptr = plan.schedule(head_groups)
        assert items.shape == (plan.n_qtiles * head_groups, 4)
        assert list_ptr[0] == 0 and list_ptr[8] == len(items) and (np.diff(list_ptr) >= 0).all()
        seen = set()
        for t, e0, z, kt0 in items.tolist():
            ne, hp = z & 0xFFFFF, (z & 0xFFFFFFFF) >> 20
            assert 0 <= t < plan.n_qtiles and 0 <= hp < head_groups and (t, hp) not in seen
            seen.add((t, hp))
            assert e0 == plan.qt_ptr[t] and ne == plan.qt_ptr[t + 1] - plan.qt_ptr[t] and ne >= 1
            assert kt0 == plan.kv_idx[e0]
        assert len(seen) == plan.n_qtiles * head_groups
        # a list is a body followed by a tail.  Body: the items of one (job, head group) are contiguous (they share keys).
        # Tail: the list's lightest items, at most 128 of them, heaviest first, so that the workgroups finish close together.
        job_of_tile = {}
        for start, length, _, k in b.jobs:
            for t in range(start // 128, -(-(start + length) // 128)):
                job_of_tile[t] = k
        for l in range(8):
            rows = items[list_ptr[l] : list_ptr[l + 1]].tolist()
            # cost of an item: per key tile, the most 32-key blocks any of the four row groups sees (they move in step)
            blocks = [sum(max(bin((int(x) >> (2 * w)) & 3).count("1") for w in range(4)) for x in plan.kv_bits[e0 : e0 + (z & 0xFFFFF)])
                      for _, e0, z, _ in rows]
            cut = len(rows)
            while cut > 0 and len(rows) - cut < 128 and (cut == len(rows) or blocks[cut - 1] >= blocks[cut]):
                cut -= 1
            runs = [(job_of_tile.get(t, -1), ((z & 0xFFFFFFFF) >> 20)) for t, _, z, _ in rows[:cut]]
            compact = [r for i, r in enumerate(runs) if i == 0 or r != runs[i - 1]]
            assert len(compact) == len(set(compact))


def test_row_map_of_a_plan_names_the_tiles_that_are_consecutive_rows():
    """spinf_tileplan_row0: per plan entry, the compact row of the tile's first key where its 64 keys are 64 consecutive rows"""
    import ctypes as C

    rng = np.random.default_rng(5)
    t = TokenTree(rng.integers(5, 99, 300).tolist(), [rng.integers(5, 99, n).tolist() for n in (9, 12, 7, 30)], [-1, -1, -1, -1], aligned=(2,))
    trees = [t, synth._tree(rng, 200, [20, 9]), synth._tree(rng, 64, [])]
    b = synth.pack(trees)[0]
    plan = sa.TilePlan.build(b.art, b.end, b.pos, None)
    real = np.flatnonzero(b.art >= 0)
    row_of = np.full(b.length, -1, np.int32)
    row_of[real] = np.arange(len(real), dtype=np.int32)
    got = np.full(len(plan.kv_idx), -7, np.int32)
    lib = sa.load_library()
    assert lib.spinf_tileplan_row0(plan._handle, row_of.ctypes.data_as(C.c_void_p), got.ctypes.data_as(C.c_void_p)) == 0
    want = []
    for kt in plan.kv_idx.tolist():
        r = row_of[kt * 64 : kt * 64 + 64]
        want.append(int(r[0]) if len(r) == 64 and r[0] >= 0 and (r == r[0] + np.arange(64)).all() else -1)
    assert got.tolist() == want
    assert -1 in want and max(want) > 0            # the case has both kinds of tile
    # the mask's own (torch) construction of the two arrays agrees
    import torch

    mask = sa.TreeMask(plan, tuple(torch.from_numpy(np.ascontiguousarray(x)) for x in (b.art, b.end, b.pos)), torch.device("cpu"))
    r_of, r0 = mask.rows(torch.from_numpy(real))
    assert r_of.tolist() == row_of.tolist() and r0.tolist() == want


def test_a_jobs_plan_does_not_depend_on_its_neighbours():
    """aligned jobs: a job's tile lists, relative to its first tile, are the same alone and packed (the host half of batch
    invariance, tests/test_packer.py:115-134)"""
    cfg = synth.attention_config("C2", contents=3)

    def rel(trees, which, window):
        b = synth.pack(trees)[0]
        plan = sa.TilePlan.build(b.art, b.end, b.pos, window)
        start, length, *_ = b.jobs[which]
        t0, t1 = start // 128, -(-(start + length) // 128)
        return [[(int(plan.kv_idx[e]) - 2 * t0, int(plan.kv_bits[e])) for e in range(plan.qt_ptr[t], plan.qt_ptr[t + 1])] for t in range(t0, t1)]

    for window in (None, 256):
        for i, t in enumerate(cfg.trees):
            assert rel([t], 0, window) == rel(cfg.trees, i, window) == rel(cfg.trees[::-1], 2 - i, window)


def test_config_workloads_match_their_closed_forms():
    c1 = synth.attention_config("C1")
    assert (c1.n_real, c1.pairs(), c1.flops()) == (192, 8544, 8749056.0) and c1.batches[0].length == 256
    # P = T(T+1)/2 + sum_b (L_b * ancestors + L_b (L_b + 1) / 2), here against the dense mask
    c2 = synth.attention_config("C2", contents=2)
    b = c2.batches[0]
    m = omask.dense_tree_mask(b.art, b.end)
    assert c2.pairs() == int(m[b.art >= 0].sum())
    assert c2.pairs(100) == int(omask.dense_tree_mask(b.art, b.end, b.pos, 100)[b.art >= 0].sum())


# ------------------------------------------------------------------------------------------------ recurrent-layer plan
def test_tree_plan_matches_reference_and_oracle(golden):
    for case in golden["cases"]:
        for b in case["batches"]:
            prev, real = np.array(b["prev"]), np.array(b["art"]) >= 0
            for short, ct in ((64, 8192), (4, 300)):
                want = b[f"plan_short{short}_ct{ct}"]
                plan = sa.tree_plan(prev, real, "cpu", path="indexed", short=short, call_tokens=ct)
                assert plan.n_keep == want["n_keep"] and plan.n_segments == want["n_segments"]
                assert plan.conv.tolist() == want["conv"]
                for lv, wl in zip(plan.levels, want["levels"]):
                    assert len(lv) == len(wl)
                    for c, wc in zip(lv, wl):
                        assert c.kind == wc["kind"] and c.idx.tolist() == wc["idx"] and c.cu.tolist() == wc["cu"]
                        assert (None if c.h0_idx is None else c.h0_idx.tolist()) == wc["h0_idx"]
                        assert (None if c.ht_idx is None else c.ht_idx.tolist()) == wc["ht_idx"]


def test_tree_plan_compact_rows_keep_and_levels():
    """tests/test_qwen_plan.py:102-164 and tests/test_stacks.py:67-75 against the mirror"""
    plan = sa.tree_plan(np.array([-1, 0, 1, 1, 3]), np.ones(5, bool), "cpu")
    assert plan.n_segments == 3
    rng = np.random.default_rng(1)
    job = Job(list(rng.integers(5, 50, 150)), [list(rng.integers(5, 50, n)) for n in (6, 70, 3, 2, 9)], [-1, 0, 0, 2, -1])
    s = pack_stream([job, Job([9] * 5, [[1], [2]])], align=True)
    real = s.art >= 0
    R = int(real.sum())
    rows = (R + 127) // 128 * 128
    cp = sa.tree_plan(s.prev, real, "cpu", short=4, rows=rows)
    ip = sa.tree_plan(s.prev, real, "cpu", short=4)
    sidx = cp.sidx.numpy()
    assert (sidx == np.flatnonzero(real)).all()
    for lc, ls in zip(cp.levels, ip.levels):
        for c, d in zip(lc, ls):
            assert (sidx[c.idx.numpy()] == d.idx.numpy()).all() and (c.cu.numpy() == d.cu.numpy()).all()
    T = len(s.prev)
    back = np.full(rows + 1, T, np.int64)
    back[:R] = sidx
    assert (back[cp.conv.numpy()[:R]] == ip.conv.numpy()[sidx]).all() and (cp.conv.numpy()[R:] == rows).all()
    assert (cp.seg_of_row[R:] == -1).all() and (cp.seg_of_row[:R] >= 0).all()
    # a leaf keeps no state unless asked to
    leaf = [i for i in np.flatnonzero(real) if not (s.prev == i).any()][0]
    c_of = np.cumsum(real) - 1
    sg = cp.seg_of_row[c_of[leaf]]
    assert cp.seg_slot[sg] == -1
    kept = sa.tree_plan(s.prev, real, "cpu", short=4, rows=rows, keep=[leaf])
    assert kept.seg_slot[sg] >= 0 and kept.n_keep[kept.seg_level[sg]] == cp.n_keep[cp.seg_level[sg]] + 1
    # the levels path covers every real token once
    lp = sa.tree_plan(s.prev, real, "cpu", max_init=3, path="levels")
    seen = np.concatenate([c.idx.numpy() for lv in lp.levels for c in lv])
    assert sorted(seen.tolist()) == np.flatnonzero(real).tolist()
    with pytest.raises(ValueError):
        sa.tree_plan(s.prev, real, "cpu", rows=R - 1)
    # the oracle's restatement agrees
    levels, n_keep, _ = oplan.tree_plan(s.prev, real, short=4)
    assert n_keep == ip.n_keep and [[c["kind"] for c in lv] for lv in levels] == [[c.kind for c in lv] for lv in ip.levels]


def test_tileplan_is_exact_on_random_forests():
    """random forests (two-level trees, aligned branch groups, dense or aligned packing, with and without a window, image groups
    and 32-key entries): the compiled plan equals the dense mask block by block"""
    from hypothesis import given, settings
    from hypothesis import strategies as st

    @settings(max_examples=30, deadline=None, derandomize=True)
    @given(st.integers(0, 2 ** 31 - 1))
    def run(seed):
        rng = np.random.default_rng(seed)
        trees = []
        for _ in range(int(rng.integers(1, 4))):
            nb = int(rng.integers(0, 6))
            lens = [int(x) for x in rng.integers(1, 40, nb)]
            parents = [-1 if i == 0 or rng.random() < 0.5 else int(rng.integers(0, i)) for i in range(nb)]
            parents = [p if p < 0 or parents[p] < 0 else -1 for p in parents]          # at most two levels, parents first
            aligned = [i for i in range(nb) if parents[i] < 0 and rng.random() < 0.2]
            trunk = int(rng.integers(0 if nb else 1, 300))
            trees.append(TokenTree(rng.integers(5, 99, trunk).tolist(), [rng.integers(5, 99, n).tolist() for n in lens], parents, tuple(aligned)))
        b = synth.pack(trees, align=bool(rng.integers(0, 2)))[0]
        window = [None, 17, 100][int(rng.integers(0, 3))]
        grp = None
        if rng.random() < 0.5:
            grp = np.full(b.length, -1, np.int32)
            for gid in range(int(rng.integers(1, 4))):
                a = int(rng.integers(0, b.length))
                grp[a : a + int(rng.integers(1, 90))] = gid
            grp[b.art < 0] = -1
        windowed = bool(rng.integers(0, 2)) and window is not None
        _check_plan(b.art, b.end, b.pos, window, grp, windowed)
        # 32-key entries: the same blocks, one sub-tile per entry
        p64 = sa.TilePlan.build(b.art, b.end, b.pos, window, grp, windowed)
        p32 = sa.TilePlan.build(b.art, b.end, b.pos, window, grp, windowed, ktile=32)
        assert (p32.active_blocks, p32.masked_blocks) == (p64.active_blocks, p64.masked_blocks)
        assert not (p32.kv_bits & np.uint32(0xAAAA)).any()                              # only sub-tile 0 of an entry
        for t in range(p64.n_qtiles):
            want = set()
            for e in range(p64.qt_ptr[t], p64.qt_ptr[t + 1]):
                for s_ in range(2):
                    if int(p64.kv_bits[e]) & (0x55 << s_):
                        want.add((2 * int(p64.kv_idx[e]) + s_, (int(p64.kv_bits[e]) >> s_) & 0x5555))
            got = {(int(p32.kv_idx[e]), int(p32.kv_bits[e])) for e in range(p32.qt_ptr[t], p32.qt_ptr[t + 1])}
            assert got == want, t

    run()


def test_static_schedule_deals_every_item_out_once():
    """the static schedule: the same items as the queue's lists, regrouped into one list per workgroup; workgroup b serves XCD
    b % 8 (its items come from that XCD's list, in that list's order); lists are balanced under the cost model"""
    cfg = synth.attention_config("C2", contents=7)
    b = cfg.batches[0]
    for ktile in (64, 32):
        plan = sa.TilePlan.build(b.art, b.end, b.pos, None, ktile=ktile)
        for head_groups, n_lists in ((8, 64), (8, 256), (3, 40), (1, 8)):
            items, list_ptr = plan.schedule(head_groups)
            sitems, sptr = plan.schedule_static(head_groups, n_lists)
            assert sitems.shape == items.shape and len(sptr) == n_lists + 1
            assert sptr[0] == 0 and sptr[-1] == len(items) and (np.diff(sptr) >= 0).all()
            key = lambda rows: sorted(map(tuple, rows.tolist()))
            assert key(sitems) == key(items)
            xcd_of = {}
            for l in range(8):
                for pos_in_list, row in enumerate(items[list_ptr[l] : list_ptr[l + 1]].tolist()):
                    xcd_of[tuple(row)] = (l, pos_in_list)
            weights = []
            for w in range(n_lists):
                rows = [tuple(r) for r in sitems[sptr[w] : sptr[w + 1]].tolist()]
                where = [xcd_of[r] for r in rows]
                assert all(l == w % 8 for l, _ in where)
                assert [p for _, p in where] == sorted(p for _, p in where)   # a workgroup takes its XCD's items in list order
                weights.append(sum(r[2] & 0xFFFFF for r in rows))
            if n_lists * 4 <= len(items):
                assert max(weights) <= 1.6 * (sum(weights) / n_lists) + 40
    lib = sa.load_library()
    assert lib.spinf_tileplan_schedule_static(plan._handle, 1, 0, None, None) == -1 and b"null argument" in lib.spinf_last_error()


def test_gdn_plan_compiler_edge_cases():
    """the C ABI of the recurrent-layer plan compiler on the degenerate inputs: an empty stream, pads only, one token, bad arguments"""
    import ctypes as C

    from spinf_serve_amd import qwen_plan

    lib = sa.load_library()
    empty = qwen_plan._compile(np.zeros(0, np.int64), np.zeros(0, np.uint8), "indexed", 64, 8192, 96, None, None)
    assert empty["n_segments"] == 0 and len(empty["idx"]) == 0 and len(empty["level_ptr"]) == 1
    pads = qwen_plan._compile(np.full(5, -1, np.int64), np.zeros(5, np.uint8), "indexed", 64, 8192, 96, None, None)
    assert pads["n_segments"] == 0 and (pads["seg_of_row"] == -1).all()
    one = sa.tree_plan(np.array([-1]), np.array([True]), "cpu")
    assert one.n_segments == 1 and len(one.levels) == 1 and one.levels[0][0].cu_cpu.tolist() == [0, 1]
    assert one.conv.tolist() == [[1, 1, 1, 0]]   # no predecessors: the zero row, then the token itself
    handle = C.c_void_p()
    prev = np.array([-1, 0, 5], np.int64)   # token 2 names a later token
    real = np.ones(3, np.uint8)
    assert lib.spinf_gdn_plan_build(prev.ctypes.data, real.ctypes.data, 3, 0, 64, 8192, 96, -1, None, 0, C.byref(handle)) == -1
    assert b"does not point backwards" in lib.spinf_last_error()
    prev = np.array([-1, 0, 1], np.int64)
    assert lib.spinf_gdn_plan_build(prev.ctypes.data, real.ctypes.data, 3, 7, 64, 8192, 96, -1, None, 0, C.byref(handle)) == -1
    assert lib.spinf_gdn_plan_build(prev.ctypes.data, real.ctypes.data, 3, 0, 64, 8192, 96, 2, None, 0, C.byref(handle)) == -1
    assert b"compact rows" in lib.spinf_last_error()
    assert lib.spinf_gdn_plan_build(prev.ctypes.data, real.ctypes.data, 3, 0, 64, 8192, 96, -1, None, 0, None) == -1
    with pytest.raises(ValueError):
        sa.tree_plan(prev, real[:2].astype(bool), "cpu")
    with pytest.raises(ValueError):
        sa.tree_plan(prev, real.astype(bool), "cpu", path="sideways")


def test_argument_blocks_have_the_size_the_library_was_built_with(lib, monkeypatch):
    """spinf_struct_sizes: the ctypes mirrors of the seven argument blocks against sizeof in the built library (load_library checks the
    same at load time and refuses a library of another version instead of passing it misread arguments)"""
    import ctypes as C

    from spinf_serve_amd import _lib

    sizes = (C.c_int64 * 7)()
    assert lib.spinf_struct_sizes(sizes, 7) == 0
    mirrors = (_lib.AttnArgs, _lib.GdnArgs, _lib.GdnPreArgs, _lib.GdnGateArgs, _lib.LmArgs, _lib.LmHeadArgs, _lib.XdecArgs)
    assert list(sizes) == [C.sizeof(m) for m in mirrors]
    assert lib.spinf_struct_sizes(sizes, 6) == -1 and b"7 sizes" in lib.spinf_last_error()

    class Grown(C.Structure):
        _fields_ = list(_lib.LmHeadArgs._fields_) + [("more", C.c_int64)]

    monkeypatch.setattr(_lib, "_LIB", None)
    monkeypatch.setattr(_lib, "LmHeadArgs", Grown)
    with pytest.raises(RuntimeError, match="different versions"):
        _lib.load_library()
