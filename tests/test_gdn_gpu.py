"""GPU parity of the Gated DeltaNet kernels (through the C ABI) against the float64 recurrence of the oracle
(spinf_serve/models/qwen35/gdn.py:176-186).  Tolerances, max abs: 2e-3 on the outputs (unit scale; bf16 inputs and bf16 MFMA
operands with fp32 accumulation, bf16 outputs: measured 2.1e-4 .. 3.8e-4; the reference quotes 4.9e-4 for its own fork identity
in bf16, docs/QWEN.md:51-52) and 5e-3 on the final states (fp32, sums over up to 200 tokens: measured 1.6e-3 .. 2.2e-3).  Every
assertion carries the measured value, and the file's last test prints the largest ones."""

import numpy as np
import pytest
import torch

import spinf_serve_amd as sa
from oracle import gdn as ogdn
from spinf_serve_amd import synth

pytestmark = pytest.mark.gpu
TOL = 2e-3
STATE_TOL = 5e-3


def _np(t):
    return t.float().cpu().numpy()


WORST = {"out": 0.0, "state": 0.0}


def _within(got, want, tol, what):
    """max abs error of a device tensor against the oracle's array, with the measured value in the failure message"""
    err = float(np.abs(_np(got) - want).max()) if want.size else 0.0
    key = "state" if tol is STATE_TOL else "out"
    WORST[key] = max(WORST[key], err)
    assert err <= tol, f"{what}: max abs error {err:.3e} against the float64 recurrence, tolerance {tol:.0e}"
    return err


def _inputs(T, H, HV, dev, seed=0, K=128, V=128):
    cfg = synth.GdnConfig("t", H, HV, K, V, [])
    cfg.batch = type("B", (), {"length": T})()
    return synth.gdn_inputs(cfg, seed=seed, device=dev)


@pytest.mark.parametrize("mode", ["recurrent", "chunked"])
@pytest.mark.parametrize("lens", [[1], [5, 64, 3], [65, 130, 64, 200], [4, 0, 33, 0]])
def test_flat_segments_match_recurrence(dev, mode, lens):
    H, HV = 2, 4
    T = sum(lens)
    t = _inputs(T, H, HV, dev, seed=len(lens))
    cu_cpu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int64)
    cu = cu_cpu.to(dev)
    n = len(lens)
    h0 = (torch.randn((n, HV, 128, 128), device=dev) * 0.1).contiguous()
    h0_idx = torch.tensor([i if i % 2 == 0 else -1 for i in range(n)], device=dev)
    ht = torch.full((n, HV, 128, 128), float("nan"), device=dev)
    ht_idx = torch.arange(n, device=dev)
    args = [t[x][None] for x in ("q", "k", "v", "g", "beta")]
    print(f"case gdn {mode} lens={lens}", flush=True)
    if mode == "recurrent":
        o = sa.recurrent(*args, 128 ** -0.5, cu, n, h0=h0, h0_idx=h0_idx, ht=ht, ht_idx=ht_idx)
    else:
        o = sa.chunked(*args, 128 ** -0.5, cu, cu_cpu.numpy(), h0=h0, h0_idx=h0_idx, ht=ht, ht_idx=ht_idx)
    torch.cuda.synchronize()
    worst = worst_s = 0.0
    for s in range(n):
        a, b = int(cu_cpu[s]), int(cu_cpu[s + 1])
        want, S = ogdn.recurrent(*(_np(t[x][a:b]) for x in ("q", "k", "v", "g", "beta")), h0=_np(h0[s]) if s % 2 == 0 else None)
        worst = max(worst, _within(o[0, a:b], want, TOL, f"{mode} lens={lens} segment {s}"))   # (an empty segment only hands its state on)
        worst_s = max(worst_s, _within(ht[s], S, STATE_TOL, f"{mode} lens={lens} state {s}"))
    print(f"  max abs err o={worst:.3e} state={worst_s:.3e}", flush=True)


def test_rows_by_index_and_skipped_states(dev):
    """idx names stream rows (outputs land on the same rows, other rows untouched); ht_idx < 0 writes nothing"""
    H, HV, T = 2, 4, 300
    t = _inputs(T, H, HV, dev, seed=9)
    rows = np.concatenate([np.arange(200, 290), np.arange(10, 30)])
    idx = torch.from_numpy(rows).to(dev)
    cu_cpu = np.array([0, 90, 110])
    cu = torch.from_numpy(cu_cpu).to(dev)
    for mode in ("recurrent", "chunked"):
        o = torch.full((1, T, HV, 128), 7.0, dtype=torch.bfloat16, device=dev)
        ht = torch.full((2, HV, 128, 128), -3.0, device=dev)
        ht_idx = torch.tensor([-1, 1], device=dev)
        args = [t[x][None] for x in ("q", "k", "v", "g", "beta")]
        if mode == "recurrent":
            sa.recurrent(*args, 128 ** -0.5, cu, 2, ht=ht, ht_idx=ht_idx, idx=idx, o=o)
        else:
            sa.chunked(*args, 128 ** -0.5, cu, cu_cpu, ht=ht, ht_idx=ht_idx, idx=idx, o=o)
        torch.cuda.synchronize()
        untouched = np.setdiff1d(np.arange(T), rows)
        assert (o[0, untouched] == 7.0).all()
        assert (ht[0] == -3.0).all() and not (ht[1] == -3.0).all()
        for a, b in ((0, 90), (90, 110)):
            r = rows[a:b]
            want, _ = ogdn.recurrent(*(_np(t[x][r]) for x in ("q", "k", "v", "g", "beta")))
            _within(o[0, r], want, TOL, f"{mode} rows {a}..{b}")


@pytest.mark.parametrize("mode", ["recurrent", "chunked"])
def test_segments_forked_from_one_state(dev, mode):
    """many short segments that start from the same stored state (what a trunk's leaves look like), mixed with segments that
    are longer than a mini-chunk, keep their final state or start from another state: each must equal its own recurrence"""
    H, HV = 2, 4
    lens = [5, 12, 16, 17, 3, 3, 40, 2, 9, 9, 9, 9, 9, 9, 9, 9, 9, 9, 1, 16, 16, 7]
    src = [0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 1, 1, 1, -1]
    kept = {2, 6, 12}
    n, T = len(lens), sum(lens)
    t = _inputs(T, H, HV, dev, seed=21)
    cu_cpu = np.concatenate([[0], np.cumsum(lens)])
    cu = torch.from_numpy(cu_cpu).to(dev)
    h0 = (torch.randn((2, HV, 128, 128), device=dev) * 0.1).contiguous()
    h0_idx = torch.tensor(src, device=dev)
    ht = torch.full((n, HV, 128, 128), float("nan"), device=dev)
    ht_idx = torch.tensor([i if i in kept else -1 for i in range(n)], device=dev)
    args = [t[x][None] for x in ("q", "k", "v", "g", "beta")]
    if mode == "recurrent":
        o = sa.recurrent(*args, 128 ** -0.5, cu, n, h0=h0, h0_idx=h0_idx, ht=ht, ht_idx=ht_idx)
    else:
        o = sa.chunked(*args, 128 ** -0.5, cu, cu_cpu, h0=h0, h0_idx=h0_idx, ht=ht, ht_idx=ht_idx)
    torch.cuda.synchronize()
    for s in range(n):
        a, b = int(cu_cpu[s]), int(cu_cpu[s + 1])
        want, S = ogdn.recurrent(*(_np(t[x][a:b]) for x in ("q", "k", "v", "g", "beta")), h0=_np(h0[src[s]]) if src[s] >= 0 else None)
        _within(o[0, a:b], want, TOL, f"{mode} segment {s}")
        if s in kept:
            _within(ht[s], S, STATE_TOL, f"{mode} state {s}")
        else:
            assert torch.isnan(ht[s]).all(), s


@pytest.mark.parametrize("V", [64, 256])
def test_recurrent_other_value_dims(dev, V):
    """value head dims other than 128 take the one-wave-per-32-columns kernel of the recurrent entry point"""
    H, HV = 2, 4
    lens = [5, 20, 33, 16]
    n, T = len(lens), sum(lens)
    t = _inputs(T, H, HV, dev, seed=5, V=V)
    cu_cpu = np.concatenate([[0], np.cumsum(lens)])
    cu = torch.from_numpy(cu_cpu).to(dev)
    h0 = (torch.randn((n, HV, 128, V), device=dev) * 0.1).contiguous()
    h0_idx = torch.tensor([0, -1, 2, 3], device=dev)
    ht = torch.full((n, HV, 128, V), float("nan"), device=dev)
    ht_idx = torch.tensor([0, 1, -1, 3], device=dev)
    args = [t[x][None] for x in ("q", "k", "v", "g", "beta")]
    o = sa.recurrent(*args, 128 ** -0.5, cu, n, h0=h0, h0_idx=h0_idx, ht=ht, ht_idx=ht_idx)
    torch.cuda.synchronize()
    for s in range(n):
        a, b = int(cu_cpu[s]), int(cu_cpu[s + 1])
        want, S = ogdn.recurrent(*(_np(t[x][a:b]) for x in ("q", "k", "v", "g", "beta")), h0=_np(h0[s]) if int(h0_idx[s]) >= 0 else None)
        _within(o[0, a:b], want, TOL, f"value dim {V} segment {s}")
        if int(ht_idx[s]) >= 0:
            _within(ht[s], S, STATE_TOL, f"value dim {V} state {s}")
        else:
            assert torch.isnan(ht[s]).all(), s


def test_tree_scan_forks_from_trunk_state(dev):
    """C5's shape scaled down: every branch continues from its trunk's final state == one sequence trunk||branch"""
    cfg = synth.gdn_config("C5", contents=2)
    t = synth.gdn_inputs(cfg, seed=1, device=dev)
    plan = cfg.plan(dev)
    assert [[c.kind for c in lv] for lv in plan.levels] == [["chunked"], ["recurrent"]]
    o = sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], plan)
    torch.cuda.synchronize()
    b = cfg.batch
    want = ogdn.tree_scan(*(_np(t[x]) for x in ("q", "k", "v", "g", "beta")), b.prev, b.art >= 0)
    err = _within(o, want, TOL, "C5 x2 contents")
    print(f"C5 x2 contents: max abs err {err:.3e}", flush=True)
    assert (o[torch.from_numpy(b.art < 0).to(dev)] == 0).all()
    # the short-segment threshold only picks the kernel: a plan that runs everything chunked agrees
    o2 = sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], cfg.plan(dev, short=4))
    _within(o2, want, TOL, "C5 x2 contents, all chunked")


def test_deep_trie(dev):
    rng = np.random.default_rng(8)
    lens, parents = [], []
    for _ in range(3):
        node = len(lens)
        lens.append(70); parents.append(-1)
        for _ in range(3):
            leaf = len(lens)
            lens.append(int(rng.integers(2, 9))); parents.append(node)
            lens.append(3); parents.append(leaf)
            lens.append(2); parents.append(leaf)
    trees = [synth._tree(rng, 131, lens, parents), synth._tree(rng, 20, [4, 4])]
    cfg = synth.GdnConfig("deep", 2, 4, 128, 128, trees)
    cfg.batch = synth.pack(trees)[0]
    t = synth.gdn_inputs(cfg, seed=2, device=dev)
    o = sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], cfg.plan(dev))
    want = ogdn.tree_scan(*(_np(t[x]) for x in ("q", "k", "v", "g", "beta")), cfg.batch.prev, cfg.batch.art >= 0)
    _within(o, want, TOL, "deep tree")


def test_decoder_steps_rerun_the_recurrence_from_the_prefix_state(dev):
    """the extraction decoder's call (spinf_serve/models/qwen35/qwen_decode.py:305-318): every step each slot re-runs the recurrence
    from its group's prefix state over its template rows plus the tokens generated so far, read out of row caches through idx,
    outputs written into a buffer at the same rows; no per-slot state is kept.  Two groups, slots of different template lengths."""
    H, HV, R = 2, 4, 512
    rng = np.random.default_rng(2)
    t = _inputs(R, H, HV, dev, seed=9)                       # the row caches: any row may belong to any slot
    caches = [t[x][None] for x in ("q", "k", "v", "g", "beta")]
    states = (torch.randn((2, HV, 128, 128), device=dev) * 0.1).contiguous()   # the two groups' prefix states
    slot_group = [0, 0, 0, 1, 1]
    templates = [5, 17, 30, 9, 40]
    free = list(rng.permutation(R))
    rows = [[int(free.pop()) for _ in range(n)] for n in templates]            # each slot's template rows, scattered
    o_buf = torch.full((1, R, HV, 128), float("nan"), device=dev, dtype=torch.bfloat16)
    h0_idx = torch.tensor(slot_group, device=dev)
    for step in range(4):
        for r in rows:
            r.append(int(free.pop()))                                            # the step's new token of every slot
        lens = [len(r) for r in rows]
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int64, device=dev)
        idx = torch.tensor([x for r in rows for x in r], dtype=torch.int64, device=dev)
        sa.recurrent(*caches, 128 ** -0.5, cu, len(rows), h0=states, h0_idx=h0_idx, idx=idx, o=o_buf)
        torch.cuda.synchronize()
        for s, r in enumerate(rows):
            want, _ = ogdn.recurrent(*(_np(t[x][r]) for x in ("q", "k", "v", "g", "beta")), h0=_np(states[slot_group[s]]))
            _within(o_buf[0, r[-1]], want[-1], TOL, f"decoder step {step} slot {s}, the new token's row")   # (the row the decoder reads)
            _within(o_buf[0, r], want, TOL, f"decoder step {step} slot {s}")
    used = sorted(x for r in rows for x in r)
    untouched = np.setdiff1d(np.arange(R), used)
    assert torch.isnan(o_buf[0, untouched].float()).all()                         # rows of no slot are never written


def test_zz_report_worst_errors():
    """(runs last in this file) the largest errors the tests above measured, for the record"""
    print(f"gdn kernels against the float64 recurrence: worst max abs error outputs {WORST['out']:.3e} (tolerance {TOL:.0e}), "
          f"states {WORST['state']:.3e} (tolerance {STATE_TOL:.0e})", flush=True)
