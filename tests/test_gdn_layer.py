"""The Gated DeltaNet layer's element-wise kernels (prologue: path convolution, silu, l2 norm, beta, g; gate: rms norm x silu(z))
against the numpy oracle, and the oracle against torch's own routines on the cases that reduce to them."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import spinf_serve_amd as sa
from oracle import gdn_layer as og
from spinf_serve_amd import synth

TOL = 2e-2   # max abs error of a bf16 result against the float32 oracle


def _bf(x):   # float32 array -> torch bf16 tensor
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(torch.bfloat16)


def _layer(T, h, hv, dk, dv, seed, extra_cols=0):
    rng = np.random.default_rng(seed)
    cols = 2 * h * dk + 2 * hv * dv + 2 * hv + extra_cols
    y = og.bf16(rng.standard_normal((T, cols)).astype(np.float32))
    conv_w = (rng.standard_normal((2 * h * dk + hv * dv, 4)) * 0.5).astype(np.float32)
    a_log = rng.uniform(-1.0, 1.5, hv).astype(np.float32)
    dt_bias = rng.standard_normal(hv).astype(np.float32)
    return y, conv_w, a_log, dt_bias


def _path_taps(prev):
    """[T, 4] rows of the 3 path predecessors and the token itself, T where there is none (qwen.py:260-265)"""
    T = len(prev)
    conv = np.full((T, 4), T, np.int64)
    conv[:, 3] = np.arange(T)
    hop = np.asarray(prev, np.int64).copy()
    for j in (2, 1, 0):
        conv[:, j] = np.where(hop >= 0, hop, T)
        hop = np.where(hop >= 0, np.asarray(prev, np.int64)[np.maximum(hop, 0)], -1)
    return conv


def test_bf16_rounding_is_torchs():
    x = np.random.default_rng(0).standard_normal(4096).astype(np.float32) * np.float32(37.0)
    x[:4] = [1.00390625, 1.01171875, -3.0e-39, 65280.0]   # ties and a denormal
    assert np.array_equal(og.bf16(x), torch.from_numpy(x).to(torch.bfloat16).float().numpy())


def test_oracle_prologue_on_one_path_is_a_depthwise_conv1d():
    """prev = i - 1: the tap convolution is conv1d with 3 zeros on the left; silu, sigmoid, softplus, normalize are torch's"""
    T, h, hv, dk, dv = 50, 2, 4, 16, 8
    y, conv_w, a_log, dt_bias = _layer(T, h, hv, dk, dv, 1)
    conv = _path_taps(np.arange(T) - 1)
    q, k, v, g, beta = og.prologue(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, normalize=True)
    cd = 2 * h * dk + hv * dv
    x = torch.from_numpy(y[:, :cd].T.copy())[None]                                     # [1, C, T]
    ref = F.conv1d(F.pad(x, (3, 0)), torch.from_numpy(conv_w)[:, None, :], groups=cd)[0].T   # [T, C]
    ref = F.silu(ref).to(torch.bfloat16).float()
    rq = ref[:, : h * dk].reshape(T, h, dk)
    rq = (rq * torch.rsqrt(rq.pow(2).sum(-1, keepdim=True) + 1e-6)).to(torch.bfloat16).float()
    # float32 sums in another order: the odd value may round to the neighbouring bf16
    assert np.abs(q - rq.numpy()).max() <= 2 ** -8
    assert (q == rq.numpy()).mean() > 0.98
    assert np.abs(v - ref[:, 2 * h * dk :].reshape(T, hv, dv).numpy()).max() <= 2 ** -6 and (v == ref[:, 2 * h * dk :].reshape(T, hv, dv).numpy()).mean() > 0.98
    assert np.allclose((q.astype(np.float64) ** 2).sum(-1), 1.0, atol=2e-2)           # unit rows
    b = torch.from_numpy(y[:, cd + hv * dv : cd + hv * dv + hv])
    a = torch.from_numpy(y[:, cd + hv * dv + hv : cd + hv * dv + 2 * hv])
    assert np.array_equal(beta, torch.sigmoid(b).to(torch.bfloat16).float().numpy()) or np.abs(beta - torch.sigmoid(b).numpy()).max() <= 2 ** -8
    rg = -torch.from_numpy(a_log).exp() * F.softplus(a + torch.from_numpy(dt_bias))
    assert np.allclose(g, rg.numpy(), rtol=1e-5, atol=1e-6)


def test_oracle_prologue_on_a_tree_equals_the_convolution_along_each_path():
    """a branch token's taps reach back into the trunk: same values as convolving trunk || branch as one sequence"""
    h, hv, dk, dv = 1, 2, 8, 8
    trunk, branches = 9, [5, 1, 3]
    prev = list(range(-1, trunk - 1))
    starts = []
    for n in branches:
        starts.append(len(prev))
        prev += [trunk - 1] + list(range(len(prev), len(prev) + n - 1))
    T = len(prev)
    y, conv_w, a_log, dt_bias = _layer(T, h, hv, dk, dv, 2)
    conv = _path_taps(prev)
    q, k, v, _, _ = og.prologue(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, normalize=False)
    for s0, n in zip(starts, branches):
        rows = list(range(trunk)) + list(range(s0, s0 + n))
        sub = og.prologue(y[rows], _path_taps(np.arange(len(rows)) - 1), conv_w, a_log, dt_bias, h, hv, dk, dv, normalize=False)
        for got, want in zip((q, k, v), sub[:3]):
            assert np.array_equal(got[rows], want)
    # and the plan's own taps (the reference's layout of them) are these
    plan = sa.tree_plan(np.asarray(prev), np.ones(T, bool), "cpu")
    assert np.array_equal(np.asarray(plan.conv), conv)


def test_oracle_gate_is_torchs_rms_norm_times_silu():
    T, hv, dv = 33, 3, 16
    rng = np.random.default_rng(3)
    o = og.bf16(rng.standard_normal((T, hv, dv)).astype(np.float32) * 3)
    z = og.bf16(rng.standard_normal((T, hv * dv)).astype(np.float32))
    nw = og.bf16(rng.uniform(0.5, 1.5, dv).astype(np.float32))
    got = og.gate(o, z, nw, 1e-6)
    n = F.rms_norm(torch.from_numpy(o), (dv,), eps=1e-6).to(torch.bfloat16)
    ref = ((_bf(nw) * n).float() * F.silu(torch.from_numpy(z).reshape(T, hv, dv))).to(torch.bfloat16).float().reshape(T, hv * dv)
    assert np.abs(got - ref.numpy()).max() <= 2 ** -5 and (got == ref.numpy()).mean() > 0.98


def test_argument_checks_come_before_any_launch():
    import ctypes as C

    from spinf_serve_amd import _lib

    lib = sa.load_library()
    a = _lib.GdnPreArgs()
    a.T = 4
    assert lib.spinf_gdn_prologue(C.byref(a), None) != 0 and b"null pointer" in lib.spinf_last_error()
    g = _lib.GdnGateArgs()
    g.T = 4
    assert lib.spinf_gdn_gate(C.byref(g), None) != 0 and b"null pointer" in lib.spinf_last_error()
    with pytest.raises(RuntimeError):
        sa.gdn_gate(torch.zeros(2, 2, 128, dtype=torch.bfloat16), torch.zeros(2, 256, dtype=torch.bfloat16), torch.ones(128), 1e-6)   # no CPU path


# ------------------------------------------------------------------------------------------------ GPU
@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("h,hv,dk,dv,normalize,extra", [(16, 32, 128, 128, True, 0), (4, 8, 128, 128, False, 24), (2, 6, 64, 64, True, 4), (1, 1, 256, 128, True, 6)])
def test_prologue_matches_the_oracle_on_a_packed_tree(dev, h, hv, dk, dv, normalize, extra):
    cfg = synth.gdn_config("C5", contents=2)
    b = cfg.batch
    plan = sa.tree_plan(b.prev, b.art >= 0, dev)
    T = b.length if (h, hv) == (16, 32) else 700
    conv = np.asarray(plan.conv.cpu())[:T].copy()
    conv[conv >= T] = T
    y, conv_w, a_log, dt_bias = _layer(T, h, hv, dk, dv, 5, extra_cols=extra)
    want = og.prologue(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, normalize)
    got = sa.gdn_prologue(_bf(y).to(dev), torch.from_numpy(conv).to(dev), torch.from_numpy(conv_w).to(dev), torch.from_numpy(a_log).to(dev),
                          torch.from_numpy(dt_bias).to(dev), h, hv, dk, dv, normalize)
    for name, g_, w_ in zip("q k v g beta".split(), got, want):
        g_ = g_.float().cpu().numpy()
        assert g_.shape == w_.shape, name
        if name == "g":
            assert np.allclose(g_, w_, rtol=2e-5, atol=1e-6), name
        else:
            assert np.abs(g_ - w_).max() <= TOL, (name, float(np.abs(g_ - w_).max()))
            assert (g_ == w_).mean() > 0.97, (name, float((g_ == w_).mean()))


@pytest.mark.gpu
def test_prologue_reads_strided_rows_and_zero_rows_outside_the_stream(dev):
    """y as a column range of a wider matrix; tap indices below 0 or above T - 1 are the zero row"""
    T, h, hv, dk, dv = 300, 2, 4, 128, 128
    y, conv_w, a_log, dt_bias = _layer(T, h, hv, dk, dv, 7)
    conv = _path_taps(np.arange(T) - 1)
    want = og.prologue(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, True)
    wide = torch.zeros(T, y.shape[1] + 64, dtype=torch.bfloat16, device=dev)
    wide[:, : y.shape[1]] = _bf(y).to(dev)
    conv2 = conv.copy()
    conv2[conv2 == T] = -1          # another spelling of "none"
    conv2[0, 0] = T + 5
    got = sa.gdn_prologue(wide[:, : y.shape[1]], torch.from_numpy(conv2).to(dev), torch.from_numpy(conv_w).to(dev), torch.from_numpy(a_log).to(dev),
                          torch.from_numpy(dt_bias).to(dev), h, hv, dk, dv, True)
    for g_, w_ in zip(got, want):
        assert np.abs(g_.float().cpu().numpy() - w_).max() <= TOL


@pytest.mark.gpu
@pytest.mark.parametrize("hv,dv,T", [(32, 128, 5000), (6, 64, 257), (1, 256, 40)])
def test_gate_matches_the_oracle(dev, hv, dv, T):
    rng = np.random.default_rng(9)
    o = og.bf16(rng.standard_normal((T, hv, dv)).astype(np.float32) * 2)
    wide = og.bf16(rng.standard_normal((T, hv * dv + 72)).astype(np.float32))   # z is a column range of the projection's rows
    nw = og.bf16(rng.uniform(0.5, 1.5, dv).astype(np.float32))
    want = og.gate(o, wide[:, 8 : 8 + hv * dv], nw, 1e-6)
    wd = _bf(wide).to(dev)
    got = sa.gdn_gate(_bf(o).to(dev), wd[:, 8 : 8 + hv * dv], _bf(nw).to(dev), 1e-6).float().cpu().numpy()
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= TOL * max(1.0, float(np.abs(want).max()))
    assert (got == want).mean() > 0.97


@pytest.mark.gpu
def test_layer_end_to_end_prologue_scan_gate(dev):
    """prologue -> tree scan -> gate on a small packed tree against the oracle's chain (float64 scan on the oracle's q, k, v)"""
    from oracle import gdn as ogdn

    cfg = synth.gdn_config("C5", contents=1)
    b = cfg.batch
    T = b.length
    h, hv, dk, dv = 2, 4, 128, 128
    plan = sa.tree_plan(b.prev, b.art >= 0, dev)
    conv = np.asarray(plan.conv.cpu())
    y, conv_w, a_log, dt_bias = _layer(T, h, hv, dk, dv, 11)
    q, k, v, g, beta = og.prologue(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, True)
    o = ogdn.tree_scan(q, k, v, g, beta, b.prev, b.art >= 0)
    cd = 2 * h * dk + hv * dv
    nw = og.bf16(np.random.default_rng(1).uniform(0.5, 1.5, dv).astype(np.float32))
    want = og.gate(og.bf16(o.astype(np.float32)), y[:, cd : cd + hv * dv], nw, 1e-6)
    yd = _bf(y).to(dev)
    gq, gk, gv, gg, gb = sa.gdn_prologue(yd, plan.conv, torch.from_numpy(conv_w).to(dev), torch.from_numpy(a_log).to(dev), torch.from_numpy(dt_bias).to(dev),
                                         h, hv, dk, dv, True)
    go = sa.gdn_tree(gq, gk, gv, gg, gb, plan)
    got = sa.gdn_gate(go, yd[:, cd : cd + hv * dv], _bf(nw).to(dev), 1e-6).float().cpu().numpy()
    real = b.art >= 0
    # the rms norm divides a head's output by its size: the scan's 2e-2 absolute bound becomes 2e-2 / rms(o) per head row, times
    # the gate factor norm_w silu(z); plus the bf16 rounding of the result itself
    rms = np.sqrt((o.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6)                        # [T, hv, 1]
    zf = y[:, cd : cd + hv * dv].reshape(T, hv, dv).astype(np.float64)
    bound = (TOL / rms) * np.abs(nw.astype(np.float64))[None, None] * np.abs(zf / (1 + np.exp(-zf))) + TOL
    err = np.abs(got.reshape(T, hv, dv) - want.reshape(T, hv, dv))
    assert (err[real] <= bound[real]).all(), float((err[real] / bound[real]).max())
    assert err[real].mean() <= 2e-3
