"""The lm head read-out kernel (soft-capping + log-softmax + column selection) against the numpy oracle, and the oracle against
torch's own routines."""

import numpy as np
import pytest
import torch

import spinf_serve_amd as sa
from oracle import lm_head as olm

TOL = 2e-5   # max abs error of a fp32 log-prob (values down to about -40)


def test_oracle_is_torchs_tanh_and_log_softmax():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((5, 1000)) * 20).astype(np.float32)
    cols = [3, 999, 0, 17]
    for cap in (None, 30.0):
        t = torch.from_numpy(x).double()
        if cap:
            t = torch.tanh(t / cap) * cap
        want = torch.log_softmax(t, -1).numpy()
        assert np.abs(olm.logprobs(x, None, cap) - want).max() < 1e-12
        assert np.abs(olm.logprobs(x, cols, cap) - want[:, cols]).max() < 1e-12
    assert np.allclose(np.exp(olm.logprobs(x, None, 30.0)).sum(1), 1.0, atol=1e-12)


def _bf16_values(rng, shape, scale):
    return torch.from_numpy((rng.standard_normal(shape) * scale).astype(np.float32)).to(torch.bfloat16)


def test_oracle_gemm_modes_are_torchs_matmul():
    """the float64 mode against torch's float64 matmul; the bf16 mode against torch's bf16 tensors on the CPU, where a logit may
    land on the neighbouring bf16 value (torch accumulates in fp32, the oracle in float64)"""
    rng = np.random.default_rng(1)
    h, w = _bf16_values(rng, (40, 128), 1.0), _bf16_values(rng, (300, 128), 1.0)
    sel, cols, cap = [3, 39, 0, 3], [0, 299, 17], 30.0
    want = torch.log_softmax(torch.tanh(h.double()[sel] @ w.double().t() / cap) * cap, -1).numpy()
    got = olm.head_logprobs(h.float().numpy(), w.float().numpy(), sel, None, cap)
    assert np.abs(got - want).max() < 1e-12
    assert np.abs(olm.head_logprobs(h.float().numpy(), w.float().numpy(), sel, cols, cap) - want[:, cols]).max() < 1e-12
    x = h[sel] @ w.t()
    want16 = torch.log_softmax((torch.tanh(x / cap) * cap).float(), -1).numpy()
    got16 = olm.head_logprobs(h.float().numpy(), w.float().numpy(), sel, None, cap, bf16_logits=True)
    d = np.abs(got16 - want16)
    assert (d < 1e-5).mean() > 0.97 and d.max() < 0.3   # one bf16 step of a logit near 30 is 0.125
    assert np.array_equal(olm.round_bf16([1.0, 1.00390625, 1.01171875, -3.0e38]), np.float64(torch.tensor([1.0, 1.00390625, 1.01171875, -3.0e38]).bfloat16().float().numpy()))


def test_argument_checks_come_before_any_launch():
    import ctypes as C

    from spinf_serve_amd import _lib

    lib = sa.load_library()
    a = _lib.LmArgs()
    a.rows, a.vocab = 4, 100
    assert lib.spinf_lm_logprobs(C.byref(a), None) != 0 and b"null pointer" in lib.spinf_last_error()
    with pytest.raises(RuntimeError):
        sa.lm_logprobs(torch.zeros(2, 64), None, 30.0)   # no CPU path
    b = _lib.LmHeadArgs()
    b.rows, b.vocab, b.hidden, b.h_rows = 4, 100, 100, 4
    need = C.c_int64()
    assert lib.spinf_lm_head_workspace(C.byref(b), C.byref(need)) != 0 and b"multiple of 64" in lib.spinf_last_error()
    b.hidden = 128
    assert lib.spinf_lm_head_workspace(C.byref(b), C.byref(need)) == 0 and need.value == 4 * 2 * 8
    assert lib.spinf_lm_head_fwd(C.byref(b), None) != 0 and b"null pointer" in lib.spinf_last_error()
    b.h_rows = 0
    assert lib.spinf_lm_head_workspace(C.byref(b), C.byref(need)) != 0 and b"h_rows" in lib.spinf_last_error()
    b.h_rows = 3   # no row list: rows 0 .. 3 of an h of three rows
    assert lib.spinf_lm_head_workspace(C.byref(b), C.byref(need)) != 0 and b"without a row list" in lib.spinf_last_error()
    with pytest.raises(RuntimeError):
        sa.lm_head_logprobs(torch.zeros(2, 64, dtype=torch.bfloat16), None, torch.zeros(8, 64, dtype=torch.bfloat16))   # no CPU path


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    return torch.device("cuda:0")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,vocab,cap", [(7, 262144, 30.0), (3, 1000, None), (2, 1003, 30.0), (5, 151936, None), (1, 8, 30.0)])
def test_logprobs_match_the_oracle(dev, dtype, rows, vocab, cap):
    rng = np.random.default_rng(rows * 1000 + vocab)
    x = torch.from_numpy((rng.standard_normal((rows, vocab)) * 12).astype(np.float32)).to(dtype)
    if vocab % 8:   # rows must stay 16-byte aligned: a wider allocation, as a GEMM output with a padded leading dimension has
        wide = torch.zeros((rows, (vocab + 7) // 8 * 8), dtype=dtype)
        wide[:, :vocab] = x
        xd = wide.to(dev)[:, :vocab]
    else:
        xd = x.to(dev)
    want = olm.logprobs(x.float().numpy(), None, cap)
    got = sa.lm_logprobs(xd, None, cap).cpu().numpy()
    assert got.shape == want.shape and np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL
    cols = torch.from_numpy(rng.integers(0, vocab, 11)).to(dev)
    sel = sa.lm_logprobs(xd, cols, cap).cpu().numpy()
    assert sel.shape == (rows, 11)
    assert np.abs(sel - want[:, cols.cpu().numpy()]).max() <= TOL


@pytest.mark.gpu
def test_rows_are_independent_of_what_they_are_batched_with(dev):
    """a read row's log-probs are the same bits alone, in a chunk of 1,024 rows, and at another row of the chunk"""
    rng = np.random.default_rng(5)
    x = torch.from_numpy((rng.standard_normal((64, 32768)) * 10).astype(np.float32)).to(dev)
    cols = torch.tensor([1, 5, 32767], device=dev)
    full = sa.lm_logprobs(x, cols, 30.0)
    assert torch.equal(sa.lm_logprobs(x[17:18], cols, 30.0), full[17:18])
    assert torch.equal(sa.lm_logprobs(x.flip(0), cols, 30.0).flip(0), full)


@pytest.mark.gpu
def test_columns_outside_the_vocabulary(dev):
    """negative columns count from the end (torch indexing, as the reference's [:, ci]); anything else outside gives NaN"""
    x = torch.randn(3, 1000, device=dev)
    cols = torch.tensor([-1, 999, -1000, 0, 1000, -1001], device=dev)
    got = sa.lm_logprobs(x, cols, 30.0)
    assert torch.equal(got[:, 0], got[:, 1]) and torch.equal(got[:, 2], got[:, 3])
    assert torch.isnan(got[:, 4:]).all() and torch.isfinite(got[:, :4]).all()
    h, w = torch.randn(3, 64, device=dev).bfloat16(), torch.randn(1000, 64, device=dev).bfloat16()
    got = sa.lm_head_logprobs(h, None, w, cols, 30.0)
    assert torch.equal(got[:, 0], got[:, 1]) and torch.equal(got[:, 2], got[:, 3])
    assert torch.isnan(got[:, 4:]).all() and torch.isfinite(got[:, :4]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("rows,vocab,hidden,cap", [(7, 1000, 128, 30.0), (130, 1003, 64, None), (300, 4099, 256, 30.0), (1, 8, 64, 30.0), (129, 131, 192, None)])
def test_fused_head_matches_the_oracle(dev, rows, vocab, hidden, cap):
    rng = np.random.default_rng(rows + vocab)
    h, w = _bf16_values(rng, (rows + 50, hidden), 1.0), _bf16_values(rng, (vocab, hidden), 12.0 / hidden ** 0.5)
    sel = rng.integers(0, rows + 50, rows)
    hd, wd, seld = h.to(dev), w.to(dev), torch.from_numpy(sel).to(dev)
    want = olm.head_logprobs(h.float().numpy(), w.float().numpy(), sel, None, cap)
    got = sa.lm_head_logprobs(hd, seld, wd, None, cap).cpu().numpy()
    assert got.shape == want.shape and np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL
    cols = rng.integers(0, vocab, 11)
    part = sa.lm_head_logprobs(hd, seld, wd, torch.from_numpy(cols).to(dev), cap)
    assert np.array_equal(part.cpu().numpy(), got[:, cols])   # the same bits as the whole row's
    # without a row list: rows 0 .. of h itself
    head = sa.lm_head_logprobs(hd[:rows], None, wd, torch.from_numpy(cols).to(dev), cap).cpu().numpy()
    assert np.abs(head - olm.head_logprobs(h.float().numpy()[:rows], w.float().numpy(), None, cols, cap)).max() <= TOL


@pytest.mark.gpu
def test_fused_head_row_list_entries_are_checked_on_the_device(dev):
    """sel is a device tensor: a negative entry counts from the end (Hf[sel] in the reference, spinf_serve/scorer.py:247-261), an
    entry outside h reads nothing outside h and gives a row of NaN; the rows beside it are not affected"""
    rng = np.random.default_rng(5)
    n = 40
    h, w = _bf16_values(rng, (n, 128), 1.0).to(dev), _bf16_values(rng, (1000, 128), 1.0).to(dev)
    good = torch.tensor([0, 39, 17, 17, 5], device=dev)
    want = sa.lm_head_logprobs(h, good, w, None, 30.0)
    sel = torch.tensor([0, -1, n, 17, -n - 1, -23, 1 << 40, 5, -(1 << 40)], device=dev)
    got = sa.lm_head_logprobs(h, sel, w, None, 30.0)
    assert torch.equal(got[[0, 1, 3, 5, 7]], want)
    assert torch.isnan(got[[2, 4, 6, 8]]).all()
    cols = torch.tensor([3, 999, 500], device=dev)
    part = sa.lm_head_logprobs(h, sel, w, cols, 30.0)
    assert torch.equal(part[[0, 1, 3, 5, 7]], want[:, cols]) and torch.isnan(part[[2, 4, 6, 8]]).all()


@pytest.mark.gpu
@pytest.mark.parametrize("cap", [30.0, None])
def test_fused_head_bf16_logits(dev, cap):
    """the reference's default mode: bf16 logits, capped in bf16 steps.  A logit whose fp32 accumulator sits at a rounding boundary
    may land on the neighbouring bf16 value (the oracle accumulates in float64): almost all values agree to fp32 accuracy, the rest
    within one bf16 step of a logit (0.125 near the cap) plus its effect on the log-sum-exp"""
    rng = np.random.default_rng(11)
    h, w = _bf16_values(rng, (200, 256), 1.0), _bf16_values(rng, (5000, 256), 0.75)
    got = sa.lm_head_logprobs(h.to(dev), None, w.to(dev), None, cap, logits="bf16").cpu().numpy()
    want = olm.head_logprobs(h.float().numpy(), w.float().numpy(), None, None, cap, bf16_logits=True)
    d = np.abs(got - want)
    assert (d < 1e-3).mean() > 0.97 and d.max() < 0.3
    lse_shift = np.abs(np.log(np.exp(got).sum(1)))   # every row still sums to one
    assert lse_shift.max() < 1e-5


@pytest.mark.gpu
def test_fused_head_rows_are_independent_of_the_batch(dev):
    """a read row's log-probs are the same bits alone, among 1,024 rows, and at another place among them: what the reference pads
    its last chunk to lm_rows for"""
    rng = np.random.default_rng(7)
    h, w = _bf16_values(rng, (1024, 512), 1.0).to(dev), _bf16_values(rng, (32768 + 40, 512), 0.5).to(dev)
    cols = torch.tensor([1, 5, 32767, 32800], device=dev)
    for cap in (30.0, None):
        full = sa.lm_head_logprobs(h, None, w, cols, cap)
        assert torch.equal(sa.lm_head_logprobs(h[517:518], None, w, cols, cap), full[517:518])
        assert torch.equal(sa.lm_head_logprobs(h, torch.arange(1023, -1, -1, device=dev), w, cols, cap).flip(0), full)
        assert torch.equal(sa.lm_head_logprobs(h[100:230], None, w, cols, cap), full[100:230])


@pytest.mark.gpu
def test_fused_head_at_the_reference_vocabulary(dev):
    """262,144 x 2,560 head, 256 read rows, against torch's fp32-output GEMM followed by the read-out kernel (itself checked
    against the oracle above): the two differ by fp32 accumulation order only"""
    g = torch.Generator(device="cpu").manual_seed(3)
    h = torch.randn(4096, 2560, generator=g).bfloat16().to(dev)
    w = (torch.randn(262144, 2560, generator=g) * 0.02).bfloat16().to(dev)
    sel = torch.randint(0, 4096, (256,), generator=g).to(dev)
    cols = torch.randint(0, 262144, (16,), generator=g).to(dev)
    got = sa.lm_head_logprobs(h, sel, w, cols, 30.0)
    want = sa.lm_logprobs(torch.mm(h[sel], w.t(), out_dtype=torch.float32), cols, 30.0)
    assert (got - want).abs().max().item() <= 1e-4


@pytest.mark.gpu
def test_fused_head_columns_at_tile_and_wave_boundaries(dev):
    """selected columns on both sides of every 32 / 128 / 256 boundary of the vocabulary tiling, read rows across the 256-row tile
    boundary, a vocabulary that ends inside a wave's quarter: the same bits as the whole row's"""
    rng = np.random.default_rng(21)
    rows, vocab, hidden = 259, 700, 128
    h, w = _bf16_values(rng, (rows, hidden), 1.0), _bf16_values(rng, (vocab, hidden), 1.0)
    cols = np.array([0, 31, 32, 127, 128, 129, 255, 256, 257, 383, 384, 511, 512, 639, 640, 699, 1, 698])
    whole = sa.lm_head_logprobs(h.to(dev), None, w.to(dev), None, 30.0)
    part = sa.lm_head_logprobs(h.to(dev), None, w.to(dev), torch.from_numpy(cols).to(dev), 30.0)
    assert torch.equal(part, whole[:, torch.from_numpy(cols).to(dev)])
    want = olm.head_logprobs(h.float().numpy(), w.float().numpy(), None, None, 30.0)
    assert np.abs(whole.cpu().numpy() - want).max() <= TOL
    assert np.abs(np.exp(whole.double().cpu().numpy()).sum(1) - 1.0).max() < 1e-5
