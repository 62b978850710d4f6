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


def test_argument_checks_come_before_any_launch():
    import ctypes as C

    from spinf_serve_amd import _lib

    lib = sa.load_library()
    a = _lib.LmArgs()
    a.rows, a.vocab = 4, 100
    assert lib.spinf_lm_logprobs(C.byref(a), None) != 0 and b"null pointer" in lib.spinf_last_error()
    with pytest.raises(RuntimeError):
        sa.lm_logprobs(torch.zeros(2, 64), None, 30.0)   # no CPU path


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
