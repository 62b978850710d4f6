"""Hardware assumptions that the kernels lean on, checked on the GPU itself (no counterpart in the reference)."""

import ctypes as C

import pytest
import torch

from spinf_serve_amd import _lib

pytestmark = pytest.mark.gpu


def test_lds_reads_of_mixed_kinds_return_in_issue_order(dev, lib):
    """Every s_waitcnt lgkmcnt(n) in the attention and scan kernels assumes that a wave's LDS reads return in the order
    they were issued, also when transposing 8-byte reads and 16-byte reads alternate.  1024 workgroups of four waves
    (four per compute unit, all hammering LDS) run 200 rounds of six interleavings of eight reads with the partial waits
    an in-order LDS allows; each result is compared with the same read done alone behind a full wait."""
    out = torch.zeros(7, dtype=torch.int32, device=dev)
    wgs, iters = 1024, 200
    _lib.check(lib.spinf_diag_lds_order(iters, wgs, out.data_ptr(), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "spinf_diag_lds_order")
    torch.cuda.synchronize()
    got = out.cpu().tolist()
    assert got[6] == wgs, got
    assert got[:6] == [0] * 6, f"LDS reads returned out of order: mismatches per interleaving {got[:6]} of {wgs * 256 * iters * 8} reads each"
