"""The lm head's read-out after the logits GEMM (spinf_serve/scorer.py:340-355, column selection :254): final soft-capping,
log-softmax over the vocabulary and the selection of the option columns in one HIP kernel of libspinf_tree.so, which reads
the logits once and writes only what is kept.  The GEMM itself stays a library GEMM.  There is no CPU path.

    logits = torch.mm(h, W.t(), out_dtype=torch.float32)          # or h @ W.t() in bf16
    lp = lm_logprobs(logits, cols, softcap)                        # [rows, len(cols)] fp32
    xlp = lm_logprobs(logits_x, None, softcap)                     # [rows, vocab] fp32 (the extraction rows)
"""

from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib


@torch.library.custom_op("spinf::lm_logprobs", mutates_args=())
def _lm_op(logits: torch.Tensor, cols: Optional[torch.Tensor], softcap: float) -> torch.Tensor:
    if not logits.is_cuda:
        raise RuntimeError("spinf::lm_logprobs runs on ROCm device tensors only (no CPU path)")
    if logits.dim() != 2 or logits.stride(1) != 1 or logits.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("logits must be a fp32 or bf16 matrix with contiguous rows")
    rows, vocab = logits.shape
    if cols is not None:
        if cols.dtype != torch.int64 or cols.dim() != 1 or cols.numel() == 0:
            raise ValueError("cols must be a non-empty int64 vector")
        cols = cols.contiguous()
    out = torch.empty((rows, vocab if cols is None else cols.numel()), dtype=torch.float32, device=logits.device)
    a = _lib.LmArgs()
    a.logits, a.ld, a.dtype = logits.data_ptr(), logits.stride(0), int(logits.dtype == torch.bfloat16)
    a.rows, a.vocab, a.softcap = rows, vocab, softcap
    if cols is not None:
        a.cols, a.n_cols = cols.data_ptr(), cols.numel()
    a.out, a.out_ld = out.data_ptr(), out.stride(0)
    lib = _lib.load_library()
    with torch.cuda.device(logits.device):
        _lib.check(lib.spinf_lm_logprobs(C.byref(a), C.c_void_p(torch.cuda.current_stream(logits.device).cuda_stream)), "spinf_lm_logprobs")
    return out


@_lm_op.register_fake
def _(logits, cols, softcap):
    return torch.empty((logits.shape[0], logits.shape[1] if cols is None else cols.numel()), dtype=torch.float32, device=logits.device)


def lm_logprobs(logits, cols=None, softcap=None):
    """logits [rows, vocab] fp32 / bf16 -> log_softmax(softcap * tanh(logits / softcap)) fp32, the columns ``cols`` of it
    (int64 device vector) or with cols None all of it"""
    return _lm_op(logits, cols, float(softcap) if softcap else 0.0)
