"""The lm head's read-out (spinf_serve/scorer.py:247-261 and :340-355): row gather, logits GEMM, final soft-capping, log-softmax
over the vocabulary and the selection of the option columns, by the HIP kernels of libspinf_tree.so.  There is no CPU path.

    lp = lm_head_logprobs(Hf, sel, W, cols, softcap)               # the whole read-out in one pass: no logits matrix exists
    xlp = lm_head_logprobs(Hf, sel_x, W, None, softcap)            # [rows, vocab] fp32 (the extraction rows)

or, after a library GEMM,

    logits = torch.mm(h, W.t(), out_dtype=torch.float32)          # or h @ W.t() in bf16
    lp = lm_logprobs(logits, cols, softcap)                        # [rows, len(cols)] fp32
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
    (int64 device vector; negative = from the end, outside the vocabulary = NaN) or with cols None all of it"""
    if cols is not None:
        cols = torch.where(cols < 0, cols + logits.shape[1], cols)
    return _lm_op(logits, cols, float(softcap) if softcap else 0.0)


@torch.library.custom_op("spinf::lm_head_logprobs", mutates_args=())
def _head_op(h: torch.Tensor, sel: Optional[torch.Tensor], w: torch.Tensor, cols: Optional[torch.Tensor], softcap: float, bf16_logits: bool) -> torch.Tensor:
    if not (h.is_cuda and w.is_cuda):
        raise RuntimeError("spinf::lm_head_logprobs runs on ROCm device tensors only (no CPU path)")
    if h.dim() != 2 or w.dim() != 2 or h.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or h.stride(1) != 1 or w.stride(1) != 1:
        raise ValueError("h [*, hidden] and W [vocab, hidden] must be bf16 matrices with contiguous rows")
    if h.shape[1] != w.shape[1]:
        raise ValueError(f"hidden sizes differ: h {h.shape[1]}, W {w.shape[1]}")
    if sel is not None:
        if sel.dtype != torch.int64 or sel.dim() != 1:
            raise ValueError("sel must be an int64 vector")
        sel = sel.contiguous()
    if cols is not None:
        if cols.dtype != torch.int64 or cols.dim() != 1 or cols.numel() == 0:
            raise ValueError("cols must be a non-empty int64 vector")
        cols = cols.contiguous()
    rows, vocab = (h.shape[0] if sel is None else sel.numel()), w.shape[0]
    out = torch.empty((rows, vocab if cols is None else cols.numel()), dtype=torch.float32, device=h.device)
    a = _lib.LmHeadArgs()
    a.h, a.h_ld, a.rows, a.h_rows = h.data_ptr(), h.stride(0), rows, h.shape[0]
    a.sel = sel.data_ptr() if sel is not None else None
    a.w, a.w_ld, a.vocab, a.hidden = w.data_ptr(), w.stride(0), vocab, h.shape[1]
    a.softcap, a.logits_dtype = softcap, int(bf16_logits)
    if cols is not None:
        a.cols, a.n_cols = cols.data_ptr(), cols.numel()
    a.out, a.out_ld = out.data_ptr(), out.stride(0)
    lib = _lib.load_library()
    need = C.c_int64()
    _lib.check(lib.spinf_lm_head_workspace(C.byref(a), C.byref(need)), "spinf_lm_head_workspace")
    work = torch.empty(max(need.value, 8), dtype=torch.uint8, device=h.device)
    a.workspace, a.workspace_bytes = work.data_ptr(), work.numel()
    with torch.cuda.device(h.device):
        _lib.check(lib.spinf_lm_head_fwd(C.byref(a), C.c_void_p(torch.cuda.current_stream(h.device).cuda_stream)), "spinf_lm_head_fwd")
    return out


@_head_op.register_fake
def _(h, sel, w, cols, softcap, bf16_logits):
    rows = h.shape[0] if sel is None else sel.numel()
    return torch.empty((rows, w.shape[0] if cols is None else cols.numel()), dtype=torch.float32, device=h.device)


def lm_head_logprobs(h, sel, w, cols=None, softcap=None, logits="fp32"):
    """h [*, hidden] bf16 (the final hidden states), sel int64 device vector of the rows to read (None: all), w [vocab, hidden] bf16
    -> log_softmax(softcap * tanh(h[sel] @ w.T / softcap)) fp32, the columns ``cols`` of it or with cols None all of it.
    logits "fp32": the logits keep their fp32 accumulators (the reference's "f32out" / "fp32" modes); "bf16": rounded to bf16 and
    capped in bf16 steps, as the reference's `h @ W.t()` on bf16 tensors.  A negative column or row of ``sel`` counts from the end,
    as in torch indexing; a column outside the vocabulary gives NaN, an entry of ``sel`` outside h a whole row of NaN (where
    torch's indexing would raise: the list is a device tensor, and checking it on the host would cost a synchronisation)."""
    if logits not in ("fp32", "bf16"):
        raise ValueError(f"logits mode {logits!r}")
    if cols is not None:
        cols = torch.where(cols < 0, cols + w.shape[0], cols)
    return _head_op(h, sel, w, cols, float(softcap) if softcap else 0.0, logits == "bf16")
