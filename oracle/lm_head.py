"""The lm head's read-out restated in numpy float64: row gather and logits GEMM (spinf_serve/scorer.py:247-250, :345-350), final
soft-capping, log-softmax over the vocabulary, column selection (scorer.py:351-353 and :254).

Test infrastructure only (see oracle/__init__.py).  Pinned in tests/test_lm_head.py against torch.tanh / torch.log_softmax, and the
GEMM modes against torch's own matmul on the CPU (float64, and bf16 tensors for the bf16 mode).
"""

from __future__ import annotations

import numpy as np


def logprobs(logits, cols=None, softcap=None):
    """logits [rows, vocab] -> log_softmax(softcap * tanh(logits / softcap)) [rows, vocab or len(cols)], float64"""
    x = np.asarray(logits, np.float64)
    if softcap:
        x = np.tanh(x / softcap) * softcap
    m = x.max(1, keepdims=True)
    lp = x - m - np.log(np.exp(x - m).sum(1, keepdims=True))
    return lp if cols is None else lp[:, np.asarray(cols)]


def round_bf16(x):
    """float values rounded to bfloat16 (nearest, ties to even), returned as float64"""
    b = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    b = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16
    return b.astype(np.uint32).view(np.float32).astype(np.float64)


def head_logprobs(h, w, sel=None, cols=None, softcap=None, bf16_logits=False):
    """h [*, hidden], w [vocab, hidden]: arrays of bf16 values -> log_softmax(cap(h[sel] @ w.T))[:, cols], float64.
    bf16_logits: the reference's default mode (scorer.py:349-352): `h @ W.t()` on bf16 tensors gives bf16 logits, and the division,
    the tanh and the multiplication of the soft-capping each round to bf16 again; log_softmax then runs on the float copy."""
    h = np.asarray(h, np.float64)
    x = (h if sel is None else h[np.asarray(sel)]) @ np.asarray(w, np.float64).T
    if not bf16_logits:
        return logprobs(x, cols, softcap)
    x = round_bf16(x)
    if softcap:
        x = round_bf16(round_bf16(np.tanh(round_bf16(x / softcap))) * softcap)
    return logprobs(x, cols, None)
