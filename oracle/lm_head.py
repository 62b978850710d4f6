"""The lm head's read-out after the logits GEMM, restated in numpy float64: final soft-capping, log-softmax over the vocabulary,
column selection (spinf_serve/scorer.py:351-353 and :254).

Test infrastructure only (see oracle/__init__.py).  Pinned in tests/test_lm_head.py against torch.tanh / torch.log_softmax.
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
