"""Dense masked-softmax attention over a packed stream: what the reference's attention op computes
(spinf_serve/models/gemma4.py:98-119 and spinf_serve/models/qwen35/qwen.py:604-623 call torch's flex_attention with
the mask of spinf_serve/scorer.py:173-177; GQA: query head h reads kv head h // (Hq // Hkv)).

out[q, h] = sum_k softmax_k(scale * <Q[q,h], K[k,kvh]> over visible k) * V[k, kvh]

Test infrastructure only (see oracle/__init__.py).
"""

from __future__ import annotations

import numpy as np

from .mask import dense_tree_mask


def masked_attention(q, k, v, mask, scale, dtype=np.float64):
    """q [n, Hq, D], k/v [n, Hkv, D], mask [n, n] bool -> out [n, Hq, D] in ``dtype``."""
    q = np.asarray(q, dtype)
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    n, hq, d = q.shape
    hkv = k.shape[1]
    g = hq // hkv
    out = np.empty((n, hq, d), dtype)
    neg = np.where(mask, 0.0, -np.inf).astype(dtype)
    for h in range(hq):
        kh = h // g
        s = (q[:, h] @ k[:, kh].T) * dtype(scale) + neg
        s -= s.max(1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(1, keepdims=True)
        out[:, h] = p @ v[:, kh]
    return out


def tree_attention(q, k, v, art, end, pos=None, window=None, scale=None, dtype=np.float64, spans=None):
    """Attention under the tree mask.  ``spans`` (list of (start, stop)) evaluates the dense mask per span of the stream
    instead of over the whole stream (jobs never see each other, so a job-aligned split changes nothing); rows outside
    every span (pads between jobs) attend to themselves only, i.e. return their own V row."""
    q = np.asarray(q)
    n, hq, d = q.shape
    scale = d ** -0.5 if scale is None else scale
    if spans is None:
        return masked_attention(q, k, v, dense_tree_mask(art, end, pos, window), scale, dtype)
    hkv = np.asarray(k).shape[1]
    g = hq // hkv
    out = np.repeat(np.asarray(v, dtype), g, axis=1)  # a lone pad row attends to itself: softmax over one key = V row
    for a, b in spans:
        m = dense_tree_mask(np.asarray(art)[a:b], np.asarray(end)[a:b] - a,
                            None if pos is None else np.asarray(pos)[a:b], window)
        out[a:b] = masked_attention(q[a:b], k[a:b], v[a:b], m, scale, dtype)
    return out


def job_spans(art):
    """Maximal runs [start, stop) that hold one job's tokens and the pads inside it (aligned gaps)."""
    art = np.asarray(art)
    spans = []
    real = np.flatnonzero(art >= 0)
    if not len(real):
        return spans
    for a in np.unique(art[real]):
        idx = np.flatnonzero(art == a)
        spans.append((int(idx[0]), int(idx[-1]) + 1))
    return spans
