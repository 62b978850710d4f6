"""CPU baselines timed next to the GPU numbers: the reference's attention semantics run on the host cores with an explicit
dense boolean tree mask per content (the mask of spinf_serve/scorer.py:173-177 fed to torch's own CPU attention, which is what
the reference's flex path computes), and the fp32 token-by-token delta rule (spinf_serve/models/qwen35/gdn.py:176-186).

Test / measurement infrastructure only (see oracle/__init__.py): used by bench.py's cpu_baseline leg, never by the product.
"""

from __future__ import annotations

import time

import numpy as np

from .attention import job_spans
from .mask import dense_tree_mask


def attention_tokens_per_s(q, k, v, art, end, pos, scale, window=None, max_seconds=25.0, chunk_rows=2048):
    """q [n, hq, d], k / v [n, hkv, d] torch CPU tensors (any float dtype; computed in fp32).  Runs whole contents, one dense
    mask per content, until max_seconds is used up.  -> (real tokens per second, contents done, real tokens done, seconds, out)"""
    import torch
    import torch.nn.functional as F

    spans = job_spans(art)
    done_tok = done = 0
    t0 = time.perf_counter()
    outs = {}
    for a, b in spans:
        m = torch.from_numpy(dense_tree_mask(np.asarray(art)[a:b], np.asarray(end)[a:b] - a, np.asarray(pos)[a:b], window))
        qq = q[a:b].float().transpose(0, 1)[None]
        kk = k[a:b].float().transpose(0, 1)[None]
        vv = v[a:b].float().transpose(0, 1)[None]
        rows = []
        for r0 in range(0, b - a, chunk_rows):   # bound the score matrix of long contents
            r1 = min(b - a, r0 + chunk_rows)
            rows.append(F.scaled_dot_product_attention(qq[:, :, r0:r1], kk[:, :, :r1], vv[:, :, :r1], attn_mask=m[r0:r1, :r1], scale=scale, enable_gqa=True))
        outs[(a, b)] = torch.cat(rows, 2)[0].transpose(0, 1)
        done += 1
        done_tok += int((np.asarray(art)[a:b] >= 0).sum())
        if time.perf_counter() - t0 > max_seconds:
            break
    dt = time.perf_counter() - t0
    return done_tok / dt, done, done_tok, dt, outs


def gdn_tokens_per_s(q, k, v, g, beta, prev, real, max_tokens=4096, max_seconds=25.0):
    """fp32 token-by-token recurrence along ``prev`` on the first max_tokens stream tokens (torch CPU)."""
    import torch

    T = min(len(prev), max_tokens)
    H, K = k.shape[1], k.shape[2]
    HV, V = v.shape[1], v.shape[2]
    rep = HV // H
    scale = K ** -0.5
    states = {}
    nchild = np.bincount(prev[:T][prev[:T] >= 0], minlength=T)
    o = torch.zeros((T, HV, V))
    qf, kf, vf, gf, bf = (x[:T].float() for x in (q, k, v, g, beta))
    t0 = time.perf_counter()
    n = 0
    for t in range(T):
        if not real[t]:
            continue
        p = int(prev[t])
        S = torch.zeros((HV, K, V)) if p < 0 else (states[p].clone() if nchild[p] > 1 else states.pop(p))
        kt = kf[t].repeat_interleave(rep, 0)
        qt = qf[t].repeat_interleave(rep, 0) * scale
        S *= torch.exp(gf[t])[:, None, None]
        d = (vf[t] - torch.einsum("hkv,hk->hv", S, kt)) * bf[t][:, None]
        S += kt[:, :, None] * d[:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, qt)
        if nchild[t] > 0:
            states[t] = S
        n += 1
        if time.perf_counter() - t0 > max_seconds:
            break
    dt = time.perf_counter() - t0
    return n / dt, n, dt, o
