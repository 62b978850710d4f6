"""Gated delta rule: token-by-token recurrence, chunked (WY) form and the scan over a packed token tree.

recurrent  restates the definition at spinf_serve/models/qwen35/gdn.py:176-186 (per value head, state S [K, V]):
               S <- exp(g_t) S ; d = beta_t (v_t - S^T k_t) ; S <- S + k_t d^T ; o_t = S^T (scale q_t)
           value head hv reads query/key head hv // (HV // H)                                  (gdn.py:167)
chunked    the chunk-64 WY form that flash-linear-attention 0.5.2 implements and gdn.py:109-133 glues together
           (third-party source absent from /root/reference; published algorithm restated, pinned by == recurrent)
tree_scan  every token continues from the state left by its path predecessor ``prev`` (qwen.py:550-590 runs the
           same thing level by level; docs/QWEN.md:51-52 states the fork identity this reproduces)

Test infrastructure only (see oracle/__init__.py).
"""

from __future__ import annotations

import numpy as np


def recurrent(q, k, v, g, beta, scale=None, h0=None, dtype=np.float64):
    """q,k [T,H,K]  v [T,HV,V]  g,beta [T,HV]  h0 [HV,K,V] or None -> (o [T,HV,V], final state [HV,K,V])."""
    q = np.asarray(q, dtype); k = np.asarray(k, dtype); v = np.asarray(v, dtype)
    g = np.asarray(g, dtype); beta = np.asarray(beta, dtype)
    T, H, K = k.shape
    HV, V = v.shape[1], v.shape[2]
    rep = HV // H
    scale = K ** -0.5 if scale is None else scale
    S = np.zeros((HV, K, V), dtype) if h0 is None else np.array(h0, dtype)
    o = np.zeros((T, HV, V), dtype)
    for t in range(T):
        kt = np.repeat(k[t], rep, axis=0)            # [HV, K]
        qt = np.repeat(q[t], rep, axis=0) * dtype(scale)
        S = S * np.exp(g[t])[:, None, None]
        d = (v[t] - np.einsum("hkv,hk->hv", S, kt)) * beta[t][:, None]
        S = S + kt[:, :, None] * d[:, None, :]
        o[t] = np.einsum("hkv,hk->hv", S, qt)
    return o, S


def chunked(q, k, v, g, beta, scale=None, h0=None, chunk=64, dtype=np.float64):
    """Same function as ``recurrent`` by the WY representation, one chunk of ``chunk`` tokens at a time."""
    q = np.asarray(q, dtype); k = np.asarray(k, dtype); v = np.asarray(v, dtype)
    g = np.asarray(g, dtype); beta = np.asarray(beta, dtype)
    T, H, K = k.shape
    HV, V = v.shape[1], v.shape[2]
    rep = HV // H
    scale = K ** -0.5 if scale is None else scale
    S = np.zeros((HV, K, V), dtype) if h0 is None else np.array(h0, dtype)
    o = np.zeros((T, HV, V), dtype)
    for c0 in range(0, T, chunk):
        c1 = min(c0 + chunk, T)
        L = c1 - c0
        for hv in range(HV):
            h = hv // rep
            kc, qc, vc = k[c0:c1, h], q[c0:c1, h] * dtype(scale), v[c0:c1, hv]
            G = np.cumsum(g[c0:c1, hv])
            b = beta[c0:c1, hv]
            Dm = np.exp(G[:, None] - G[None, :])                    # decay from j to i
            A = -np.tril((b[:, None] * (kc @ kc.T)) * Dm, -1)       # strictly lower
            Tm = np.linalg.inv(np.eye(L, dtype=dtype) - A)
            U = Tm @ (b[:, None] * vc)
            W = Tm @ (b[:, None] * kc * np.exp(G)[:, None])
            Vn = U - W @ S[hv]
            o[c0:c1, hv] = (qc * np.exp(G)[:, None]) @ S[hv] + np.tril((qc @ kc.T) * Dm) @ Vn
            S[hv] = np.exp(G[-1]) * S[hv] + (kc * np.exp(G[-1] - G)[:, None]).T @ Vn
    return o, S


def tree_scan(q, k, v, g, beta, prev, real, scale=None, dtype=np.float64, keep=None):
    """Scan along the paths of a packed tree: token i starts from the state after prev[i] (zero when prev[i] < 0).
    Pads (real False) produce zeros.  Returns o [T,HV,V]; with ``keep`` (iterable of positions) also {pos: state}."""
    q = np.asarray(q, dtype); k = np.asarray(k, dtype); v = np.asarray(v, dtype)
    g = np.asarray(g, dtype); beta = np.asarray(beta, dtype)
    T, H, K = k.shape
    HV, V = v.shape[1], v.shape[2]
    rep = HV // H
    scale = K ** -0.5 if scale is None else scale
    prev = np.asarray(prev)
    nchild = np.bincount(prev[prev >= 0], minlength=T)
    o = np.zeros((T, HV, V), dtype)
    states = {}
    left = nchild.copy()
    keep = set() if keep is None else set(int(x) for x in keep)
    kept = {}
    for t in range(T):
        if not real[t]:
            continue
        p = int(prev[t])
        if p < 0:
            S = np.zeros((HV, K, V), dtype)
        else:
            S = states[p]
            left[p] -= 1
            S = S.copy() if (left[p] > 0 or p in keep) else states.pop(p)
        kt = np.repeat(k[t], rep, axis=0)
        qt = np.repeat(q[t], rep, axis=0) * dtype(scale)
        S *= np.exp(g[t])[:, None, None]
        d = (v[t] - np.einsum("hkv,hk->hv", S, kt)) * beta[t][:, None]
        S += kt[:, :, None] * d[:, None, :]
        o[t] = np.einsum("hkv,hk->hv", S, qt)
        if nchild[t] > 0 or t in keep:
            states[t] = S
        if t in keep:
            kept[t] = S.copy()
    return (o, kept) if keep else o
