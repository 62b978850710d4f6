"""The extraction decoder's attention step ("x_decode", spinf_serve/decode.py:71-104) restated in numpy float64.

One decoding step for the Q = slots x beams queries of each of G groups: a query attends to its group's prefix (where the
stored position is not padding), to its own slot's template tokens and to the tokens its own beam has generated up to the
current step; sliding layers also hide prefix / template keys that lie a window or more behind the query.  One softmax over
the three key ranges together (decode.py:96).  The reference rounds scores and probabilities to bf16 on the way (its bf16
einsums); this restatement does not, the parity bar is a tolerance.

Test infrastructure only (see oracle/__init__.py).  Pinned in tests/test_xdecode.py against torch's
scaled_dot_product_attention with the explicit mask over the concatenated keys, and against oracle/attention.py's tree
attention: a beam's step equals the last row of causal attention over prefix | template | generated tokens.
"""

from __future__ import annotations

import numpy as np


def template_mask(own_t, Q: int, beam: int):
    """[G, Q, Tt] bool: template token j of a group is visible to the queries of the slot that owns it (decode.py:161-162)"""
    qj = np.arange(Q) // beam
    own_t = np.asarray(own_t)
    return (own_t[:, None, :] == qj[None, :, None]) & (own_t[:, None, :] >= 0)


def x_attention(q, kp, vp, pos_p, kt, vt, pos_t, own_t, gk, gv, qpos, step: int, beam: int, scale: float, window=None, softcap=None):
    """q [G, H, Q, d]; kp, vp [G, h, Lp, d]; pos_p [G, Lp]; kt, vt [G, h, Tt, d]; pos_t, own_t [G, Tt]; gk, gv [G, h, Q, S, d];
    qpos [G, Q] -> [G, Q, H, d] float64"""
    q = np.asarray(q, np.float64)
    kp, vp, kt, vt, gk, gv = (np.asarray(x, np.float64) for x in (kp, vp, kt, vt, gk, gv))
    pos_p, pos_t, qpos = np.asarray(pos_p), np.asarray(pos_t), np.asarray(qpos)
    G, H, Q, d = q.shape
    h, S = kp.shape[1], gk.shape[3]
    r = H // h
    qq = q.reshape(G, h, r, Q, d)
    sp = np.einsum("ghrqd,ghkd->ghrqk", qq, kp) * scale      # decode.py:83
    st = np.einsum("ghrqd,ghkd->ghrqk", qq, kt) * scale      # :84
    sg = np.einsum("ghrqd,ghqsd->ghrqs", qq, gk) * scale     # :85
    if softcap:
        sp, st, sg = (np.tanh(x / softcap) * softcap for x in (sp, st, sg))   # :86-87
    mp = np.broadcast_to((pos_p >= 0)[:, None, :], (G, Q, pos_p.shape[1]))   # :152
    mt = template_mask(own_t, Q, beam)
    if window is not None:   # :88-89
        mp = mp & ((qpos[:, :, None] - pos_p[:, None, :]) < window)
        mt = mt & ((qpos[:, :, None] - pos_t[:, None, :]) < window)
    mg = np.broadcast_to(np.arange(S) <= step, (G, Q, S))    # :92
    s = np.concatenate([sp, st, sg], -1)
    m = np.concatenate([mp, mt, mg], -1)[:, None, None]
    s = np.where(m, s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    a = np.exp(s)
    a /= a.sum(-1, keepdims=True)
    Lp, Lt = sp.shape[-1], st.shape[-1]
    out = np.einsum("ghrqk,ghkd->ghrqd", a[..., :Lp], vp)
    out += np.einsum("ghrqk,ghkd->ghrqd", a[..., Lp : Lp + Lt], vt)
    out += np.einsum("ghrqs,ghqsd->ghrqd", a[..., Lp + Lt :], gv)
    return out.reshape(G, H, Q, d).transpose(0, 2, 1, 3)
