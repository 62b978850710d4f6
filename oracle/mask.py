"""The tree mask as a dense boolean matrix and its block classification.

dense_tree_mask restates the predicate of spinf_serve/scorer.py:173-177 (dense form: tests/test_packer.py:74-79);
block_classes restates the full / partial / none rule of spinf_serve/packer.py:426-491 for text-only streams.

Test infrastructure only (see oracle/__init__.py).
"""

from __future__ import annotations

import numpy as np

from .layout import BLOCK


def dense_tree_mask(art, end, pos=None, window=None, grp=None, grp_windowed=False):
    """visible[q, k]: token q attends to token k (scorer.py:173-177).  window: sliding layers add pos[q]-pos[k] < W.
    grp (scorer.py:184-198): the tokens of an image group also attend to each other both ways; past the window (full_img /
    sliding_img of a model with _vision_bidir_all), or with grp_windowed only within it (the other sliding_img)."""
    art = np.asarray(art)
    end = np.asarray(end)
    n = len(art)
    q = np.arange(n)[:, None]
    k = np.arange(n)[None, :]
    m = (k <= q) & (art[q] >= 0) & (art[k] == art[q]) & (q < end[k])
    m = m | (q == k)
    inw = None
    if window is not None:
        pos = np.asarray(pos).astype(np.int64)
        inw = pos[:, None] - pos[None, :] < window
        m = m & inw
    if grp is not None:
        grp = np.asarray(grp)
        same = (grp[:, None] == grp[None, :]) & (grp[:, None] >= 0)
        if grp_windowed and inw is not None:
            same = same & inw
        m = m | same
    return m


def ancestor_mask(prev, real):
    """The same relation derived independently: q sees k iff k lies on q's path (walk ``prev``); pads see themselves."""
    n = len(prev)
    m = np.eye(n, dtype=bool)
    for q in range(n):
        if not real[q]:
            continue
        j = int(prev[q])
        while j >= 0:
            m[q, j] = True
            j = int(prev[j])
    return m


def block_classes(art, end, pos, window=None, always_window=False, block=BLOCK):
    """-> (full, partial) boolean [nb, nb] for the global layers and, when the window binds, for the sliding layers
    (packer.py:470-490, text-only streams): full = every pair attends, partial = decided per element, neither = skipped."""
    art = np.asarray(art)
    end = np.asarray(end)
    pos = np.asarray(pos)
    n = len(art)
    nb = -(-n // block)
    if nb * block != n:
        padn = nb * block - n
        art = np.concatenate([art, np.full(padn, -1, art.dtype)])
        end = np.concatenate([end, np.full(padn, -1, end.dtype)])
        pos = np.concatenate([pos, np.zeros(padn, pos.dtype)])
    ab = art.reshape(nb, block)
    eb = end.reshape(nb, block)
    pb = pos.reshape(nb, block).astype(np.int64)
    realb = ab >= 0
    one = np.array([(r.min() == r.max()) and r.min() >= 0 for r in ab])
    jobs = [set(r.tolist()) - {-1} for r in ab]
    big = np.iinfo(np.int64).max
    min_pos = np.where(realb, pb, big).min(1)
    max_pos = np.where(realb, pb, -big).max(1)
    binding = window is not None and (always_window or int(pos.max()) >= window)
    out = []
    for windowed in ((False, True) if binding else (False,)):
        full = np.zeros((nb, nb), bool)
        part = np.zeros((nb, nb), bool)
        for i in range(nb):
            for j in range(i + 1):
                if windowed and j < i and min_pos[i] - max_pos[j] >= window:
                    continue
                if (j < i and one[i] and one[j] and ab[i, 0] == ab[j, 0] and eb[j].min() >= (i + 1) * block and not windowed):
                    full[i, j] = True
                elif j == i or ((jobs[i] & jobs[j]) and eb[j].max() > i * block):
                    part[i, j] = True
        out.append((full, part))
    return out[0], (out[1] if binding else None)
