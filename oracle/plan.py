"""Segments and levels of a packed token tree for the recurrent layers (restates the "indexed" path of
spinf_serve/models/qwen35/qwen.py:158-276).

A segment starts at a real token whose path predecessor is not the previous stream token, or is missing, or has
several children (qwen.py:185-187); it runs to the next start or pad.  Segments are grouped by depth; a segment with
children keeps its final state in a slot of its level (qwen.py:220-223); each level splits into a "chunked" call
(segments longer than ``short``) and a "recurrent" call (the rest) (qwen.py:224), a chunked call is cut at
``call_tokens`` (qwen.py:228-236).

Test infrastructure only (see oracle/__init__.py).
"""

from __future__ import annotations

import numpy as np


def segments(prev, real):
    """-> (starts [n], lens [n], parent segment [n] (-1 none), depth [n], has_kids [n], seg id per token [T])."""
    prev = np.asarray(prev, np.int64)
    real = np.asarray(real, bool)
    T = len(prev)
    nchild = np.bincount(prev[prev >= 0], minlength=T)
    starts = []
    seg = np.full(T, -1, np.int64)
    for i in range(T):
        if not real[i]:
            continue
        p = prev[i]
        if p != i - 1 or p < 0 or nchild[p] > 1:
            starts.append(i)
        seg[i] = len(starts) - 1
    starts = np.array(starts, np.int64)
    n = len(starts)
    lens = np.bincount(seg[real], minlength=n).astype(np.int64) if n else np.zeros(0, np.int64)
    parent = np.array([seg[prev[s]] if prev[s] >= 0 else -1 for s in starts], np.int64)
    depth = np.zeros(n, np.int64)
    for s in range(n):
        if parent[s] >= 0:
            depth[s] = depth[parent[s]] + 1
    kids = np.zeros(n, bool)
    kids[parent[parent >= 0]] = True
    return starts, lens, parent, depth, kids, seg


def tree_plan(prev, real, short=64, call_tokens=8192, keep=None):
    """-> list of levels; a level is a list of calls; a call is a dict
    {kind, idx (token positions, segments back to back), cu (cumulative lengths), h0_idx, ht_idx}; plus n_keep per level."""
    starts, lens, parent, depth, kids, seg = segments(prev, real)
    if keep is not None:
        for s in keep:
            if real[s]:
                kids[seg[s]] = True
    n = len(starts)
    slot = np.full(n, -1, np.int64)
    levels, n_keep = [], []
    for d in range(int(depth.max()) + 1 if n else 0):
        segs = np.flatnonzero(depth == d)
        kept = segs[kids[segs]]
        slot[kept] = np.arange(len(kept))
        n_keep.append(len(kept))
        calls = []
        for kind, whole in (("chunked", segs[lens[segs] > short]), ("recurrent", segs[lens[segs] <= short])):
            if not len(whole):
                continue
            parts = [whole]
            if kind == "chunked" and lens[whole].sum() > call_tokens:
                parts, run, acc = [], [], 0
                for sg in whole:
                    if run and acc + lens[sg] > call_tokens:
                        parts.append(np.array(run)); run, acc = [], 0
                    run.append(sg); acc += lens[sg]
                parts.append(np.array(run))
            for part in parts:
                idx = np.concatenate([np.arange(starts[s], starts[s] + lens[s]) for s in part])
                cu = np.concatenate([[0], np.cumsum(lens[part])])
                h0 = None if d == 0 else np.where(parent[part] >= 0, slot[np.maximum(parent[part], 0)], -1)
                ht = np.where(kids[part], slot[part], -1) if kids[part].any() else None
                calls.append(dict(kind=kind, idx=idx, cu=cu, h0_idx=h0, ht_idx=ht))
        levels.append(calls)
    return levels, n_keep, dict(starts=starts, lens=lens, parent=parent, depth=depth, slot=slot, seg=seg)
