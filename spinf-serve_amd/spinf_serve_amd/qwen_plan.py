"""Recurrent-layer planning and the tree scan of the hybrid (Qwen) stack, with the reference's interface
(spinf_serve/models/qwen35/qwen.py: Call :125-135, TreePlan :137-155, tree_plan :158-276, gdn_tree / gdn_indexed :514-590).

tree_plan is host numpy: segments (maximal runs along ``prev`` between forks), their levels, and per level the calls
that run them; gdn_tree drives the HIP kernels level by level, states read and written by index.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from . import gdn


@dataclass
class Call:
    idx: object            # [n] int64 rows of the call's segments, back to back (device)
    cu: object             # [segs + 1] int64 cumulative lengths (device)
    cu_cpu: object         # the same on the host
    parent: object | None  # levels path: [segs] rows of the previous level's kept states, or None (roots)
    keep: bool             # levels path: leave the final states (segments with children)
    kind: str = "chunked"  # indexed path: chunked | recurrent
    h0_idx: object | None = None   # [segs] slot in the previous level's states (-1 zero); None at level 0
    ht_idx: object | None = None   # [segs] slot in this level's states (-1 none); None when nothing is kept


@dataclass
class TreePlan:
    conv: object           # [T, 4] int64: path predecessors 3, 2, 1 back and the token itself; T = "none" (a zero row)
    levels: list
    n_segments: int
    path: str = "levels"
    n_keep: list | None = None
    rows: int | None = None
    sidx: object | None = None
    seg_of_row: object | None = None
    seg_level: object | None = None
    seg_slot: object | None = None
    cap: dict | None = None
    pad_rows: object | None = None   # [pads] int64 (device): rows of the tensors no segment covers; their outputs are zero


def _segments(prev, real):
    T = len(prev)
    prev = np.asarray(prev, np.int64)
    has = prev >= 0
    fanout = np.bincount(prev[has], minlength=T)
    pclip = np.where(has, prev, 0)
    head = real & (~has | (prev != np.arange(T) - 1) | (fanout[pclip] > 1))
    starts = np.flatnonzero(head)
    seg = np.where(real, np.cumsum(head) - 1, -1)
    n = len(starts)
    lens = np.bincount(seg[real], minlength=n) if n else np.zeros(0, np.int64)
    parent = np.where(prev[starts] >= 0, seg[np.maximum(prev[starts], 0)], -1) if n else np.zeros(0, np.int64)
    return starts, lens.astype(np.int64), parent.astype(np.int64), seg


def _depth_exact(parent):
    """levels of the segment tree; parents precede their children in the stream"""
    d = np.zeros(len(parent), np.int64)
    for s, pa in enumerate(parent):
        if pa >= 0:
            d[s] = d[pa] + 1
    return d


def tree_plan(prev, real, device, max_init: int = 96, path: str = "indexed", short: int = 64, rows: int | None = None,
              keep=None, call_tokens: int = 8192) -> TreePlan:
    """prev[i] = token before i on its path (-1 none), real[i] = not a pad.  Arguments as the reference's tree_plan
    (qwen.py:158-174): rows = plan over compact rows (real tokens first), keep = positions whose segment must leave its
    final state, short / call_tokens = the indexed path's kernel choice and call size."""
    prev = np.asarray(prev, np.int64)
    real = np.asarray(real, bool)
    T = len(prev)
    real_idx = np.flatnonzero(real)
    to_row = None
    if rows is not None:
        if len(real_idx) > rows:
            raise ValueError(f"tree_plan: {len(real_idx)} real tokens do not fit {rows} compact rows")
        to_row = np.full(T + 1, rows, np.int64)
        to_row[real_idx] = np.arange(len(real_idx))
    starts, lens, parent, seg = _segments(prev, real)
    depth = _depth_exact(parent)
    n = len(starts)
    kids = np.zeros(n, bool)
    kids[parent[parent >= 0]] = True
    if keep is not None:
        for s in keep:
            if real[s]:
                kids[seg[s]] = True
    dev = torch.device(device)

    def put(x):
        return torch.from_numpy(np.ascontiguousarray(x)).to(dev, non_blocking=True)

    def rows_of(part):
        t = np.concatenate([np.arange(starts[s], starts[s] + lens[s]) for s in part])
        return t if to_row is None else to_row[t]

    levels, n_keep = [], []
    slot = np.full(n, -1, np.int64)
    for d in range(int(depth.max()) + 1 if n else 0):
        at = np.flatnonzero(depth == d)
        calls = []
        if path == "indexed":
            kept = at[kids[at]]
            slot[kept] = np.arange(len(kept))
            n_keep.append(len(kept))
            for kind, group in (("chunked", at[lens[at] > short]), ("recurrent", at[lens[at] <= short])):
                if not len(group):
                    continue
                parts = [group]
                if kind == "chunked" and int(lens[group].sum()) > call_tokens:
                    parts, run, acc = [], [], 0
                    for s in group:
                        if run and acc + lens[s] > call_tokens:
                            parts.append(np.asarray(run))
                            run, acc = [], 0
                        run.append(s)
                        acc += int(lens[s])
                    parts.append(np.asarray(run))
                for part in parts:
                    cu = torch.from_numpy(np.concatenate([[0], np.cumsum(lens[part])]))
                    h0 = None if d == 0 else put(np.where(parent[part] >= 0, slot[np.maximum(parent[part], 0)], -1))
                    ht = put(np.where(kids[part], slot[part], -1)) if kids[part].any() else None
                    calls.append(Call(put(rows_of(part)), cu.to(dev, non_blocking=True), cu, None, False, kind, h0, ht))
        elif path == "levels":
            for keepers in (True, False):
                group = at[kids[at] == keepers]
                if not len(group):
                    continue
                if keepers:
                    slot[group] = np.arange(len(group))
                step = len(group) if d == 0 else max_init
                for a in range(0, len(group), step):
                    part = group[a : a + step]
                    cu = torch.from_numpy(np.concatenate([[0], np.cumsum(lens[part])]))
                    par = None if d == 0 else put(slot[parent[part]])
                    calls.append(Call(put(rows_of(part)), cu.to(dev, non_blocking=True), cu, par, keepers))
        else:
            raise ValueError(f"tree_plan: unknown path {path!r}")
        levels.append(calls)
    # conv taps: 3 path predecessors and the token itself; T = none
    conv = np.empty((T, 4), np.int64)
    conv[:, 3] = np.arange(T)
    hop = np.where(real, prev, -1)
    for j in (2, 1, 0):
        conv[:, j] = np.where(hop >= 0, hop, T)
        hop = np.where(hop >= 0, prev[np.maximum(hop, 0)], -1)
    sidx, seg_rows = None, seg
    if to_row is not None:
        cc = np.full((rows, 4), rows, np.int64)
        cc[: len(real_idx)] = to_row[conv[real_idx]]
        conv = cc
        sidx = put(real_idx)
        seg_rows = np.full(rows, -1, np.int64)
        seg_rows[: len(real_idx)] = seg[real_idx]
    return TreePlan(put(conv), levels, n, path, n_keep if path == "indexed" else None, rows, sidx, seg_rows, depth, slot,
                    pad_rows=put(np.flatnonzero(seg_rows < 0)))


@torch.compiler.disable
def gdn_tree(q, k, v, g, beta, plan: TreePlan, mod=None):
    """q, k [T, Hk, Dk] (l2-normalised), v [T, Hv, Dv], g, beta [T, Hv] -> o [T, Hv, Dv]: every segment starts from its
    parent's final state (spinf_serve/models/qwen35/qwen.py:514-590).  Both kernels index the stream rows themselves, so a level
    costs at most two launches and no gathers."""
    cap = plan.cap
    li = mod.li if mod is not None else -1
    if cap is not None:
        for r0, n, name in cap["tok"]:
            cap["out"]["gdn"].setdefault(name, {})[li] = tuple(t[r0 : r0 + n].clone() for t in (q, k, v, g, beta))
    scale = q.shape[-1] ** -0.5
    if plan.pad_rows is not None and len(plan.seg_of_row) == v.shape[0]:
        o = torch.empty_like(v)      # every covered row is written by a kernel; only the pads need the zero fill
        if plan.pad_rows.numel():
            o.index_fill_(0, plan.pad_rows, 0)
    else:
        o = torch.zeros_like(v)
    g32 = g if g.dtype == torch.float32 else g.float()
    b16 = beta if beta.dtype == torch.bfloat16 else beta.to(torch.bfloat16)
    want = []
    if cap is not None:
        for row, name in cap["state"]:
            sg = int(plan.seg_of_row[row])
            lvl, sl = int(plan.seg_level[sg]), int(plan.seg_slot[sg])
            if sg < 0 or sl < 0:
                raise RuntimeError(f"gdn_tree: no kept state for row {row} (segment {sg}, slot {sl})")
            want.append((lvl, sl, name))
    indexed = plan.path == "indexed"
    prev_states = None
    for d, calls in enumerate(plan.levels):
        if indexed:
            nk = plan.n_keep[d]
        else:
            nk = sum(len(c.cu_cpu) - 1 for c in calls if c.keep)
        states = q.new_empty((nk, v.shape[1], q.shape[-1], v.shape[-1]), dtype=torch.float32) if nk else None
        base = 0
        for c in calls:
            nseg = len(c.cu_cpu) - 1
            if indexed:
                h0_idx, ht_idx, kind = c.h0_idx, c.ht_idx, c.kind
            else:
                h0_idx = c.parent
                ht_idx = torch.arange(base, base + nseg, device=q.device) if c.keep else None
                base += nseg if c.keep else 0
                kind = "chunked" if int((c.cu_cpu[1:] - c.cu_cpu[:-1]).max()) > 64 else "recurrent"
            kw = dict(h0=prev_states if h0_idx is not None else None, h0_idx=h0_idx,
                      ht=states if ht_idx is not None else None, ht_idx=ht_idx, idx=c.idx, o=o[None])
            if kind == "recurrent":
                gdn.recurrent(q[None], k[None], v[None], g32[None], b16[None], scale, c.cu, nseg, **kw)
            else:
                gdn.chunked(q[None], k[None], v[None], g32[None], b16[None], scale, c.cu, c.cu_cpu, **kw)
        for lvl, sl, name in want:
            if lvl == d:
                cap["out"]["state"].setdefault(name, {})[li] = states[sl].clone()
        prev_states = states
    return o
