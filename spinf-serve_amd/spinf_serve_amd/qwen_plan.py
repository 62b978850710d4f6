"""Recurrent-layer planning and the tree scan of the hybrid (Qwen) stack behind the reference's interface
(spinf_serve/models/qwen35/qwen.py: Call :125-135, TreePlan :137-155, tree_plan :158-276, gdn_tree / gdn_indexed :514-590).

The plan itself is compiled by the library's host C++ (spinf_gdn_plan_build, csrc/gdnplan.cpp): one pass over the stream gives
the segments and their depth, a counting sort the levels, and the calls are slices of flat arrays.  This module only wraps those
arrays into the reference's Call / TreePlan objects and drives the HIP kernels level by level, states read and written by index.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np
import torch

from . import _lib, gdn


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


_PATHS = {"indexed": 0, "levels": 1}


def _compile(prev, real, path, short, call_tokens, max_init, rows, keep):
    """-> the flat arrays of spinf_gdn_plan_export, as a dict of numpy arrays"""
    lib = _lib.load_library()
    keep = np.ascontiguousarray([] if keep is None else list(keep), np.int64)
    handle = C.c_void_p()
    _lib.check(lib.spinf_gdn_plan_build(prev.ctypes.data, real.ctypes.data, len(prev), _PATHS[path], int(short), int(call_tokens), int(max_init),
                                        -1 if rows is None else int(rows), keep.ctypes.data if len(keep) else None, len(keep), C.byref(handle)),
               "tree_plan")
    try:
        counts = (C.c_int64 * 6)()
        _lib.check(lib.spinf_gdn_plan_counts(handle, counts), "tree_plan")
        n_seg, n_lev, n_call, n_cseg, n_rows, n_conv = (int(c) for c in counts)
        shapes = dict(level_ptr=(n_lev + 1, np.int64), call_kind=(n_call, np.int32), call_keep=(n_call, np.int32), call_seg_ptr=(n_call + 1, np.int64),
                      call_row_ptr=(n_call + 1, np.int64), seg_len=(n_cseg, np.int64), h0_idx=(n_cseg, np.int64), ht_idx=(n_cseg, np.int64),
                      idx=(n_rows, np.int64), n_keep=(n_lev, np.int64), conv=(n_conv * 4, np.int64), seg_of_row=(n_conv, np.int64),
                      seg_level=(n_seg, np.int64), seg_slot=(n_seg, np.int64))
        out = {name: np.zeros(max(size, 1), dtype) for name, (size, dtype) in shapes.items()}
        _lib.check(lib.spinf_gdn_plan_export(handle, *(out[name].ctypes.data for name in shapes)), "tree_plan")
        out = {name: out[name][: shapes[name][0]] for name in shapes}
        out["n_segments"] = n_seg
        return out
    finally:
        lib.spinf_gdn_plan_free(handle)


def tree_plan(prev, real, device, max_init: int = 96, path: str = "indexed", short: int = 64, rows: int | None = None,
              keep=None, call_tokens: int = 8192) -> TreePlan:
    """prev[i] = token before i on its path (-1 none), real[i] = not a pad.  Arguments as the reference's tree_plan
    (qwen.py:158-174): rows = plan over compact rows (real tokens first), keep = positions whose segment must leave its
    final state, short / call_tokens = the indexed path's kernel choice and call size."""
    if path not in _PATHS:
        raise ValueError(f"tree_plan: unknown path {path!r}")
    prev = np.ascontiguousarray(prev, np.int64)
    real = np.ascontiguousarray(real, bool).view(np.uint8)
    if len(real) != len(prev):
        raise ValueError("tree_plan: prev and real differ in length")
    a = _compile(prev, real, path, short, call_tokens, max_init, rows, keep)
    dev = torch.device(device)

    def up(x):
        return torch.from_numpy(np.ascontiguousarray(x)).to(dev, non_blocking=True)

    indexed = path == "indexed"
    levels = []
    for d in range(len(a["level_ptr"]) - 1):
        calls = []
        for c in range(a["level_ptr"][d], a["level_ptr"][d + 1]):
            s0, s1 = a["call_seg_ptr"][c], a["call_seg_ptr"][c + 1]
            cu = torch.from_numpy(np.concatenate([[0], np.cumsum(a["seg_len"][s0:s1])]).astype(np.int64))
            idx = up(a["idx"][a["call_row_ptr"][c] : a["call_row_ptr"][c + 1]])
            starts = None if d == 0 else up(a["h0_idx"][s0:s1])
            if indexed:
                ends = up(a["ht_idx"][s0:s1]) if a["call_keep"][c] else None
                calls.append(Call(idx, cu.to(dev, non_blocking=True), cu, None, False, "chunked" if a["call_kind"][c] else "recurrent", starts, ends))
            else:
                calls.append(Call(idx, cu.to(dev, non_blocking=True), cu, starts, bool(a["call_keep"][c])))
        levels.append(calls)
    seg_of_row = a["seg_of_row"]
    sidx = up(np.flatnonzero(real)) if rows is not None else None
    return TreePlan(up(a["conv"].reshape(-1, 4)), levels, a["n_segments"], path, a["n_keep"].tolist() if indexed else None, rows, sidx, seg_of_row,
                    a["seg_level"], a["seg_slot"], pad_rows=up(np.flatnonzero(seg_of_row < 0)))


def _kept_state_requests(plan: TreePlan, cap):
    """cap["state"] = [(row, name)]: the final state of the segment that holds `row` -> {level: [(slot, name)]}"""
    by_level = {}
    for row, name in cap["state"]:
        sg = int(plan.seg_of_row[row])
        slot = int(plan.seg_slot[sg]) if sg >= 0 else -1
        if slot < 0:
            raise RuntimeError(f"gdn_tree: no kept state for row {row} (segment {sg}, slot {slot})")
        by_level.setdefault(int(plan.seg_level[sg]), []).append((slot, name))
    return by_level


@torch.compiler.disable
def gdn_tree(q, k, v, g, beta, plan: TreePlan, mod=None):
    """q, k [T, Hk, Dk] (l2-normalised), v [T, Hv, Dv], g, beta [T, Hv] -> o [T, Hv, Dv]: every segment starts from its
    parent's final state (spinf_serve/models/qwen35/qwen.py:514-590).  Both kernels index the stream rows themselves, so a level
    costs at most two launches and no gathers.

    Capture (extraction, qwen.py:520-526,558-565): with plan.cap = {"tok": [(first row, rows, name)], "state": [(row, name)],
    "out": {"gdn": {}, "state": {}}} the layer's scan inputs of the row ranges and the final states of the named rows' segments
    are kept under out[...][name][layer]."""
    cap = plan.cap
    layer = mod.li if mod is not None else -1
    wanted = {}
    if cap is not None:
        for first, count, name in cap["tok"]:
            rows = slice(first, first + count)
            cap["out"]["gdn"].setdefault(name, {})[layer] = (q[rows].clone(), k[rows].clone(), v[rows].clone(), g[rows].clone(), beta[rows].clone())
        wanted = _kept_state_requests(plan, cap)
    scale = q.shape[-1] ** -0.5
    if plan.pad_rows is not None and len(plan.seg_of_row) == v.shape[0]:
        o = torch.empty_like(v)      # every covered row is written by a kernel; only the pads need the zero fill
        if plan.pad_rows.numel():
            o.index_fill_(0, plan.pad_rows, 0)
    else:
        o = torch.zeros_like(v)
    g32 = g if g.dtype == torch.float32 else g.float()
    b16 = beta if beta.dtype == torch.bfloat16 else beta.to(torch.bfloat16)
    indexed = plan.path == "indexed"
    above = None   # the states the level above left
    for d, calls in enumerate(plan.levels):
        n_slots = plan.n_keep[d] if indexed else sum(len(c.cu_cpu) - 1 for c in calls if c.keep)
        states = q.new_empty((n_slots, v.shape[1], q.shape[-1], v.shape[-1]), dtype=torch.float32) if n_slots else None
        next_slot = 0
        for c in calls:
            n_seg = len(c.cu_cpu) - 1
            if indexed:
                h0_idx, ht_idx, kind = c.h0_idx, c.ht_idx, c.kind
            else:   # levels path: a keeping call's segments take the next slots in order
                h0_idx = c.parent
                ht_idx = torch.arange(next_slot, next_slot + n_seg, device=q.device) if c.keep else None
                next_slot += n_seg if c.keep else 0
                kind = "chunked" if int((c.cu_cpu[1:] - c.cu_cpu[:-1]).max()) > 64 else "recurrent"
            kw = dict(h0=above if h0_idx is not None else None, h0_idx=h0_idx, ht=states if ht_idx is not None else None, ht_idx=ht_idx, idx=c.idx, o=o[None])
            if kind == "recurrent":
                gdn.recurrent(q[None], k[None], v[None], g32[None], b16[None], scale, c.cu, n_seg, **kw)
            else:
                gdn.chunked(q[None], k[None], v[None], g32[None], b16[None], scale, c.cu, c.cu_cpu, **kw)
        for slot, name in wanted.get(d, ()):
            cap["out"]["state"].setdefault(name, {})[layer] = states[slot].clone()
        above = states
    return o
