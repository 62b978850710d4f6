"""The mask side of the attention boundary: what Scorer._init_flex / Scorer._block_masks build per forward
(spinf_serve/scorer.py:163-238), as an opaque handle the attention op understands.

A TreeMask holds the stream's art / end / pos on the device and, instead of FlexAttention's nb x nb block tables
(spinf_serve/packer.py:426-491), a compact per-query-tile list of visible key tiles compiled on the host by the
library's tile-plan compiler.  No dense mask is built anywhere.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib


@dataclass
class TilePlan:
    """host arrays of a compiled plan (see include/spinf_tree.h)"""

    qt_ptr: np.ndarray
    kv_idx: np.ndarray
    kv_bits: np.ndarray
    order: np.ndarray
    n: int
    window: int
    active_blocks: int
    masked_blocks: int

    @classmethod
    def build(cls, art, end, pos, window=None) -> "TilePlan":
        lib = _lib.load_library()
        art = np.ascontiguousarray(art, np.int32)
        end = np.ascontiguousarray(end, np.int32)
        pos = np.ascontiguousarray(pos, np.int32)
        n = len(art)
        if len(end) != n or len(pos) != n:
            raise ValueError("art, end and pos differ in length")
        w = int(window) if window else 0
        h = C.c_void_p()
        _lib.check(lib.spinf_tileplan_build(art.ctypes.data, end.ctypes.data, pos.ctypes.data, n, w, C.byref(h)), "tileplan_build")
        try:
            counts = (C.c_int64 * 5)()
            _lib.check(lib.spinf_tileplan_counts(h, counts), "tileplan_counts")
            nqt, nent = int(counts[0]), int(counts[1])
            qt_ptr = np.zeros(nqt + 1, np.int32)
            kv_idx = np.zeros(max(nent, 1), np.int32)
            kv_bits = np.zeros(max(nent, 1), np.uint32)
            order = np.zeros(max(nqt, 1), np.int32)
            _lib.check(lib.spinf_tileplan_export(h, qt_ptr.ctypes.data, kv_idx.ctypes.data, kv_bits.ctypes.data, order.ctypes.data), "tileplan_export")
        finally:
            lib.spinf_tileplan_free(h)
        return cls(qt_ptr, kv_idx[:nent], kv_bits[:nent], order[:nqt], n, w, int(counts[2]), int(counts[3]))

    @property
    def n_qtiles(self) -> int:
        return len(self.order)


def _upload(a, dtype, device):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(a, dtype))
    if device.type == "cuda":
        t = t.pin_memory().to(device, non_blocking=True)
    return t


class TreeMask:
    """Device-side handle: the stream's metadata + one compiled plan.  ``seq_lengths`` mirrors BlockMask.seq_lengths
    (spinf_serve/models/qwen35/qwen.py:615 reads it)."""

    def __init__(self, plan: TilePlan, meta, device):
        self.plan = plan
        self.n = plan.n
        self.window = plan.window
        self.seq_lengths = (plan.n, plan.n)
        self.device = device
        self.art, self.end, self.pos = meta
        one = np.zeros(1, np.int32)
        self.qt_ptr = _upload(plan.qt_ptr, np.int32, device)
        self.kv_idx = _upload(plan.kv_idx if len(plan.kv_idx) else one, np.int32, device)
        self.kv_bits = _upload((plan.kv_bits if len(plan.kv_bits) else one.view(np.uint32)).view(np.int32), np.int32, device)
        self.order = _upload(plan.order if len(plan.order) else one, np.int32, device)

    @classmethod
    def build(cls, art, end, pos, window=None, device="cuda", meta=None):
        """compile the plan on the host and upload it; ``meta``: device art / end / pos tensors to share with another mask"""
        import torch

        device = torch.device(device)
        if meta is None:
            meta = tuple(_upload(a, np.int32, device) for a in (art, end, pos))
        return cls(TilePlan.build(art, end, pos, window), meta, device)


def block_masks(batch, sliding_window=None, device="cuda"):
    """-> {"full_attention": TreeMask, "sliding_attention": TreeMask}: the dict Scorer._block_masks returns
    (spinf_serve/scorer.py:207-238).  With a window the sliding plan is always built (the reference's always_window,
    spinf_serve/packer.py:448-450); without one both keys name the global mask."""
    full = TreeMask.build(batch.art, batch.end, batch.pos, None, device)
    if not sliding_window:
        return {"full_attention": full, "sliding_attention": full}
    slid = TreeMask.build(batch.art, batch.end, batch.pos, sliding_window, device, meta=(full.art, full.end, full.pos))
    return {"full_attention": full, "sliding_attention": slid}
