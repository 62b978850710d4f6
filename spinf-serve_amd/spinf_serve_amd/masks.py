"""The mask side of the attention boundary: what Scorer._init_flex / Scorer._block_masks build per forward
(spinf_serve/scorer.py:163-238), as an opaque handle the attention op understands.

A TreeMask holds the stream's art / end / pos on the device and, instead of FlexAttention's nb x nb block tables
(spinf_serve/packer.py:426-491), a compact per-query-tile list of visible key tiles compiled on the host by the
library's tile-plan compiler.  No dense mask is built anywhere.
"""

from __future__ import annotations

import ctypes as C
import numpy as np

from . import _lib


class TilePlan:
    """host arrays of a compiled plan (see include/spinf_tree.h) and the native handle that makes its work lists"""

    def __init__(self, handle, qt_ptr, kv_idx, kv_bits, order, n, window, active_blocks, masked_blocks):
        self._handle = handle
        self.qt_ptr, self.kv_idx, self.kv_bits, self.order = qt_ptr, kv_idx, kv_bits, order
        self.n, self.window = n, window
        self.active_blocks, self.masked_blocks = active_blocks, masked_blocks
        self._schedules = {}

    def __del__(self):
        h, self._handle = getattr(self, "_handle", None), None
        if h:
            try:
                _lib.load_library().spinf_tileplan_free(h)
            except Exception:  # noqa: BLE001  (interpreter shutdown)
                pass

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
        except Exception:
            lib.spinf_tileplan_free(h)
            raise
        return cls(h, qt_ptr, kv_idx[:nent], kv_bits[:nent], order[:nqt], n, w, int(counts[2]), int(counts[3]))

    @property
    def n_qtiles(self) -> int:
        return len(self.order)

    def schedule(self, head_groups: int):
        """-> (items [n_qtiles * head_groups, 4] int32, list_ptr [9] int32): the kernel's work lists"""
        got = self._schedules.get(head_groups)
        if got is None:
            items = np.zeros((max(self.n_qtiles * head_groups, 1), 4), np.int32)
            list_ptr = np.zeros(9, np.int32)
            _lib.check(_lib.load_library().spinf_tileplan_schedule(self._handle, head_groups, items.ctypes.data, list_ptr.ctypes.data), "tileplan_schedule")
            got = self._schedules[head_groups] = (items[: self.n_qtiles * head_groups], list_ptr)
        return got


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
        self.kv_idx = _upload(plan.kv_idx if len(plan.kv_idx) else one, np.int32, device)
        self.kv_bits = _upload((plan.kv_bits if len(plan.kv_bits) else one.view(np.uint32)).view(np.int32), np.int32, device)
        self._sched = {}
        self._rows = None

    def rows(self, sidx):
        """compact rows (spinf_serve/models/qwen35/qwen.py:613-622): sidx [R] = stream position of each real row (a device
        tensor) -> (row_of [n], kv_row0 [entries]) int32 device tensors for the kernel: the row of each stream position (-1:
        pad) and, per plan entry, the row of its first key where its 64 keys are consecutive rows (else -1).  Kept for the
        sidx tensor it was built from (one forward: every layer passes the same tensor)."""
        import torch

        if self._rows is not None and self._rows[0] is sidx:
            return self._rows[1], self._rows[2]
        n = self.n
        row_of = torch.full((n + 63,), -1, dtype=torch.int32, device=self.device)   # padded: every key tile is 64 long
        row_of[sidx.to(self.device, torch.long)] = torch.arange(sidx.shape[0], dtype=torch.int32, device=self.device)
        tiles = row_of[: (n + 63) // 64 * 64].view(-1, 64)
        run = (tiles - tiles[:, :1]) == torch.arange(64, dtype=torch.int32, device=self.device)
        tile_row0 = torch.where((tiles[:, 0] >= 0) & run.all(1), tiles[:, 0], torch.full_like(tiles[:, 0], -1))
        kv_row0 = tile_row0[self.kv_idx.long()].contiguous()
        self._rows = (sidx, row_of[:n].contiguous(), kv_row0)
        return self._rows[1], self._rows[2]

    def schedule(self, head_groups: int):
        """device copy of the work lists for this many head groups (built on first use, then kept)"""
        got = self._sched.get(head_groups)
        if got is None:
            items, list_ptr = self.plan.schedule(head_groups)
            if not len(items):
                items = np.zeros((1, 4), np.int32)
            got = self._sched[head_groups] = (_upload(items, np.int32, self.device), _upload(list_ptr, np.int32, self.device), self.plan.n_qtiles * head_groups)
        return got

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
