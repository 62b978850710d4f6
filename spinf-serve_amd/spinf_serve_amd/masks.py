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

    def __init__(self, handle, qt_ptr, kv_idx, kv_bits, order, n, window, active_blocks, masked_blocks, grp_mode=0, ktile=64):
        self._handle = handle
        self.ktile = ktile
        self.qt_ptr, self.kv_idx, self.kv_bits, self.order = qt_ptr, kv_idx, kv_bits, order
        self.n, self.window, self.grp_mode = n, window, grp_mode
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
    def build(cls, art, end, pos, window=None, grp=None, grp_windowed=False, ktile=64) -> "TilePlan":
        """grp (image groups, spinf_serve/scorer.py:184-198): [n] int32, -1 none; the tokens of a group also see each other both
        ways, past the window unless grp_windowed.  ktile: keys per entry, 64, or 32 for the head dim 512 kernel."""
        lib = _lib.load_library()
        art = np.ascontiguousarray(art, np.int32)
        end = np.ascontiguousarray(end, np.int32)
        pos = np.ascontiguousarray(pos, np.int32)
        n = len(art)
        if len(end) != n or len(pos) != n:
            raise ValueError("art, end and pos differ in length")
        w = int(window) if window else 0
        h = C.c_void_p()
        mode = 0
        gptr = None
        if grp is not None:
            grp = np.ascontiguousarray(grp, np.int32)
            if len(grp) != n:
                raise ValueError("grp differs in length from art")
            mode = 2 if grp_windowed else 1
            gptr = grp.ctypes.data
        _lib.check(lib.spinf_tileplan_build_ktile(art.ctypes.data, end.ctypes.data, pos.ctypes.data, gptr, mode, n, w, int(ktile), C.byref(h)),
                   "tileplan_build")
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
        return cls(h, qt_ptr, kv_idx[:nent], kv_bits[:nent], order[:nqt], n, w, int(counts[2]), int(counts[3]), mode, int(ktile))

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

    def schedule_static(self, head_groups: int, n_lists: int):
        """-> (items [n_qtiles * head_groups, 4] int32, list_ptr [n_lists + 1] int32): the items dealt out to n_lists workgroups
        ahead of the launch (the kernel with decoupled waves)"""
        got = self._schedules.get((head_groups, n_lists))
        if got is None:
            items = np.zeros((max(self.n_qtiles * head_groups, 1), 4), np.int32)
            list_ptr = np.zeros(n_lists + 1, np.int32)
            _lib.check(_lib.load_library().spinf_tileplan_schedule_static(self._handle, head_groups, n_lists, items.ctypes.data, list_ptr.ctypes.data),
                       "tileplan_schedule_static")
            got = self._schedules[(head_groups, n_lists)] = (items[: self.n_qtiles * head_groups], list_ptr)
        return got


def _static_lists(device) -> int:
    """workgroups of a static schedule on this device: one per compute unit"""
    import torch

    return int(torch.cuda.get_device_properties(device).multi_processor_count)


def _upload(a, dtype, device):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(a, dtype))
    if device.type == "cuda":
        t = t.pin_memory().to(device, non_blocking=True)
    return t


class TreeMask:
    """Device-side handle: the stream's metadata + one compiled plan.  ``seq_lengths`` mirrors BlockMask.seq_lengths
    (spinf_serve/models/qwen35/qwen.py:615 reads it)."""

    def __init__(self, plan: TilePlan, meta, device, grp=None, host=None):
        self.plan = plan
        self._host = host                   # (art, end, pos, grp, grp_windowed) on the host, for a plan of another key-tile size
        self._other = None
        self.grp = grp                      # device copy of the image groups the plan was built with, or None
        self.grp_mode = plan.grp_mode if grp is not None else 0
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

    def for_head_dim(self, d: int, ring: bool = False) -> "TreeMask":
        """the mask with the plan granularity the kernel takes: 32-key entries at head dim 512 and for the kernel with decoupled
        waves (ring), 64-key ones otherwise (the second plan is compiled on first use and shares the device metadata)"""
        ktile = 32 if d == 512 or ring else 64
        if ktile == self.plan.ktile:
            return self
        if self._other is None:
            if self._host is None:
                raise ValueError(f"this mask was built for key tiles of {self.plan.ktile}; head dim {d} takes {ktile}")
            art, end, pos, grp, grp_windowed = self._host
            plan = TilePlan.build(art, end, pos, self.window, grp, grp_windowed, ktile)
            self._other = TreeMask(plan, (self.art, self.end, self.pos), self.device, self.grp)
            self._other._other = self
        return self._other

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
        kt = self.plan.ktile
        tiles = row_of[: (n + kt - 1) // kt * kt].view(-1, kt)
        run = (tiles - tiles[:, :1]) == torch.arange(kt, dtype=torch.int32, device=self.device)
        tile_row0 = torch.where((tiles[:, 0] >= 0) & run.all(1), tiles[:, 0], torch.full_like(tiles[:, 0], -1))
        kv_row0 = tile_row0[self.kv_idx.long()].contiguous()
        self._rows = (sidx, row_of[:n].contiguous(), kv_row0)
        return self._rows[1], self._rows[2]

    def schedule(self, head_groups: int, n_lists: int = 0):
        """device copy of the work lists for this many head groups (built on first use, then kept); n_lists > 0: the static
        schedule for that many workgroups"""
        got = self._sched.get((head_groups, n_lists))
        if got is None:
            items, list_ptr = self.plan.schedule_static(head_groups, n_lists) if n_lists else self.plan.schedule(head_groups)
            if not len(items):
                items = np.zeros((1, 4), np.int32)
            got = self._sched[(head_groups, n_lists)] = (_upload(items, np.int32, self.device), _upload(list_ptr, np.int32, self.device), self.plan.n_qtiles * head_groups)
        return got

    @classmethod
    def build(cls, art, end, pos, window=None, device="cuda", meta=None, grp=None, grp_windowed=False, grp_dev=None):
        """compile the plan on the host and upload it; ``meta``: device art / end / pos tensors to share with another mask;
        grp: image groups (see TilePlan.build), grp_dev: their device copy to share"""
        import torch

        device = torch.device(device)
        if meta is None:
            meta = tuple(_upload(a, np.int32, device) for a in (art, end, pos))
        if grp is not None and grp_dev is None:
            grp_dev = _upload(grp, np.int32, device)
        return cls(TilePlan.build(art, end, pos, window, grp, grp_windowed), meta, device, grp_dev if grp is not None else None,
                   host=(art, end, pos, grp, grp_windowed))


def block_masks(batch, sliding_window=None, device="cuda", grp=None, bidir_all=True):
    """-> {"full_attention": TreeMask, "sliding_attention": TreeMask}: the dict Scorer._block_masks returns
    (spinf_serve/scorer.py:207-238).  With a window the sliding plan is always built (the reference's always_window,
    spinf_serve/packer.py:448-450); without one both keys name the global mask.
    grp: image groups of the stream's tokens (-1 none).  bidir_all (the model's _vision_bidir_all, scorer.py:186-198): the
    tokens of an image see each other both ways on every layer and past the window; otherwise on the sliding layers only,
    within the window, and the global layers stay causal."""
    full = TreeMask.build(batch.art, batch.end, batch.pos, None, device, grp=grp if bidir_all else None)
    if not sliding_window:
        return {"full_attention": full, "sliding_attention": full}
    grp_dev = full.grp if grp is not None else None
    slid = TreeMask.build(batch.art, batch.end, batch.pos, sliding_window, device, meta=(full.art, full.end, full.pos), grp=grp,
                          grp_windowed=not bidir_all, grp_dev=grp_dev)
    return {"full_attention": full, "sliding_attention": slid}
