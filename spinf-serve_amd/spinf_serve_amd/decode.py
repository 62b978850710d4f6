"""The extraction decoder's attention step behind the reference's boundary (spinf_serve/decode.py:35-104).

  XCaches       the tensors of decode.Decoder that the attention reads (decode.py:129-171): prefix, template and generated K/V
                by layer, their positions and owners, the queries' positions, the current step
  GroupKV       the cache object transformers' layers write the new tokens' K/V into (decode.py:51-68)
  x_attention   the attention interface callable "x_decode" (decode.py:71-104): same signature, same result layout
  register      AttentionInterface.register("x_decode", x_attention) (decode.py:35-41)

A step is ONE launch of spinf_xdecode_attn_fwd in libspinf_tree.so (plus a small merge launch when the key stream is split
over workgroups): nothing is copied per slot or per beam, no mask tensor is built.  There is no CPU or PyTorch path.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Optional

import torch

from . import _lib

_CURRENT: list = [None]  # the caches of the decoder whose step is running (the attention interface reads them)


@dataclass
class XCaches:
    """by layer index: kp, vp [G, h, Lp, d], pos_p [G, Lp] (-1 = padding), kt, vt [G, h, Tt, d], gk, gv [G, h, Q, S, d]; shared by
    the layers: pos_t, own_t [G, Tt] (position and owning slot of each template token, -1 = padding), qpos [G, Q] int64,
    step_t [1] int64 (device), beam (queries per slot).  Positions and owners are kept as int32 device tensors."""

    kp: dict = field(default_factory=dict)
    vp: dict = field(default_factory=dict)
    pos_p: dict = field(default_factory=dict)
    kt: dict = field(default_factory=dict)
    vt: dict = field(default_factory=dict)
    gk: dict = field(default_factory=dict)
    gv: dict = field(default_factory=dict)
    pos_t: Optional[torch.Tensor] = None
    own_t: Optional[torch.Tensor] = None
    qpos: Optional[torch.Tensor] = None
    step_t: Optional[torch.Tensor] = None
    beam: int = 6
    len_p: dict = field(default_factory=dict)   # by layer: [G] int32, entries of each group's prefix that can hold keys (set_lengths)
    len_t: Optional[torch.Tensor] = None        # [G] int32, the same for the template range
    _spaces: dict = field(default_factory=dict)   # workspace of the split launches, by device
    _host_len: dict = field(default_factory=dict)   # by layer: (len_p, len_t) as host tuples (set_lengths)
    _plans: dict = field(default_factory=dict)      # split plans by geometry and lengths (plan_ragged)

    def set_lengths(self) -> None:
        """once per decoder, after the caches are filled: how far each group's prefix (pos_p >= 0) and template range
        (own_t >= 0) reach; the kernel then neither reads nor schedules the padding behind (decode.py:136-150 pads every group
        to the longest)"""
        def reach(valid):   # [G, L] bool -> index of the last True + 1
            L = valid.shape[1]
            idx = torch.arange(1, L + 1, device=valid.device, dtype=torch.int32)
            return (valid * idx).amax(1).to(torch.int32).contiguous() if L else torch.zeros(valid.shape[0], dtype=torch.int32, device=valid.device)

        for li, pos in self.pos_p.items():
            self.len_p[li] = reach(pos >= 0)
        self.len_t = reach(self.own_t >= 0)
        lt = tuple(self.len_t.tolist())
        self._host_len = {li: (tuple(n.tolist()), lt) for li, n in self.len_p.items()}
        self._plans.clear()

    def workspace(self, device, nbytes: int) -> torch.Tensor:
        w = self._spaces.get(device)
        if w is None or w.numel() < nbytes:
            w = self._spaces[device] = torch.empty(nbytes, dtype=torch.uint8, device=device)
        return w


class GroupKV:
    """stores the new tokens' K/V at the current step and hands the layer index to the attention (decode.py:51-68)"""

    is_compileable = False

    def __init__(self, caches: XCaches):
        self.caches = caches

    def update(self, key_states, value_states, layer_idx, *args, **kwargs):
        c = self.caches  # key_states [G, h, Q, d] -> entry step of every query's generated K/V
        c.gk[layer_idx].index_copy_(3, c.step_t, key_states.unsqueeze(3))
        c.gv[layer_idx].index_copy_(3, c.step_t, value_states.unsqueeze(3))
        return ("x", layer_idx), ("x", layer_idx)

    def get_seq_length(self, layer_idx: int = 0) -> int:
        return 0


def _i32(t: Optional[torch.Tensor], what: str) -> Optional[torch.Tensor]:
    if t is None:
        return None
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise ValueError(f"{what} must be a contiguous int32 tensor")
    return t


@torch.library.custom_op("spinf::xdecode_attn", mutates_args=("workspace",))
def _xdecode_op(query: torch.Tensor, kp: torch.Tensor, vp: torch.Tensor, pos_p: torch.Tensor, kt: torch.Tensor, vt: torch.Tensor,
                pos_t: torch.Tensor, own_t: torch.Tensor, gk: torch.Tensor, gv: torch.Tensor, qpos: torch.Tensor, step_t: torch.Tensor,
                len_p: Optional[torch.Tensor], len_t: Optional[torch.Tensor], workspace: Optional[torch.Tensor], nsplit: int, tiles_per_split: int, beam: int, scale: float, window: int, softcap: float) -> torch.Tensor:
    if not query.is_cuda:
        raise RuntimeError("spinf::xdecode_attn runs on ROCm device tensors only (no CPU path)")
    G, H, Q, d = query.shape
    h, Lp, Tt, S = gk.shape[1], kp.shape[2], kt.shape[2], gk.shape[3]
    for name, t in (("query", query), ("kp", kp), ("vp", vp), ("kt", kt), ("vt", vt), ("gk", gk), ("gv", gv)):
        if t.dtype != torch.bfloat16:
            raise ValueError(f"{name} must be bf16")
    for name, t, shape in (("kp", kp, (G, h, Lp, d)), ("vp", vp, (G, h, Lp, d)), ("kt", kt, (G, h, Tt, d)), ("vt", vt, (G, h, Tt, d)),
                           ("gk", gk, (G, h, Q, S, d)), ("gv", gv, (G, h, Q, S, d))):
        if tuple(t.shape) != shape or not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous {shape}, got {tuple(t.shape)}")
    if tuple(pos_p.shape) != (G, Lp) or tuple(pos_t.shape) != (G, Tt) or tuple(own_t.shape) != (G, Tt):
        raise ValueError("pos_p [G, Lp], pos_t and own_t [G, Tt] expected")
    if qpos.dtype != torch.int64 or tuple(qpos.shape) != (G, Q) or not qpos.is_contiguous() or step_t.dtype != torch.int64:
        raise ValueError("qpos [G, Q] and step_t [1] must be int64")
    if query.stride(3) != 1:
        query = query.contiguous()
    out = torch.empty((G, Q, H, d), dtype=torch.bfloat16, device=query.device)
    a = _lib.XdecArgs()
    a.q, a.q_g, a.q_h, a.q_q = query.data_ptr(), query.stride(0), query.stride(1), query.stride(2)
    a.kp, a.vp, a.pos_p = kp.data_ptr(), vp.data_ptr(), _i32(pos_p, "pos_p").data_ptr()
    a.kt, a.vt, a.pos_t, a.own_t = kt.data_ptr(), vt.data_ptr(), _i32(pos_t, "pos_t").data_ptr(), _i32(own_t, "own_t").data_ptr()
    a.gk, a.gv, a.qpos, a.step = gk.data_ptr(), gv.data_ptr(), qpos.data_ptr(), step_t.data_ptr()
    for name, t in (("len_p", len_p), ("len_t", len_t)):
        if t is not None:
            if tuple(t.shape) != (G,):
                raise ValueError(f"{name} must hold one length per group")
            setattr(a, name, _i32(t, name).data_ptr())
    a.out = out.data_ptr()
    a.nsplit, a.tiles_per_split = nsplit, tiles_per_split
    if workspace is not None:
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()
    a.G, a.H, a.h, a.Q, a.S, a.Lp, a.Tt, a.d, a.beam, a.window = G, H, h, Q, S, Lp, Tt, d, beam, window
    a.scale, a.softcap = scale, softcap
    lib = _lib.load_library()
    with torch.cuda.device(query.device):
        _lib.check(lib.spinf_xdecode_attn_fwd(C.byref(a), C.c_void_p(torch.cuda.current_stream(query.device).cuda_stream)), "spinf_xdecode_attn_fwd")
    return out


@_xdecode_op.register_fake
def _(query, kp, vp, pos_p, kt, vt, pos_t, own_t, gk, gv, qpos, step_t, len_p, len_t, workspace, nsplit, tiles_per_split, beam, scale, window, softcap):
    G, H, Q, d = query.shape
    return torch.empty((G, Q, H, d), dtype=torch.bfloat16, device=query.device)


def plan_splits(G: int, H: int, h: int, Q: int, S: int, Lp: int, Tt: int, d: int, beam: int) -> tuple[int, int]:
    """-> (nsplit, workspace bytes) the library suggests for these sizes"""
    a = _lib.XdecArgs()
    a.G, a.H, a.h, a.Q, a.S, a.Lp, a.Tt, a.d, a.beam = G, H, h, Q, S, Lp, Tt, d, beam
    ns, wb = C.c_int32(0), C.c_int64(0)
    _lib.check(_lib.load_library().spinf_xdecode_plan(C.byref(a), C.byref(ns), C.byref(wb)), "spinf_xdecode_plan")
    return ns.value, wb.value


_TILE, _ROWS = 32, 128   # keys per tile, rows per workgroup (csrc/xdecode_attn.hip)


def _list_tiles(Lp: int, Tt: int, S: int, len_p: int, len_t: int, qlo: int, qhi: int) -> int:
    """tiles of the list of a workgroup that owns queries qlo .. qhi (TileList of csrc/xdecode_attn.hip)"""
    lk = Lp + Tt
    e0 = -(-len_p // _TILE)
    s1 = max(Lp // _TILE if len_t > 0 else e0, e0)
    e1 = max(-(-(Lp + len_t) // _TILE) if len_t > 0 else s1, s1)
    s2 = max((lk + qlo * S) // _TILE, e1)
    e2 = max(-(-(lk + (qhi + 1) * S) // _TILE), s2)
    return e0 + (e1 - s1) + (e2 - s2)


def plan_ragged(G: int, H: int, h: int, Q: int, S: int, Lp: int, Tt: int, d: int, beam: int, len_p, len_t) -> tuple[int, int]:
    """-> (nsplit, tiles per split) for groups whose prefix / template ranges reach len_p[g] / len_t[g] entries: the split size
    with the shortest estimated step: the longer of (a) the simulated schedule (workgroups in launch order onto the places the
    GPU runs at a time; a workgroup costs its tiles + 2, a list that is split also its partial results' traffic, 7 tiles a piece
    at 128 rows x 256 head dims) at 2 us a tile and (b) all the tiles of the step at the rate the memory delivers them (6.5 ns a
    tile), plus 10 us for the merge launch of a split step.  The two rates are measured ones (XDEC, XDEC_long, XDEC_qwen of bench.py)."""
    import heapq

    r = H // h
    R = Q * r
    a = _lib.XdecArgs()
    a.G, a.H, a.h, a.Q, a.S, a.Lp, a.Tt, a.d, a.beam = G, H, h, Q, S, Lp, Tt, d, beam
    nt_max = C.c_int32(0)
    _lib.check(_lib.load_library().spinf_xdecode_tiles(C.byref(a), C.byref(nt_max)), "spinf_xdecode_tiles")
    nt_max = nt_max.value
    chunks = [(c * _ROWS // r, (min(c * _ROWS + _ROWS, R) - 1) // r, min(_ROWS, R - c * _ROWS)) for c in range(-(-R // _ROWS))]
    lists = [[_list_tiles(Lp, Tt, S, min(len_p[g], Lp), min(len_t[g], Tt), lo, hi) for g in range(G)] for lo, hi, _ in chunks]
    mean = sum(map(sum, lists)) / (G * len(chunks))
    places = 256 if d == 512 else 512
    cands = {nt_max} | {-(-nt_max // k) for k in range(2, 9)} | {int(mean * f) + 1 for f in (1.0, 1.15, 1.3, 1.5)}
    best = None
    for per in sorted(c for c in cands if 8 <= c <= nt_max or c == nt_max):
        ns_max = -(-nt_max // per)
        if ns_max > 16:
            continue
        free = [0.0] * places
        heapq.heapify(free)
        end = total = 0.0
        for (lo, hi, rows), nts in zip(chunks, lists):
            part = 7.0 * rows * (min(d, 256) + 2) / (_ROWS * 258)
            for nt in nts:
                ns = -(-nt // per)
                for _ in range(h):
                    for sp in range(ns_max):
                        t = min(per, nt - sp * per)
                        cost = 0.2 if t <= 0 else t + 2 + (part if ns > 1 else 0.0)
                        t0 = heapq.heappop(free)
                        heapq.heappush(free, t0 + cost)
                        end = max(end, t0 + cost)
                        total += cost
        est = max(end * 2.0, total * 0.0065) + (10.0 if ns_max > 1 else 0.0)   # microseconds
        if best is None or est < best[0]:
            best = (est, ns_max, per)
    return best[1], best[2]


def xdecode_attn(query, caches: XCaches, layer_idx: int, scale=None, window=None, softcap=None, nsplit=None):
    """query [G, H, Q, d] bf16 -> [G, Q, H, d] bf16: softmax over (the group's prefix | the slot's own template | the beam's own
    generated tokens up to caches.step_t), see x_attention"""
    c = caches
    G, H, Q, d = query.shape
    kp, gk = c.kp[layer_idx], c.gk[layer_idx]
    per = 0
    if nsplit is None and layer_idx in c._host_len:   # the groups' own lengths are known: split sizes that balance them
        geo = (G, H, gk.shape[1], Q, gk.shape[3], kp.shape[2], c.kt[layer_idx].shape[2], d, c.beam)
        key = geo + c._host_len[layer_idx]
        if key not in c._plans:
            c._plans[key] = plan_ragged(*geo, *c._host_len[layer_idx])
        nsplit, per = c._plans[key]
    elif nsplit is None:
        nsplit, _ = plan_splits(G, H, gk.shape[1], Q, gk.shape[3], kp.shape[2], c.kt[layer_idx].shape[2], d, c.beam)
    nbytes = G * H * Q * nsplit * (d + 2) * 4 if nsplit > 1 else 0
    work = c.workspace(query.device, nbytes) if nbytes else None
    return _xdecode_op(query, kp, c.vp[layer_idx], c.pos_p[layer_idx], c.kt[layer_idx], c.vt[layer_idx], c.pos_t, c.own_t, gk, c.gv[layer_idx],
                       c.qpos, c.step_t, c.len_p.get(layer_idx), c.len_t, work, int(nsplit), int(per), int(c.beam), float(scale if scale is not None else d**-0.5), int(window or 0),
                       float(softcap or 0.0))


@torch.compiler.disable
def x_attention(module, query, key, value, attention_mask, scaling=None, sliding_window=None, softcap=None, **kw):
    """the attention interface "x_decode" (decode.py:71-104): `key` is what GroupKV.update returned, ("x", layer index); the
    K/V live in the caches of the decoder whose step is running.  -> (attn_output [G, Q, H, d], None)"""
    caches = _CURRENT[0]
    if caches is None:
        raise RuntimeError("x_decode attention outside a decoding step (no caches set)")
    return xdecode_attn(query, caches, key[1], scaling, sliding_window, softcap), None


def register(name: str = "x_decode") -> None:
    from transformers import AttentionInterface

    if name not in AttentionInterface._global_mapping:
        AttentionInterface.register(name, x_attention)
