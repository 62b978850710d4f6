"""The attention op of the packed forward, with the reference's two call signatures.

  tree_attn(q, k, v, mask, scale)                     the custom op spinf::tree_attn on token-major tensors
  tree_flex_forward(module, query, key, value, ...)   transformers AttentionInterface callable "tree_flex"
                                                      (spinf_serve/models/gemma4.py:98-119)
  tree_attention(q, k, v, mask, scale, sidx, ...)     the Qwen stack's function (spinf_serve/models/qwen35/qwen.py:604-623)

The op is a thin wrapper over spinf_tree_attn_fwd of libspinf_tree.so; it runs on ROCm tensors only.
"""

from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

from . import _lib
from .masks import TreeMask

# kernel tuning variant handed to the library (0 = its default choice: eight waves, the two heads of a GQA pair per work item, where
# a group is even; 1 = one head per work item, four waves; 2 = four waves with two heads each, head dim <= 128; 3 is set by
# tree_attn itself where head dim 128 goes to the kernel with decoupled waves); results do not depend on it
VARIANT = int(os.environ.get("SPINF_ATTN_VARIANT", "0"))
# the kernel with decoupled waves over a static schedule, where the library has one for the geometry (0: the lockstep kernels only)
RING = int(os.environ.get("SPINF_ATTN_RING", "-1"))      # -1 = auto


# a static schedule (items dealt out to the workgroups on the host) also for the lockstep kernels
STATIC = int(os.environ.get("SPINF_ATTN_STATIC", "-1"))  # -1 = auto


RING_MAX_ITEMS_PER_WG = 8
# head dim 128: the kernel with decoupled waves over 64-key tiles (the library's variant 3) where the geometry allows
RING_128 = False

# test hook (spinf_attn_args.debug_expire): k > 0 = polls after which a wave of the decoupled kernel gives up a wait (2^18 otherwise)
DEBUG_EXPIRE = 0


def _check_tensors(q, k, v, n_mask, compact, others=()):
    """what every kernel launch assumes about q, k, v (and the device of whatever else it reads): raises before any launch"""
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise ValueError("spinf::tree_attn takes bf16 q, k, v")
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise ValueError("q, k, v must be [rows, heads, head dim]")
    rows, hq, d = q.shape
    hkv = k.shape[1]
    if k.shape != (rows, hkv, d) or v.shape != (rows, hkv, d):
        raise ValueError(f"k / v shapes {tuple(k.shape)} {tuple(v.shape)} do not match q {tuple(q.shape)}")
    if hkv <= 0 or hq % hkv:
        raise ValueError(f"{hq} query heads do not group over {hkv} key / value heads")
    if q.stride(2) != 1 or k.stride(2) != 1 or v.stride(2) != 1:
        raise ValueError("the head dimension must be contiguous")
    if not compact and rows != n_mask:
        raise ValueError(f"mask describes {n_mask} tokens, q / k / v have {rows}")
    if not q.is_cuda:
        raise RuntimeError("spinf::tree_attn runs on ROCm device tensors only (no CPU path)")
    for t in (k, v, *others):
        if t is not None and t.device != q.device:
            raise ValueError(f"all tensors of the call must be on {q.device}, one is on {t.device}")


def _ring_lists(q, hq, hkv, d, variant, sidx, mask):
    """-> (workgroups of the static schedule or 0, whether the call goes to the kernel with decoupled waves).

    Measured on MI355X: the decoupled kernel wins where a workgroup gets only a handful of items (C2: 6.75 per workgroup), since
    its waves run through the item boundaries; with many items per workgroup (C3's 65,536-token passes: 16) the lockstep kernel
    is 6 - 10 % faster.  The lockstep kernel takes its shared queues (measured over C3's 13 passes, the variants taking turns: sliding
    layers 9.64 ms on the queues, 10.33 on static lists, 10.39 on the decoupled kernel; global layers 11.38 / 12.11 / 12.20).
    SPINF_ATTN_RING / SPINF_ATTN_STATIC = 0 / 1 switch the two for every call where the geometry allows, "auto" (the default)
    follows the measurements.  Head dim 128 has the decoupled kernel too (the library's
    variant 3, 64-key tiles): 55.5 against 48.5 ms on C4, so "auto" leaves it to the lockstep kernel (RING_128 or
    SPINF_ATTN_RING=1 select it)."""
    from .masks import _static_lists

    n_wg = _static_lists(q.device)
    ring = (d == 512 or (variant == 0 and d in (128, 256) and (hq // hkv) % 2 == 0)) and sidx is None and mask.grp is None
    if ring and RING < 0:
        ring = d == 512 or (d == 256 and mask.plan.n_qtiles * (hq // 2) <= RING_MAX_ITEMS_PER_WG * n_wg) or (d == 128 and RING_128)
    elif not RING:
        ring = False
    static = d != 512 and STATIC > 0
    if ring or static:
        return n_wg, ring
    return 0, False


def _attn_args(q, k, v, out, n, art, end, pos, kv_idx, kv_bits, items, list_ptr, n_items, scale, window, variant, row_of, kv_row0, grp, grp_mode, ktile, n_lists=0):
    """the C ABI's argument block (spinf_attn_args) for these tensors"""
    hq, d = q.shape[1], q.shape[2]
    hkv = k.shape[1]
    a = _lib.AttnArgs()
    a.q, a.k, a.v, a.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.q_tok, a.q_head = q.stride(0), q.stride(1)
    a.k_tok, a.k_head = k.stride(0), k.stride(1)
    a.v_tok, a.v_head = v.stride(0), v.stride(1)
    a.o_tok, a.o_head = out.stride(0), out.stride(1)
    a.n, a.hq, a.hkv, a.d, a.scale, a.window = n, hq, hkv, d, scale, window
    a.art, a.end, a.pos = art.data_ptr(), end.data_ptr(), pos.data_ptr()
    a.kv_idx, a.kv_bits, a.items, a.list_ptr = kv_idx.data_ptr(), kv_bits.data_ptr(), items.data_ptr(), list_ptr.data_ptr()
    a.n_items = n_items
    a.variant = variant
    a.ktile = ktile
    a.n_lists = n_lists
    a.debug_expire = DEBUG_EXPIRE
    if row_of is not None:
        a.row_of, a.kv_row0 = row_of.data_ptr(), kv_row0.data_ptr()
    if grp is not None:
        if grp.dtype != torch.int32 or grp.numel() < n:
            raise ValueError("grp must be int32 [n]")
        a.grp, a.grp_mode = grp.data_ptr(), grp_mode
    return a


@torch.library.custom_op("spinf::tree_attn", mutates_args=())
def _tree_attn_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, art: torch.Tensor, end: torch.Tensor, pos: torch.Tensor,
                  kv_idx: torch.Tensor, kv_bits: torch.Tensor, items: torch.Tensor, list_ptr: torch.Tensor, n_items: int,
                  scale: float, window: int, variant: int, row_of: Optional[torch.Tensor], kv_row0: Optional[torch.Tensor],
                  n_mapped: int, grp: Optional[torch.Tensor], grp_mode: int, ktile: int, n_lists: int) -> torch.Tensor:
    """q [rows, hq, d], k / v [rows, hkv, d] (any token / head strides, d contiguous) -> out [rows, hq, d] contiguous, bf16.
    rows = the stream length, or with row_of / kv_row0 (compact rows) any number of rows: the kernel maps stream positions to
    rows through row_of; rows 0 .. n_mapped-1 are the rows row_of names (each written by the kernel), later rows come back zero."""
    _check_tensors(q, k, v, art.numel(), row_of is not None, (art, end, pos, kv_idx, kv_bits, items, list_ptr, row_of, kv_row0, grp))
    rows, hq, d = q.shape
    n = art.numel() if row_of is not None else rows
    if art.numel() < n:
        raise ValueError(f"mask built for {art.numel()} tokens, stream has {n}")
    if (row_of is None) != (kv_row0 is None):
        raise ValueError("row_of and kv_row0 come together")
    if row_of is not None:
        if row_of.dtype != torch.int32 or kv_row0.dtype != torch.int32 or row_of.numel() != n or kv_row0.numel() != kv_idx.numel():
            raise ValueError("row_of [n] and kv_row0 [entries] must be int32")
        if not 0 <= n_mapped <= rows:
            raise ValueError(f"{n_mapped} mapped rows, q has {rows}")
        out = torch.empty((rows, hq, d), dtype=torch.bfloat16, device=q.device)
        out[n_mapped:].zero_()
    else:
        out = torch.empty((rows, hq, d), dtype=torch.bfloat16, device=q.device)
    a = _attn_args(q, k, v, out, n, art, end, pos, kv_idx, kv_bits, items, list_ptr, n_items, scale, window, variant, row_of, kv_row0, grp, grp_mode, ktile, n_lists)
    lib = _lib.load_library()
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _lib.check(lib.spinf_tree_attn_fwd(C.byref(a), C.c_void_p(stream)), "spinf_tree_attn_fwd")
    return out


@_tree_attn_op.register_fake
def _(q, k, v, art, end, pos, kv_idx, kv_bits, items, list_ptr, n_items, scale, window, variant, row_of, kv_row0, n_mapped, grp, grp_mode, ktile, n_lists):
    return torch.empty(q.shape, dtype=torch.bfloat16, device=q.device)


def tree_attn(q, k, v, mask: TreeMask, scale=None, variant=None, sidx=None):
    """q [n, hq, d], k / v [n, hkv, d] bf16 -> [n, hq, d]: softmax(scale q k^T under the tree mask) v.
    sidx [R] (compact rows): q, k, v hold real tokens only, row r is stream position sidx[r]; the kernel reads and writes them
    in place of the scatter into stream layout and the gather back (rows >= R come back zero)."""
    if not isinstance(mask, TreeMask):
        raise TypeError("attention_mask must be a TreeMask (masks.block_masks)")
    _check_tensors(q, k, v, mask.n, sidx is not None, (mask.art, mask.end, mask.pos, mask.kv_idx, mask.kv_bits, mask.grp, sidx))
    if sidx is not None and sidx.shape[0] > q.shape[0]:
        raise ValueError(f"sidx names {sidx.shape[0]} rows, q has {q.shape[0]}")
    scale = float(q.shape[-1] ** -0.5 if scale is None else scale)
    variant = int(VARIANT if variant is None else variant)
    if (sidx is not None or mask.grp is not None) and variant == 2:
        variant = 0   # the two-heads-per-wave kernels take neither compact rows nor image groups
    if sidx is not None and mask.grp is not None:
        raise ValueError("image groups go with the stream layout (no sidx)")
    hq, hkv, d = q.shape[1], k.shape[1], q.shape[2]
    n_lists, ring = _ring_lists(q, hq, hkv, d, variant, sidx, mask)
    if ring and d == 128:
        variant = 3   # (64-key plan entries, as the lockstep kernels take)
    mask = mask.for_head_dim(d, ring=ring and d != 128)
    per_item = _lib.load_library().spinf_attn_heads_per_item(hq, hkv, d, variant)
    if per_item <= 0:
        raise ValueError(f"{hq} query heads do not group over {hkv} key / value heads")
    items, list_ptr, n_items = mask.schedule(hq // per_item, n_lists)
    row_of, kv_row0 = mask.rows(sidx) if sidx is not None else (None, None)
    return _tree_attn_op(q, k, v, mask.art, mask.end, mask.pos, mask.kv_idx, mask.kv_bits, items, list_ptr, n_items,
                         scale, int(mask.window), variant, row_of, kv_row0, 0 if sidx is None else int(sidx.shape[0]),
                         mask.grp, int(mask.grp_mode), int(mask.plan.ktile), n_lists)


def tree_attn_noalloc(q, k, v, mask: TreeMask, out, scale=None):
    """tree_attn into a caller-owned ``out`` [n, hq, d] through spinf_tree_attn_fwd_noalloc: the pass that allocates nothing on
    the device (for callers under graph capture or in loops that must not allocate; no counterpart in the reference).  The
    mask's schedule must already be on the device (any earlier call with this head geometry uploads it); stream layout only;
    at most 65,536 work items.  Same bits as tree_attn."""
    if not isinstance(mask, TreeMask):
        raise TypeError("attention_mask must be a TreeMask (masks.block_masks)")
    if out.shape != q.shape or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise ValueError("out must be a contiguous bf16 tensor of q's shape")
    _check_tensors(q, k, v, mask.n, False, (out, mask.art, mask.end, mask.pos, mask.kv_idx, mask.kv_bits, mask.grp))
    n, hq, d = q.shape
    hkv = k.shape[1]
    n_lists, ring = _ring_lists(q, hq, hkv, d, 0, None, mask)
    variant = 3 if ring and d == 128 else 0
    mask = mask.for_head_dim(d, ring=ring and d != 128)
    per_item = _lib.load_library().spinf_attn_heads_per_item(hq, hkv, d, variant)
    if per_item <= 0:
        raise ValueError(f"{hq} query heads do not group over {hkv} key / value heads")
    items, list_ptr, n_items = mask.schedule(hq // per_item, n_lists)
    scale = float(d ** -0.5 if scale is None else scale)
    a = _attn_args(q, k, v, out, n, mask.art, mask.end, mask.pos, mask.kv_idx, mask.kv_bits, items, list_ptr, n_items, scale, int(mask.window), variant,
                   None, None, mask.grp, int(mask.grp_mode), int(mask.plan.ktile), n_lists)
    lib = _lib.load_library()
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _lib.check(lib.spinf_tree_attn_fwd_noalloc(C.byref(a), C.c_void_p(stream)), "spinf_tree_attn_fwd_noalloc")
    return out


def tree_attn_byte_pattern(q, k, v, mask: TreeMask, out, status, parts=3, nslot=4):
    """A yardstick, not an operator (spinf_diag_attn_stream): the data movement of tree_attn's kernel with decoupled waves for these
    tensors (head dim 256, the same static schedule: query loads, every K / V tile of every work item through the LDS ring by the
    same DMA requests, output stores in the kernel's pattern) with nothing computed; ``out`` [n, hq, d] comes back as ones on the
    real rows.  status: 2 int32 on the device, zeroed by the caller: [0] += waves that gave up a wait, [1] += tiles seen landed.
    parts: 3 = all of it, 1 = the K / V tiles only, 2 = the queries and outputs only; nslot: ring slots in use (tile requests in
    flight), 1 .. 4."""
    if not isinstance(mask, TreeMask):
        raise TypeError("attention_mask must be a TreeMask (masks.block_masks)")
    if out.shape != q.shape or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise ValueError("out must be a contiguous bf16 tensor of q's shape")
    if status.dtype != torch.int32 or status.numel() < 2 or not status.is_contiguous():
        raise ValueError("status must be 2 contiguous int32")
    _check_tensors(q, k, v, mask.n, False, (out, status, mask.art, mask.end, mask.pos, mask.kv_idx, mask.kv_bits))
    n, hq, d = q.shape
    hkv = k.shape[1]
    if d != 256 or (hq // hkv) % 2 or mask.grp is not None:
        raise ValueError("the byte-pattern yardstick covers head dim 256 with an even number of query heads per key / value head, no image groups")
    n_lists = _static_lists_of(q.device)
    mask = mask.for_head_dim(d, ring=True)
    items, list_ptr, n_items = mask.schedule(hq // 2, n_lists)
    a = _attn_args(q, k, v, out, n, mask.art, mask.end, mask.pos, mask.kv_idx, mask.kv_bits, items, list_ptr, n_items, float(d ** -0.5), int(mask.window), 0,
                   None, None, None, 0, int(mask.plan.ktile), n_lists)
    lib = _lib.load_library()
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _lib.check(lib.spinf_diag_attn_stream(C.byref(a), int(parts), int(nslot), C.c_void_p(status.data_ptr()), C.c_void_p(stream)), "spinf_diag_attn_stream")
    return out


def _static_lists_of(device):
    from .masks import _static_lists

    return _static_lists(device)


# K/V capture for extraction, as spinf_serve/models/gemma4.py:66-70: while CAPTURE[device] = {"window", "ranges": [(start, n, key)],
# "kv": {}} is set, every call keeps the layer's keys / values of the ranges (sliding layers only their last window - 1)
CAPTURE: dict = {}


@torch.compiler.disable
def tree_flex_forward(module, query, key, value, attention_mask, scaling=None, sliding_window=None, **kw):
    """transformers attention interface: query [1, Hq, N, D], key / value [1, Hkv, N, D] (views of token-major tensors),
    attention_mask a TreeMask -> (attn_output [1, N, Hq, D] contiguous, None)   (spinf_serve/models/gemma4.py:98-119)"""
    cap = CAPTURE.get(query.device)
    if cap is not None:
        keep = cap["window"] - 1
        sliding = module.config.layer_types[module.layer_idx] == "sliding_attention"
        for start, n, name in cap["ranges"]:
            a = start + (max(0, n - keep) if sliding else 0)
            cap["kv"].setdefault(name, {})[module.layer_idx] = (key[:, :, a : start + n].clone(), value[:, :, a : start + n].clone())
    if query.shape[0] != 1:
        raise ValueError("the packed stream is one sequence: batch size must be 1")
    out = tree_attn(query[0].transpose(0, 1), key[0].transpose(0, 1), value[0].transpose(0, 1), attention_mask, scaling)
    return out[None], None


def register_tree_attention(name: str = "tree_flex") -> None:
    """registers tree_flex_forward with transformers, as spinf_serve/models/gemma4.py:121-122 does"""
    from transformers import AttentionInterface

    if name not in AttentionInterface._global_mapping:
        AttentionInterface.register(name, tree_flex_forward)


@torch.compiler.disable
def tree_attention(q, k, v, mask, scale, sidx=None, plan=None, mod=None):
    """q [1, H, rows, d], k / v [1, Hkv, rows, d] -> [1, H, rows, d]   (spinf_serve/models/qwen35/qwen.py:604-623).
    sidx (compact rows): stream position of each real row.  The reference scatters the rows into the stream layout the mask
    describes (pads: zero rows attending to themselves) and gathers the output back; here the kernel goes through the row map
    and the result for every real row is the same bit for bit."""
    cap = plan.cap if plan is not None else None
    if cap is not None:
        for r0, n, name in cap["ranges"]:
            cap["out"]["kv"].setdefault(name, {})[mod.li] = (k[:, :, r0 : r0 + n].clone(), v[:, :, r0 : r0 + n].clone())
    if sidx is None:
        o = tree_attn(q[0].transpose(0, 1), k[0].transpose(0, 1), v[0].transpose(0, 1), mask, scale)
        return o.transpose(0, 1)[None]
    # compact rows: the kernel maps stream positions to rows itself (no scatter into stream layout, no gather back)
    o = tree_attn(q[0].transpose(0, 1), k[0].transpose(0, 1), v[0].transpose(0, 1), mask, scale, sidx=sidx)
    return o.transpose(0, 1)[None]
