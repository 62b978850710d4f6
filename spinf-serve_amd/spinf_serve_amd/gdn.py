"""Gated DeltaNet over trie segments with the reference's two entry points (spinf_serve/models/qwen35/gdn.py:109-133, 197-235).

Both run in libspinf_tree.so as fused WY-form kernels, one workgroup per (segment, head) on 32-token chunks: `chunked` for
long segments, `recurrent` for short ones (leaves that fork from one state are taken two to a chunk).  Unlike the reference's chunked(), the kernel reads and writes the stream rows through `idx` itself, so callers
need no gather / scatter around it, and it writes no per-chunk state snapshots.

q and k arrive l2-normalised; g is the log decay (fp32), beta the write strength, scale 1 / sqrt(K).
"""

from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from . import _lib


@torch.library.custom_op("spinf::gdn_scan", mutates_args=("o", "ht"))
def _gdn_scan_op(mode: int, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor, beta: torch.Tensor, scale: float,
                 cu: torch.Tensor, n: int, h0: Optional[torch.Tensor], h0_idx: Optional[torch.Tensor], ht: Optional[torch.Tensor],
                 ht_idx: Optional[torch.Tensor], idx: Optional[torch.Tensor], o: torch.Tensor, max_len: int) -> None:
    """the registered op over spinf_gdn_fwd: mode 0 = recurrent, 1 = chunked; writes the call's rows of `o` and the kept states
    into `ht` (inductor sees one opaque node that mutates the two, as it sees the reference's @torch.compiler.disable call)"""
    _launch(mode, q, k, v, g, beta, scale, cu, n, h0, h0_idx, ht, ht_idx, idx, o, max_len)


def _run(mode, q, k, v, g, beta, scale, cu, n, h0, h0_idx, ht, ht_idx, idx, o, max_len):
    if not q.is_cuda:
        raise RuntimeError("the Gated DeltaNet scan runs on ROCm device tensors only (no CPU path)")
    g = g if g.dtype == torch.float32 else g.float()
    beta = beta if beta.dtype == torch.bfloat16 else beta.to(torch.bfloat16)
    if o is None:
        o = torch.zeros_like(v) if idx is not None else torch.empty_like(v)
    _gdn_scan_op(mode, q, k, v, g, beta, float(scale), cu, int(n), h0, h0_idx, ht, ht_idx, idx, o, int(max_len))
    return o


def _launch(mode, q, k, v, g, beta, scale, cu, n, h0, h0_idx, ht, ht_idx, idx, o, max_len):
    if not q.is_cuda:
        raise RuntimeError("the Gated DeltaNet scan runs on ROCm device tensors only (no CPU path)")
    _, rows, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if q.dtype != torch.bfloat16 or k.dtype != torch.bfloat16 or v.dtype != torch.bfloat16:
        raise ValueError("q, k, v must be bf16")
    if g.dtype != torch.float32 or beta.dtype != torch.bfloat16:
        raise ValueError("g must be fp32 and beta bf16")
    if not (o.is_contiguous() or (o.stride(-1) == 1 and o.stride(-2) == V)):
        raise ValueError("o must be dense per row")
    if q.stride(1) != k.stride(1) or g.stride(1) != beta.stride(1):
        raise ValueError("q / k and g / beta must share their row strides")
    if q.stride(3) != 1 or q.stride(2) != K or v.stride(3) != 1 or v.stride(2) != V or g.stride(2) != 1 or beta.stride(2) != 1:
        raise ValueError("heads must be dense inside a row")
    for t, name in ((cu, "cu"), (idx, "idx"), (h0_idx, "h0_idx"), (ht_idx, "ht_idx")):
        if t is not None and (t.dtype != torch.int64 or not t.is_cuda or not t.is_contiguous()):
            raise ValueError(f"{name} must be a contiguous int64 device tensor")
    for t, name in ((h0, "h0"), (ht, "ht")):
        if t is not None and (t.dtype != torch.float32 or not t.is_contiguous() or t.shape[1:] != (HV, K, V)):
            raise ValueError(f"{name} must be contiguous fp32 [*, {HV}, {K}, {V}]")
    a = _lib.GdnArgs()
    a.q, a.k, a.v, a.g, a.beta, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), beta.data_ptr(), o.data_ptr()
    a.q_tok, a.v_tok, a.g_tok, a.o_tok = q.stride(1), v.stride(1), g.stride(1), o.stride(1)
    a.h, a.hv, a.dk, a.dv, a.scale = H, HV, K, V, float(scale)
    a.cu, a.idx, a.n_seg, a.max_len = cu.data_ptr(), (idx.data_ptr() if idx is not None else None), int(n), int(max_len)
    a.h0 = h0.data_ptr() if (h0 is not None and h0_idx is not None) else None
    a.h0_idx = h0_idx.data_ptr() if (h0 is not None and h0_idx is not None) else None
    a.ht = ht.data_ptr() if (ht is not None and ht_idx is not None) else None
    a.ht_idx = ht_idx.data_ptr() if (ht is not None and ht_idx is not None) else None
    a.mode = mode
    lib = _lib.load_library()
    with torch.cuda.device(q.device):
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _lib.check(lib.spinf_gdn_fwd(C.byref(a), C.c_void_p(stream)), "spinf_gdn_fwd")
    return o


def recurrent(q, k, v, g, beta, scale, cu, n, h0=None, h0_idx=None, ht=None, ht_idx=None, idx=None, o=None):
    """q, k [1, rows, H, K], v [1, rows, HV, V], g / beta [1, rows, HV], cu [n + 1] int64 (device) -> o [1, rows, HV, V].
    idx [sum of lengths] int64: the call's tokens are these rows of the tensors and the outputs go to the same rows of `o`
    (spinf_serve/models/qwen35/gdn.py:197-201); without idx rows 0.. in call order."""
    return _run(0, q, k, v, g, beta, scale, cu, n, h0, h0_idx, ht, ht_idx, idx, o, 0)


def chunked(q, k, v, g, beta, scale, cu, cu_cpu, h0=None, h0_idx=None, ht=None, ht_idx=None, chunk_size=64, idx=None, o=None):
    """gdn.chunked's contract (spinf_serve/models/qwen35/gdn.py:109-112): sequence n = call rows cu[n] .. cu[n+1]-1 starts from
    h0[h0_idx[n]] (zero when absent or negative) and leaves its final state in ht[ht_idx[n]] where that is >= 0.
    idx / o: optional row indirection as in `recurrent` (not in the reference, which gathers before and scatters after)."""
    if chunk_size <= 0:
        raise ValueError("chunk_size must be positive")  # the result does not depend on it: the kernel chunks by 32 internally
    if k.shape[-1] != 128:
        raise ValueError("the state kernel is written for K = 128")  # gdn.py:120
    n = len(cu_cpu) - 1
    lens = cu_cpu[1:] - cu_cpu[:-1]
    return _run(1, q, k, v, g, beta, scale, cu, n, h0, h0_idx, ht, ht_idx, idx, o, int(lens.max()) if n else 0)
