"""The element-wise work of the Qwen stack's GatedDeltaNet.forward on either side of the scan
(spinf_serve/models/qwen35/qwen.py:657-672), as two HIP kernels of libspinf_tree.so.

    q, k, v, g, beta = gdn_prologue(y, plan.conv, conv_w, A_log, dt_bias, hk, hv, dk, dv, normalize=plan.path == "indexed")
    o = gdn_tree(q, k, v, g, beta, plan)
    out = gdn_gate(o, y[:, conv_dim : conv_dim + hv * dv], norm_w, eps)        # then out_proj

y is the input projection's output [T, conv_dim + hv dv + 2 hv] (q k v | z | b | a).  There is no CPU path.
"""

from __future__ import annotations

import ctypes as C

import torch

from . import _lib


@torch.library.custom_op("spinf::gdn_prologue", mutates_args=())
def _prologue_op(y: torch.Tensor, conv: torch.Tensor, conv_w: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                 h: int, hv: int, dk: int, dv: int, normalize: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    if not y.is_cuda:
        raise RuntimeError("spinf::gdn_prologue runs on ROCm device tensors only (no CPU path)")
    if y.dtype != torch.bfloat16 or y.dim() != 2 or y.stride(1) != 1:
        raise ValueError("y must be a bf16 matrix with contiguous rows")
    T = y.shape[0]
    kd, vd = h * dk, hv * dv
    if y.shape[1] < 2 * kd + 2 * vd + 2 * hv:
        raise ValueError(f"y has {y.shape[1]} columns, q k v z b a need {2 * kd + 2 * vd + 2 * hv}")
    if conv.shape != (T, 4) or conv.dtype != torch.int64:
        raise ValueError("conv must be int64 [T, 4]")
    if conv_w.shape != (2 * kd + vd, 4):
        raise ValueError(f"conv_w must be [{2 * kd + vd}, 4]")
    conv = conv.contiguous()
    conv_w = conv_w.float().contiguous()
    a_log = a_log.float().contiguous()
    dt_bias = dt_bias.float().contiguous()
    dev = y.device
    q = torch.empty((T, h, dk), dtype=torch.bfloat16, device=dev)
    k = torch.empty((T, h, dk), dtype=torch.bfloat16, device=dev)
    v = torch.empty((T, hv, dv), dtype=torch.bfloat16, device=dev)
    g = torch.empty((T, hv), dtype=torch.float32, device=dev)
    beta = torch.empty((T, hv), dtype=torch.bfloat16, device=dev)
    a = _lib.GdnPreArgs()
    a.y, a.y_tok = y.data_ptr(), y.stride(0)
    a.conv, a.conv_w, a.a_log, a.dt_bias = conv.data_ptr(), conv_w.data_ptr(), a_log.data_ptr(), dt_bias.data_ptr()
    a.q, a.k, a.v, a.g, a.beta = q.data_ptr(), k.data_ptr(), v.data_ptr(), g.data_ptr(), beta.data_ptr()
    a.T, a.h, a.hv, a.dk, a.dv, a.normalize = T, h, hv, dk, dv, int(normalize)
    lib = _lib.load_library()
    with torch.cuda.device(dev):
        _lib.check(lib.spinf_gdn_prologue(C.byref(a), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)), "spinf_gdn_prologue")
    return q, k, v, g, beta


@_prologue_op.register_fake
def _(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, normalize):
    T = y.shape[0]
    e = lambda shape, dt: torch.empty(shape, dtype=dt, device=y.device)  # noqa: E731
    return (e((T, h, dk), torch.bfloat16), e((T, h, dk), torch.bfloat16), e((T, hv, dv), torch.bfloat16), e((T, hv), torch.float32),
            e((T, hv), torch.bfloat16))


def gdn_prologue(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, normalize=True):
    """-> q, k [T, h, dk], v [T, hv, dv] bf16, g [T, hv] fp32, beta [T, hv] bf16   (qwen.py:657-668 in one pass over y)"""
    return _prologue_op(y, conv, conv_w, a_log, dt_bias, int(h), int(hv), int(dk), int(dv), bool(normalize))


@torch.library.custom_op("spinf::gdn_gate", mutates_args=())
def _gate_op(o: torch.Tensor, z: torch.Tensor, norm_w: torch.Tensor, eps: float) -> torch.Tensor:
    if not o.is_cuda:
        raise RuntimeError("spinf::gdn_gate runs on ROCm device tensors only (no CPU path)")
    if o.dtype != torch.bfloat16 or z.dtype != torch.bfloat16 or o.dim() != 3:
        raise ValueError("o [T, hv, dv] and z [T, hv dv] must be bf16")
    T, hv, dv = o.shape
    if z.shape != (T, hv * dv) or z.stride(1) != 1 or o.stride(2) != 1 or o.stride(1) != dv:
        raise ValueError("z must be [T, hv dv] with contiguous rows, o dense inside a row")
    norm_w = norm_w.to(torch.bfloat16).contiguous()
    out = torch.empty((T, hv * dv), dtype=torch.bfloat16, device=o.device)
    a = _lib.GdnGateArgs()
    a.o, a.o_tok, a.z, a.z_tok, a.norm_w, a.eps = o.data_ptr(), o.stride(0), z.data_ptr(), z.stride(0), norm_w.data_ptr(), eps
    a.out, a.T, a.hv, a.dv = out.data_ptr(), T, hv, dv
    lib = _lib.load_library()
    with torch.cuda.device(o.device):
        _lib.check(lib.spinf_gdn_gate(C.byref(a), C.c_void_p(torch.cuda.current_stream(o.device).cuda_stream)), "spinf_gdn_gate")
    return out


@_gate_op.register_fake
def _(o, z, norm_w, eps):
    return torch.empty((o.shape[0], o.shape[1] * o.shape[2]), dtype=torch.bfloat16, device=o.device)


def gdn_gate(o, z, norm_w, eps):
    """o [T, hv, dv], z [T, hv dv] (a column range of y is fine) -> [T, hv dv]: norm_w * rms_norm(o) * silu(z)   (qwen.py:670-672)"""
    return _gate_op(o, z, norm_w, float(eps))
