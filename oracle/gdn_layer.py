"""The element-wise work of a Gated DeltaNet layer on either side of the scan, restated in numpy (float32, rounded to bf16
where the reference's tensors are bf16).

prologue   spinf_serve/models/qwen35/qwen.py:657-668: ext = [qkv; zero row]; y = sum_j ext[conv[:, j]] * conv_w[:, j] in float32;
           qkv = silu(y) in the layer's dtype; q, k, v = the three column ranges; beta = sigmoid(b) in the layer's dtype;
           g = -exp(A_log) * softplus(a + dt_bias) in float32; on the indexed path q, k <- x * rsqrt(sum x^2 + 1e-6) per head,
           back in the layer's dtype
gate       qwen.py:670-672: of = o * rsqrt(mean(o^2) + eps) per head in float32; (norm_w * of.to(dtype)) in the layer's dtype;
           times silu(z) in float32; result in the layer's dtype

Test infrastructure only (see oracle/__init__.py).  Pinned in tests/test_gdn_layer.py against library routines on special
cases: along a single path the tap convolution is torch.nn.functional.conv1d (depthwise, left zero padding); a branch's
tokens equal the convolution over trunk || branch; silu / sigmoid / softplus / normalize / rms_norm are torch's own.
"""

from __future__ import annotations

import numpy as np


def bf16(x):
    """float32 -> nearest bf16 (ties to even), returned as float32"""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + np.uint32(0x7FFF)
    return ((u + r) & np.uint32(0xFFFF0000)).view(np.float32)


def silu(x):
    return x / (np.float32(1) + np.exp(-x, dtype=np.float32))


def prologue(y, conv, conv_w, a_log, dt_bias, h, hv, dk, dv, normalize):
    """y [T, >= 2 h dk + 2 hv dv + 2 hv] (bf16 values), conv [T, 4] int (T = zero row), conv_w [conv_dim, 4]
    -> q, k [T, h, dk], v [T, hv, dv], g [T, hv] (float32), beta [T, hv]; bf16 values as float32 except g"""
    y = np.asarray(y, np.float32)
    T = y.shape[0]
    kd, vd = h * dk, hv * dv
    cd = 2 * kd + vd
    ext = np.concatenate([y[:, :cd], np.zeros((1, cd), np.float32)])
    w = np.asarray(conv_w, np.float32)
    acc = np.zeros((T, cd), np.float32)
    for j in range(4):
        acc = acc + ext[np.asarray(conv)[:, j]] * w[None, :, j]
    qkv = bf16(silu(acc))
    q, k, v = qkv[:, :kd].reshape(T, h, dk), qkv[:, kd : 2 * kd].reshape(T, h, dk), qkv[:, 2 * kd :].reshape(T, hv, dv)
    b, a = y[:, cd + vd : cd + vd + hv], y[:, cd + vd + hv : cd + vd + 2 * hv]
    beta = bf16(np.float32(1) / (np.float32(1) + np.exp(-b, dtype=np.float32)))
    x = a + np.asarray(dt_bias, np.float32)[None]
    sp = np.where(x > 20, x, np.log1p(np.exp(np.minimum(x, 20), dtype=np.float32)))
    g = (-np.exp(np.asarray(a_log, np.float32)))[None] * sp.astype(np.float32)
    if normalize:
        q = bf16(q / np.sqrt((q * q).sum(-1, keepdims=True, dtype=np.float32) + np.float32(1e-6)))
        k = bf16(k / np.sqrt((k * k).sum(-1, keepdims=True, dtype=np.float32) + np.float32(1e-6)))
    return q, k, v, g.astype(np.float32), beta


def gate(o, z, norm_w, eps):
    """o [T, hv, dv], z [T, hv dv], norm_w [dv] (bf16 values) -> [T, hv dv] bf16 values as float32"""
    o = np.asarray(o, np.float32)
    T, hv, dv = o.shape
    of = o / np.sqrt((o * o).mean(-1, keepdims=True, dtype=np.float32) + np.float32(eps))
    n = bf16(np.asarray(norm_w, np.float32)[None, None] * bf16(of))
    return bf16(n * silu(np.asarray(z, np.float32).reshape(T, hv, dv))).reshape(T, hv * dv)
