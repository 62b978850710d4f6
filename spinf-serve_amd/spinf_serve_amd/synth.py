"""Seeded synthetic workloads: the benchmark configurations of the tree-mask attention path and of the Gated DeltaNet scan.

Each attention config is a set of contents (trunk + question branches, optionally two-level) laid out by the package's own
layout module with aligned jobs (every content starts on a 128-token boundary, spinf_serve/packer.py:421-422), plus the head
geometry and value distribution.  Everything derives from numpy.random.default_rng(seed).

  C1     2 x (64 + 4 x 8), 4/2 heads, d 64, scale d^-0.5, N(0,1)           (the CPU plumbing case)
  C2     24 x (470 + 56 x U{8..16}), 16/8, d 256, scale 1/16, 0.5 N(0,1)   (the headline case)
  C3     512 contents, trunk lognormal(median 800, sigma 0.6) clipped 64..4096, U{8..64} branches of U{4..24}, passes of
         <= 65,536 tokens, 16/8, d 256, window 1024 on sliding layers
  C4     64 x (8192 + 16 nodes x 32 + 16 x 12 leaves x U{6..10}), 32/16, d 128
  C5     Gated DeltaNet: 128 x (2048 + 32 x 12), 16 qk / 32 v heads, 128 x 128 state
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

from .layout import BLOCK, TokenTree, pack_stream, pack_streams


@dataclass
class AttnConfig:
    name: str
    hq: int
    hkv: int
    d: int
    scale: float
    std: float
    window: int | None
    trees: list
    batches: list = field(default_factory=list)
    note: str = ""

    @property
    def n_real(self) -> int:
        return sum(b.n_tokens for b in self.batches)

    def pairs(self, window=None) -> int:
        """visible (q, k) pairs over all batches, pad self-pairs excluded: a real token sees the pos+1 tokens of its path,
        the last `window` of them on a sliding layer"""
        tot = 0
        for b in self.batches:
            p = b.pos[b.art >= 0].astype(np.int64) + 1
            tot += int((np.minimum(p, window) if window else p).sum())
        return tot

    def flops(self, window=None) -> float:
        return 4.0 * self.d * self.hq * self.pairs(window)

    def bytes(self) -> float:
        return 2.0 * self.n_real * (2 * self.hq + 2 * self.hkv) * self.d


def _tree(rng, trunk, branch_lens, parents=None):
    ids = lambda n: rng.integers(5, 32000, int(n)).tolist()  # noqa: E731
    return TokenTree(ids(trunk), [ids(n) for n in branch_lens], list(parents) if parents is not None else [])


def pack(trees, budget=None, align=True):
    """-> batches.  budget None: one stream in the given order; else first-fit-decreasing streams of <= budget tokens"""
    if budget is None:
        return [pack_stream(trees, align=align)]
    return pack_streams(trees, budget, align=align)


def attention_config(name: str, seed: int = 0, contents: int | None = None) -> AttnConfig:
    """name: C1 | C2 | C3 | C4 | smoke; contents overrides the number of contents (scaled-down parity cases)."""
    rng = np.random.default_rng(seed)
    if name == "C1":
        n = contents or 2
        trees = [_tree(rng, 64, [8] * 4) for _ in range(n)]
        cfg = AttnConfig(name, 4, 2, 64, 64 ** -0.5, 1.0, None, trees)
        cfg.batches = pack(trees)
    elif name == "smoke":
        trees = [_tree(rng, 150, rng.integers(3, 14, 9)), _tree(rng, 70, [5, 9])]
        cfg = AttnConfig(name, 4, 2, 128, 128 ** -0.5, 0.5, None, trees)
        cfg.batches = pack(trees)
    elif name == "C2":
        n = contents or 24
        trees = [_tree(rng, 470, rng.integers(8, 17, 56)) for _ in range(n)]
        cfg = AttnConfig(name, 16, 8, 256, 1.0 / 16, 0.5, None, trees)
        cfg.batches = pack(trees)
    elif name == "C2_512":   # C2's stream at the head geometry of the Gemma-4 full-attention layers
        n = contents or 24
        trees = [_tree(rng, 470, rng.integers(8, 17, 56)) for _ in range(n)]
        cfg = AttnConfig(name, 16, 1, 512, 512 ** -0.5, 0.5, None, trees)
        cfg.batches = pack(trees)
    elif name == "C3":
        n = contents or 512
        trees = []
        for _ in range(n):
            trunk = int(np.clip(np.exp(np.log(800.0) + 0.6 * rng.standard_normal()), 64, 4096))
            trees.append(_tree(rng, trunk, rng.integers(4, 25, int(rng.integers(8, 65)))))
        cfg = AttnConfig(name, 16, 8, 256, 1.0 / 16, 0.5, 1024, trees, note="trunk lognormal sigma 0.6")
        cfg.batches = pack(trees, budget=65536)
    elif name == "C4":
        n = contents or 64
        trees = []
        for _ in range(n):
            lens, parents = [], []
            for _node in range(16):
                node = len(lens)
                lens.append(32)
                parents.append(-1)
                for _leaf in range(12):
                    lens.append(int(rng.integers(6, 11)))
                    parents.append(node)
            trees.append(_tree(rng, 8192, lens, parents))
        cfg = AttnConfig(name, 32, 16, 128, 128 ** -0.5, 0.5, None, trees)
        cfg.batches = pack(trees)
    else:
        raise ValueError(f"unknown attention config {name!r}")
    return cfg


def qkv(cfg: AttnConfig, batch, seed: int = 0, device="cuda"):
    """Q [N, hq, d], K / V [N, hkv, d] bf16 ~ std N(0, 1) for the batch's stream (pads included: they attend to themselves)"""
    import torch

    gen = torch.Generator(device="cpu").manual_seed(seed + 7919 * batch.length)
    n = batch.length

    def mk(h):
        # generated on the host in chunks so that a multi-GB stream never holds an fp32 copy at once
        out = torch.empty((n, h, cfg.d), dtype=torch.bfloat16, device=device)
        step = max(1, (1 << 24) // (h * cfg.d))
        for a in range(0, n, step):
            b = min(n, a + step)
            out[a:b] = (torch.randn((b - a, h, cfg.d), generator=gen) * cfg.std).to(torch.bfloat16).to(device)
        return out

    return mk(cfg.hq), mk(cfg.hkv), mk(cfg.hkv)


def qkv_device(cfg: AttnConfig, batch, seed: int = 0, device="cuda"):
    """Q, K, V of qkv()'s shapes and value distribution, drawn by the device's generator: for streams of several GB, where the
    host generator takes half a minute.  (Other values than qkv()'s for the same seed.)"""
    import torch

    gen = torch.Generator(device=device).manual_seed(seed + 7919 * batch.length)
    n = batch.length

    def mk(h):
        out = torch.empty((n, h, cfg.d), dtype=torch.bfloat16, device=device)
        step = max(1, (1 << 26) // (h * cfg.d))
        for a in range(0, n, step):
            b = min(n, a + step)
            out[a:b] = (torch.randn((b - a, h, cfg.d), generator=gen, device=device) * cfg.std).to(torch.bfloat16)
        return out

    return mk(cfg.hq), mk(cfg.hkv), mk(cfg.hkv)


# ------------------------------------------------------------------------------------------------ Gated DeltaNet
@dataclass
class GdnConfig:
    name: str
    h: int
    hv: int
    dk: int
    dv: int
    trees: list
    batch: object = None

    def plan(self, device, **kw):
        """the recurrent-layer plan of the stream.  call_tokens (the reference's cap on a chunked call, there to bound its
        per-chunk state snapshots, spinf_serve/models/qwen35/qwen.py:228-236) is lifted by default: the fused kernel writes
        no snapshots, so one launch per level and kind serves the whole stream"""
        from .qwen_plan import tree_plan

        kw.setdefault("call_tokens", 1 << 40)
        return tree_plan(self.batch.prev, self.batch.art >= 0, device, path="indexed", **kw)

    @property
    def n_real(self) -> int:
        return self.batch.n_tokens

    def bytes(self) -> float:
        """algorithmic bytes: per token q, k (bf16), v, o (bf16), g (fp32), beta (bf16); per content one fp32 trunk state
        written and read once"""
        tok = 2 * self.h * self.dk * 2 + 2 * self.hv * self.dv * 2 + self.hv * 4 + self.hv * 2
        state = 2 * self.hv * self.dk * self.dv * 4
        forks = sum(1 for t in self.trees if len(t.branches))
        return float(self.n_real * tok + forks * state)


def gdn_config(name: str, seed: int = 0, contents: int | None = None) -> GdnConfig:
    rng = np.random.default_rng(seed)
    if name == "C5":
        n = contents or 128
        trees = [_tree(rng, 2048, [12] * 32) for _ in range(n)]
        cfg = GdnConfig(name, 16, 32, 128, 128, trees)
    elif name == "smoke":
        trees = [_tree(rng, 150, [5, 12, 7]), _tree(rng, 40, [3], None)]
        cfg = GdnConfig(name, 2, 4, 128, 128, trees)
    else:
        raise ValueError(f"unknown Gated DeltaNet config {name!r}")
    cfg.batch = pack(trees)[0]
    return cfg


def gdn_inputs(cfg: GdnConfig, seed: int = 0, device="cuda"):
    """q, k ~ N(0,1) l2-normalised (eps 1e-6) bf16; v ~ N(0,1) bf16; beta = sigmoid(N(0,1)) bf16; g = -softplus(N(0,1)) fp32"""
    import torch
    import torch.nn.functional as F

    gen = torch.Generator(device="cpu").manual_seed(seed + 104729)
    n = cfg.batch.length

    def norm(x):
        return (x * torch.rsqrt(x.pow(2).sum(-1, keepdim=True) + 1e-6)).to(torch.bfloat16)

    def chunks(shape_tail, fn):
        out = torch.empty((n, *shape_tail), dtype=fn(torch.zeros(1, *shape_tail)).dtype, device=device)
        step = max(1, (1 << 23) // int(np.prod(shape_tail)))
        for a in range(0, n, step):
            b = min(n, a + step)
            out[a:b] = fn(torch.randn((b - a, *shape_tail), generator=gen)).to(device)
        return out

    return {
        "q": chunks((cfg.h, cfg.dk), norm),
        "k": chunks((cfg.h, cfg.dk), norm),
        "v": chunks((cfg.hv, cfg.dv), lambda x: x.to(torch.bfloat16)),
        "beta": chunks((cfg.hv,), lambda x: torch.sigmoid(x).to(torch.bfloat16)),
        "g": chunks((cfg.hv,), lambda x: -F.softplus(x)),
    }


# ------------------------------------------------------------------------------------------------ extraction decode step
def xdecode_case(G=4, H=16, h=8, d=256, slots=4, beam=6, S=17, prefix=(300, 470), template=(6, 14), window=None, step=None, seed=0,
                 device="cuda", layer=0):
    """A synthetic decoding step of the extraction decoder (spinf_serve/decode.py:106-171): G groups with `slots` slots each
    (Q = slots * beam queries), prefix lengths uniform in `prefix`, template lengths uniform in `template` per slot, S generated
    entries per query of which 0 .. step are written.  A sliding layer (window) stores the last window - 1 prefix tokens
    (spinf_serve/models/gemma4.py:100-106).  K, V ~ 0.5 N(0, 1) bf16, queries N(0, 1) bf16.
    -> (query [G, H, Q, d] as the transposed view of [G, Q, H, d], XCaches)"""
    import torch

    from .decode import XCaches

    rng = np.random.default_rng(seed)
    Q = slots * beam
    P = rng.integers(prefix[0], prefix[1] + 1, G)
    T = rng.integers(template[0], template[1] + 1, (G, slots))
    stored = np.minimum(P, window - 1) if window else P
    Lp, Tt = int(stored.max()), int(T.sum(1).max())
    pos_p = np.full((G, Lp), -1, np.int32)
    pos_t = np.full((G, Tt), -1, np.int32)
    own_t = np.full((G, Tt), -1, np.int32)
    qpos = np.zeros((G, Q), np.int64)
    step = S - 1 if step is None else step
    for g in range(G):
        pos_p[g, : stored[g]] = np.arange(P[g] - stored[g], P[g])
        o = 0
        for j in range(slots):
            pos_t[g, o : o + T[g, j]] = np.arange(P[g], P[g] + T[g, j])
            own_t[g, o : o + T[g, j]] = j
            o += T[g, j]
            qpos[g, j * beam : (j + 1) * beam] = P[g] + T[g, j] + step
    gen = torch.Generator().manual_seed(seed)

    def rnd(*shape, s=0.5):
        return (torch.randn(*shape, generator=gen) * s).to(torch.bfloat16).to(device)

    c = XCaches(beam=beam)
    c.kp[layer], c.vp[layer] = rnd(G, h, Lp, d), rnd(G, h, Lp, d)
    c.kt[layer], c.vt[layer] = rnd(G, h, Tt, d), rnd(G, h, Tt, d)
    c.gk[layer], c.gv[layer] = rnd(G, h, Q, S, d), rnd(G, h, Q, S, d)
    c.pos_p[layer] = torch.from_numpy(pos_p).to(device)
    c.pos_t, c.own_t = torch.from_numpy(pos_t).to(device), torch.from_numpy(own_t).to(device)
    c.qpos = torch.from_numpy(qpos).to(device)
    c.step_t = torch.full((1,), step, dtype=torch.int64, device=device)
    c.set_lengths()
    query = rnd(G, Q, H, d, s=1.0).transpose(1, 2)
    return query, c


def xdecode_bytes(c, layer=0, H=None) -> int:
    """algorithmic bytes of one step: every stored prefix / template key and value row once, the written generated entries once
    (entries 0 .. step), the queries and the outputs once"""
    kp, kt, gk = c.kp[layer], c.kt[layer], c.gk[layer]
    G, h, Lp, d = kp.shape
    Q, S = gk.shape[2], gk.shape[3]
    step = int(c.step_t.item())
    rows = int((c.pos_p[layer] >= 0).sum().item()) * h + int((c.own_t >= 0).sum().item()) * h + G * h * Q * (step + 1)
    return rows * d * 2 * 2 + 2 * G * Q * (H or h) * d * 2
