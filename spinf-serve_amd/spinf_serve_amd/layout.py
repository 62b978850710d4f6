"""Stream layout of packed token trees: the half of the reference's packer that the attention path depends on
(Packer._pack, spinf_serve/packer.py:352-423, Batch fields :252-272).

A job is a trunk (prefix) and branches in pre-order (a branch's parent comes before it); the stream holds the jobs back to back,
each job starting on a 128-token boundary when ``align`` (that is what makes a job's attention tiles independent of its
neighbours).  Per token the layout gives what the mask rule (spinf_serve/scorer.py:173-177) and the recurrent plan need:

  pos   depth on the token's root-to-leaf path            seg   0 trunk, b + 1 branch b, -1 pad
  art   slot of the job in the stream, -1 pad             end   exclusive end of the token's subtree (trunk: the job's end)
  prev  the token before it on its path, -1 none

The request front end of the reference's packer (lead-ins, read plans, option tries, windowed bin packing with a cost budget) is
not part of this package: the reference keeps it.  ``pack_streams`` is a plain first-fit-decreasing split for the synthetic
workloads only.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

BLOCK = 128   # spinf_serve/packer.py:22


def ceil_block(n: int) -> int:
    return -(-int(n) // BLOCK) * BLOCK


@dataclass
class TokenTree:
    """prefix: trunk token ids; branches: token id lists in pre-order; parents[b]: branch index of b's parent, -1 = the trunk;
    aligned: branches that start on a 128-token boundary relative to the job's start (query groups)"""
    prefix: list
    branches: list
    parents: list = field(default_factory=list)
    aligned: tuple = ()

    def __post_init__(self):
        if not self.parents:
            self.parents = [-1] * len(self.branches)
        if len(self.parents) != len(self.branches):
            raise ValueError("one parent per branch")
        for b, pa in enumerate(self.parents):
            if not -1 <= pa < b:
                raise ValueError(f"branch {b}: parent {pa} does not come before it")

    def starts(self):
        """offsets of the branches relative to the job's start, and the job's length"""
        k = len(self.prefix)
        marks = set(self.aligned)
        out = np.empty(len(self.branches), np.int64)
        for b, br in enumerate(self.branches):
            if b in marks:
                k = ceil_block(k)
            out[b] = k
            k += len(br)
        return out, k

    @property
    def n_tokens(self) -> int:
        return int(self.starts()[1])


@dataclass
class Batch:
    ids: np.ndarray    # [N] int64
    pos: np.ndarray    # [N] int32
    seg: np.ndarray    # [N] int32
    art: np.ndarray    # [N] int32
    end: np.ndarray    # [N] int32
    prev: np.ndarray   # [N] int64
    n_tokens: int      # real tokens
    jobs: list = field(default_factory=list)   # per job: (start, length incl. gaps, trunk length, index of its tree in the list given)
    grp: np.ndarray | None = None

    @property
    def length(self) -> int:
        return len(self.ids)


def pack_stream(trees, align: bool = True, min_stream: int = 0, length: int | None = None) -> Batch:
    """Lay the jobs out in the given order.  length: the stream's length (default: whole blocks, at least min_stream)."""
    spans = [t.starts() for t in trees]
    cursor, job_start = 0, []
    for _, job_len in spans:
        job_start.append(cursor)
        cursor += ceil_block(job_len) if align else job_len
    n = max(ceil_block(cursor), ceil_block(min_stream)) if length is None else int(length)
    if spans and n < job_start[-1] + spans[-1][1]:
        raise ValueError(f"a stream of {n} tokens does not hold the jobs ({job_start[-1] + spans[-1][1]})")
    ids = np.zeros(n, np.int64)
    pos = np.zeros(n, np.int32)
    seg = np.full(n, -1, np.int32)
    art = np.full(n, -1, np.int32)
    end = np.full(n, -1, np.int32)
    prev = np.full(n, -1, np.int64)
    jobs, real = [], 0
    for slot, (t, (rel, job_len), s0) in enumerate(zip(trees, spans, job_start)):
        P, nb = len(t.prefix), len(t.branches)
        lens = np.fromiter((len(b) for b in t.branches), np.int64, nb)
        parents = np.asarray(t.parents, np.int64)
        # trunk
        trunk = np.arange(s0, s0 + P)
        ids[trunk] = t.prefix
        pos[trunk] = np.arange(P)
        seg[trunk] = 0
        art[trunk] = slot
        end[trunk] = s0 + job_len
        prev[trunk[1:]] = trunk[:-1]
        if nb:
            start = s0 + rel
            # depth of a branch = tokens of its ancestor branches; size of its subtree = its own tokens and its descendants'
            depth = np.zeros(nb, np.int64)
            size = lens.copy()
            for b in range(nb):
                if parents[b] >= 0:
                    depth[b] = depth[parents[b]] + lens[parents[b]]
            for b in range(nb - 1, -1, -1):
                if parents[b] >= 0:
                    size[parents[b]] += size[b]
            # every branch token at once
            owner = np.repeat(np.arange(nb), lens)
            offs = np.arange(int(lens.sum())) - np.repeat(np.cumsum(lens) - lens, lens)
            at = start[owner] + offs
            ids[at] = np.concatenate([np.asarray(b, np.int64) for b in t.branches]) if len(at) else []
            pos[at] = P + depth[owner] + offs
            seg[at] = owner + 1
            art[at] = slot
            end[at] = (start + size)[owner]
            prev[at] = at - 1
            # a branch's first token continues its parent's last token (or the trunk's, or nothing without a trunk)
            heads = lens > 0
            last_of_parent = np.where(parents >= 0, start[np.maximum(parents, 0)] + lens[np.maximum(parents, 0)] - 1, s0 + P - 1 if P else -1)
            prev[start[heads]] = last_of_parent[heads]
        jobs.append((s0, int(job_len), P, slot))
        real += P + int(lens.sum())
    return Batch(ids, pos, seg, art, end, prev, real, jobs)


def pack_streams(trees, budget: int, align: bool = True) -> list:
    """First-fit-decreasing split of the jobs into streams of at most ``budget`` tokens (ties keep the given order); for the
    synthetic workloads."""
    budget = ceil_block(budget)
    size = [ceil_block(t.n_tokens) if align else t.n_tokens for t in trees]
    bins = []   # [tokens, job indices]
    for i in sorted(range(len(trees)), key=lambda i: -trees[i].n_tokens):
        if size[i] > budget:
            raise ValueError(f"job {i}: {size[i]} tokens exceed the stream budget {budget}")
        home = next((b for b in bins if b[0] + size[i] <= budget), None)
        if home is None:
            bins.append([size[i], [i]])
        else:
            home[0] += size[i]
            home[1].append(i)
    out = []
    for _, members in bins:
        b = pack_stream([trees[i] for i in members], align=align)
        b.jobs = [(s0, n, P, members[k]) for s0, n, P, k in b.jobs]
        out.append(b)
    return out
