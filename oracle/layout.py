"""Stream layout of packed token trees (restates spinf_serve/packer.py:352-423, Batch fields :252-272).

A job is a shared prefix (the trunk) followed by branches in pre-order; ``parents[b]`` names the branch that
branch b continues (-1: the prefix).  The stream holds, per token:

  pos   depth of the token on its root-to-leaf path                          (packer.py:378,398)
  seg   0 for the prefix, b+1 for branch b, -1 for pads                      (packer.py:379,399)
  art   slot of the job inside the stream, -1 for pads                       (packer.py:385,396)
  end   exclusive end of the token's subtree (job end for prefix tokens)     (packer.py:402-408)
  prev  the token before it on its path, -1 at a job's first token and pads  (packer.py:380,394-395)

Test infrastructure only (see oracle/__init__.py).
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

BLOCK = 128  # packer.py:22


def ceil_block(n: int) -> int:
    return -(-n // BLOCK) * BLOCK


@dataclass
class Job:
    prefix: list            # token ids of the trunk
    branches: list          # list of token-id lists, pre-order
    parents: list = field(default_factory=list)   # [] = every branch continues the prefix
    aligned: tuple = ()     # branch indices that start on a BLOCK boundary relative to the job start

    @property
    def n_tokens(self) -> int:   # packer.py:129-138 (GroupedTree.n_tokens counts the gaps before aligned branches)
        n = len(self.prefix)
        for b, br in enumerate(self.branches):
            if b in self.aligned:
                n = ceil_block(n)
            n += len(br)
        return n


@dataclass
class Stream:
    ids: np.ndarray
    pos: np.ndarray
    seg: np.ndarray
    art: np.ndarray
    end: np.ndarray
    prev: np.ndarray
    starts: list            # per job: (stream start, [branch starts])
    n_real: int


def pack_stream(jobs, align: bool = False, length: int | None = None) -> Stream:
    """Lay the jobs out back to back (packer.py:364-422).  ``length``: stream length (default: whole blocks)."""
    cursor = 0
    rows = []   # (ids, pos, seg, art, end, prev) per token, appended job by job
    spans = []
    # first pass: positions
    layout = []
    for a, job in enumerate(jobs):
        s0 = cursor
        P = len(job.prefix)
        parents = list(job.parents) if job.parents else [-1] * len(job.branches)
        cursor += P
        starts, depth = [], []
        for b, br in enumerate(job.branches):
            pa = parents[b]
            depth.append(0 if pa < 0 else depth[pa] + len(job.branches[pa]))        # packer.py:388
            if b in job.aligned:
                cursor = s0 + ceil_block(cursor - s0)                                # packer.py:390-391
            starts.append(cursor)
            cursor += len(br)
        layout.append((s0, P, parents, starts, depth, cursor))
        if align:
            cursor = ceil_block(cursor)                                              # packer.py:421-422
    n = ceil_block(cursor) if length is None else length
    if n < cursor:
        raise ValueError("stream length too short for the jobs")
    ids = np.zeros(n, np.int64)
    pos = np.zeros(n, np.int32)
    seg = np.full(n, -1, np.int32)
    art = np.full(n, -1, np.int32)
    end = np.full(n, -1, np.int32)
    prev = np.full(n, -1, np.int64)
    real = 0
    for a, (job, (s0, P, parents, starts, depth, job_end)) in enumerate(zip(jobs, layout)):
        for i in range(P):
            t = s0 + i
            ids[t], pos[t], seg[t], art[t], end[t] = job.prefix[i], i, 0, a, job_end
            prev[t] = t - 1 if i else -1
        # subtree sizes: children fold into parents, last branch first (packer.py:403-406)
        size = [len(br) for br in job.branches]
        for b in range(len(size) - 1, -1, -1):
            if parents[b] >= 0:
                size[parents[b]] += size[b]
        for b, br in enumerate(job.branches):
            pa = parents[b]
            for i, tok in enumerate(br):
                t = starts[b] + i
                ids[t], pos[t], seg[t], art[t] = tok, P + depth[b] + i, b + 1, a
                end[t] = starts[b] + size[b]
                if i:
                    prev[t] = t - 1
                elif pa >= 0:
                    prev[t] = starts[pa] + len(job.branches[pa]) - 1                 # packer.py:394
                else:
                    prev[t] = s0 + P - 1 if P else -1
        real += P + sum(len(br) for br in job.branches)
        spans.append((s0, starts))
    return Stream(ids, pos, seg, art, end, prev, spans, real)
