"""Host-side tree packing with the reference's interface (spinf_serve/packer.py): the metadata producer of the
tree-mask attention path.

A job = one content (the shared prefix, read once as a causal trunk) and its question branches in pre-order; jobs are
laid back to back into streams.  The stream metadata (``Batch.art / end / pos / prev``) is everything the attention
kernels and the recurrent-layer planner need: token q sees token k <= q of its job iff q < end[k]
(spinf_serve/scorer.py:173-177).

Names, fields, argument meaning and errors follow the reference (Tree :25-35, build_tree :38-64, ReadPlan :67-104,
GroupedTree :107-138, trie_branches :141-185, build_grouped_tree :188-198, split_* :201-233, Owner :236-249,
Batch :252-272, Packer :275-423).  Media (image groups) are outside this path and not carried.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

BLOCK = 128  # jobs align to it, streams are multiples of it (spinf_serve/packer.py:22)


def _up(n: int) -> int:
    return (n + BLOCK - 1) & ~(BLOCK - 1)


def _common_prefix(prompt_ids) -> int:
    """length of the prompts' shared prefix, leaving every prompt at least one token of its own (packer.py:44-47)"""
    if not prompt_ids:
        raise ValueError("a job needs at least one prompt")
    first = prompt_ids[0]
    limit = min(len(x) for x in prompt_ids) - 1
    p = 0
    while p < limit and all(x[p] == first[p] for x in prompt_ids):
        p += 1
    return p


@dataclass
class Tree:
    prefix: list
    branches: list
    reads: list          # (branch, offset in the branch, target token, prompt, option)
    n_options: list      # per prompt

    @property
    def n_tokens(self) -> int:
        return len(self.prefix) + sum(len(b) for b in self.branches)


def build_tree(prompt_ids, option_ids) -> Tree:
    """One branch per prompt plus one per distinct multi-token lead-in; option token j is read at the position of token
    j-1 (chain rule), so options that share a lead-in share its branch (packer.py:38-64)."""
    p = _common_prefix(prompt_ids)
    if len(prompt_ids) != len(option_ids):
        raise ValueError("prompt_ids and option_ids differ in length")
    branches, reads = [], []
    for c, (ids, opts) in enumerate(zip(prompt_ids, option_ids)):
        own = list(ids[p:])
        slot = {(): len(branches)}
        branches.append(own)
        for o, toks in enumerate(opts):
            if not toks:
                raise ValueError(f"prompt {c}: option {o} is empty")
            for j, tok in enumerate(toks):
                lead = tuple(toks[:-1]) if j else ()
                if lead not in slot:
                    slot[lead] = len(branches)
                    branches.append(own + list(lead))
                reads.append((slot[lead], len(own) - 1 + j, tok, c, o))
    return Tree(list(prompt_ids[0][:p]), branches, reads, [len(o) for o in option_ids])


@dataclass(eq=False)
class ReadPlan:
    """Rows and entries to read a prompt's options (packer.py:67-104): row 0 is the prompt's last token, every distinct
    lead-in L = option[:-1] adds len(L) rows; entry e adds log P(entry_tok[e]) at entry_row[e] to option entry_opt[e]."""

    leadins: list
    entry_row: np.ndarray
    entry_tok: np.ndarray
    entry_opt: np.ndarray
    n_opts: int
    n_rows: int

    @classmethod
    def build(cls, option_ids) -> "ReadPlan":
        first_row: dict = {}
        rows, toks, opts = [], [], []
        n_rows = 1
        for o, t in enumerate(option_ids):
            if not t:
                raise ValueError(f"option {o} is empty")
            rows.append(0); toks.append(t[0]); opts.append(o)
            if len(t) == 1:
                continue
            lead = tuple(t[:-1])
            if lead not in first_row:
                first_row[lead] = n_rows
                n_rows += len(lead)
            base = first_row[lead]
            rows.extend(range(base, base + len(t) - 1)); toks.extend(t[1:]); opts.extend([o] * (len(t) - 1))
        i64 = lambda x: np.asarray(x, np.int64)  # noqa: E731
        return cls(list(first_row), i64(rows), i64(toks), i64(opts), len(option_ids), n_rows)


@dataclass
class GroupedTree:
    """A job read through ReadPlans (packer.py:107-138).  parents[b]: the branch that b continues (-1 the prefix),
    branches in pre-order; aligned: branches that start on a BLOCK boundary relative to the job's start."""

    prefix: list
    branches: list
    prompt_rows: list
    plans: list
    media: list = field(default_factory=list)
    xbranches: list = field(default_factory=list)
    parents: list = field(default_factory=list)
    aligned: list = field(default_factory=list)

    @property
    def n_tokens(self) -> int:
        n = len(self.prefix)
        marks = set(self.aligned)
        for b, br in enumerate(self.branches):
            n = (_up(n) if b in marks else n) + len(br)
        return n


def trie_branches(suffixes, plans):
    """Suffixes (+ each plan's lead-ins under its suffix) as one token trie; a branch is a maximal chain without a fork
    (packer.py:141-185).  -> (branches in pre-order, parents, prompt_rows[c] = [(branch, offset)] per read row)."""
    child = [{}]      # node -> {token: node}; node 0 = end of the shared prefix
    token = [-1]

    def descend(node, seq):
        out = []
        for t in seq:
            nxt = child[node].get(t)
            if nxt is None:
                nxt = len(child)
                child[node][t] = nxt
                child.append({})
                token.append(t)
            out.append(nxt)
            node = nxt
        return out

    if len(suffixes) != len(plans):
        raise ValueError("suffixes and plans differ in length")
    read_nodes = []
    for suf, plan in zip(suffixes, plans):
        tail = descend(0, suf)[-1]
        nodes = [tail]
        for lead in plan.leadins:
            nodes.extend(descend(tail, lead))
        read_nodes.append(nodes)
    where = {}
    branches, parents = [], []
    todo = [(n, -1) for n in reversed(list(child[0].values()))]
    while todo:
        node, par = todo.pop()
        b = len(branches)
        chain = []
        while True:
            where[node] = (b, len(chain))
            chain.append(token[node])
            if len(child[node]) != 1:
                break
            node = next(iter(child[node].values()))
        branches.append(chain)
        parents.append(par)
        todo.extend((n, b) for n in reversed(list(child[node].values())))
    return branches, parents, [[where[n] for n in nodes] for nodes in read_nodes]


def build_grouped_tree(prompt_ids, plans) -> GroupedTree:
    p = _common_prefix(prompt_ids)
    branches, parents, rows = trie_branches([list(x[p:]) for x in prompt_ids], plans)
    return GroupedTree(list(prompt_ids[0][:p]), branches, rows, list(plans), parents=parents)


def _halve(n_prompts, make, budget):
    """contiguous runs of prompts that each fit the budget, halving (packer.py:201-233)"""
    done = []
    work = [(0, n_prompts)]
    while work:
        a, b = work.pop()
        t = make(a, b)
        if t.n_tokens <= budget:
            done.append((a, t))
        elif b - a == 1:
            raise ValueError(f"prompt {a} alone is {t.n_tokens} tokens, over the budget {budget}")
        else:
            m = (a + b) // 2
            work.extend([(m, b), (a, m)])
    done.sort(key=lambda it: it[0])
    return done


def split_trees(prompt_ids, option_ids, budget):
    return _halve(len(prompt_ids), lambda a, b: build_tree(prompt_ids[a:b], option_ids[a:b]), budget)


def split_grouped_trees(prompt_ids, plans, budget):
    return _halve(len(prompt_ids), lambda a, b: build_grouped_tree(prompt_ids[a:b], plans[a:b]), budget)


@dataclass
class Owner:
    job_id: object
    n_rows: int
    n_tokens: int
    plan: list
    n_options: list
    row_start: np.ndarray | None = None
    plans: list | None = None
    start: int = 0
    prefix_len: int = 0
    xbranches: list = field(default_factory=list)


@dataclass
class Batch:
    ids: np.ndarray   # [N] int64
    pos: np.ndarray   # [N] int32 depth on the path
    seg: np.ndarray   # [N] int32 0 prefix, b branch b, -1 pad
    art: np.ndarray   # [N] int32 job slot, -1 pad
    sel: np.ndarray   # read rows
    owners: list
    n_tokens: int
    media: list = field(default_factory=list)
    grp: np.ndarray | None = None
    end: np.ndarray | None = None    # [N] int32 exclusive end of the token's subtree, -1 pad
    prev: np.ndarray | None = None   # [N] int64 path predecessor, -1 none

    @property
    def length(self) -> int:
        return len(self.ids)


class Packer:
    """First-fit-decreasing packing of jobs into streams of at most ``budget`` tokens (packer.py:275-350).  align: every job
    starts on a BLOCK boundary, which is what makes a job's attention tiles independent of its neighbours."""

    def __init__(self, budget, max_tokens=None, align=False, min_stream=0, cost=None, cost_budget=0):
        self.budget = _up(budget)
        self.max_tokens = max(self.budget, (max_tokens or 0) + BLOCK - 1) // BLOCK * BLOCK
        self.align = align
        self.min_stream = min(self.budget, _up(min_stream)) if align else 0
        self.cost, self.cost_budget = cost, cost_budget
        self.buf = []

    # ---- queueing
    def push(self, job_id, tree, window=96):
        n = tree.n_tokens
        if n > self.max_tokens:
            raise ValueError(f"job {job_id}: {n} tokens exceed the maximum {self.max_tokens}")
        if n > self.budget:                       # a long document runs alone, at once
            yield self._pack([(job_id, tree)], self._length(n))
            return
        self.buf.append((job_id, tree))
        if len(self.buf) >= window:
            yield from self._flush(False)

    def flush(self):
        yield from self._flush(True)

    def _length(self, n):
        return max(_up(n), self.min_stream)

    def _size(self, tree):
        return _up(tree.n_tokens) if self.align else tree.n_tokens

    def _flush(self, final):
        bins = []   # [tokens, items, cost]
        for item in sorted(self.buf, key=lambda it: -it[1].n_tokens):   # stable: ties keep arrival order
            n = self._size(item[1])
            c = self.cost(item[1]) if self.cost is not None else 0
            home = next((b for b in bins if b[0] + n <= self.budget and (c == 0 or b[2] + c <= self.cost_budget)), None)
            if home is None:
                bins.append([n, [item], c])
            else:
                home[0] += n
                home[1].append(item)
                home[2] += c
        self.buf = []
        if not final and len(bins) > 1:           # the least full stream waits for the next window
            bins.sort(key=lambda b: -b[0])
            self.buf = bins.pop()[1]
        for n, items, _ in bins:
            yield self._pack(items, self._length(n))

    # ---- layout
    def _pack(self, items, n) -> Batch:
        ids = np.zeros(n, np.int64)
        pos = np.zeros(n, np.int32)
        seg = np.full(n, -1, np.int32)
        art = np.full(n, -1, np.int32)
        end = np.full(n, -1, np.int32)
        prev = np.full(n, -1, np.int64)
        sel, owners = [], []
        cursor = real = 0
        for slot, (job_id, t) in enumerate(items):
            if getattr(t, "media", None):
                raise NotImplementedError("media prefixes are outside the tree-mask attention path")
            grouped = isinstance(t, GroupedTree)
            nb = len(t.branches)
            lens = np.fromiter((len(b) for b in t.branches), np.int64, nb)
            parents = np.asarray(getattr(t, "parents", None) or [-1] * nb, np.int64)
            marks = set(getattr(t, "aligned", ()))
            P = len(t.prefix)
            s0 = cursor
            # branch starts (gaps before aligned branches) and depths (sum of the ancestors' lengths)
            start = np.empty(nb, np.int64)
            depth = np.zeros(nb, np.int64)
            k = s0 + P
            for b in range(nb):
                if parents[b] >= 0:
                    depth[b] = depth[parents[b]] + lens[parents[b]]
                if b in marks:
                    k = s0 + _up(k - s0)
                start[b] = k
                k += lens[b]
            job_end = k
            # subtree sizes, children folded into parents from the back (pre-order: children follow parents)
            size = lens.copy()
            for b in range(nb - 1, -1, -1):
                if parents[b] >= 0:
                    size[parents[b]] += size[b]
            # prefix
            sl = slice(s0, s0 + P)
            ids[sl] = t.prefix
            pos[sl] = np.arange(P)
            seg[sl] = 0
            art[sl] = slot
            end[sl] = job_end
            prev[s0 + 1 : s0 + P] = np.arange(s0, s0 + P - 1)
            # branches
            for b in range(nb):
                L = int(lens[b])
                if not L:
                    continue
                a0 = int(start[b])
                sl = slice(a0, a0 + L)
                ids[sl] = t.branches[b]
                pos[sl] = np.arange(P + depth[b], P + depth[b] + L)
                seg[sl] = b + 1
                art[sl] = slot
                end[sl] = a0 + size[b]
                prev[a0 + 1 : a0 + L] = np.arange(a0, a0 + L - 1)
                pa = parents[b]
                prev[a0] = (start[pa] + lens[pa] - 1) if pa >= 0 else (s0 + P - 1 if P else -1)
            real += P + int(lens.sum())
            if grouped:
                n0 = len(sel)
                row_start = np.empty(len(t.prompt_rows), np.int64)
                for c, rows in enumerate(t.prompt_rows):
                    row_start[c] = len(sel) - n0
                    sel.extend(int(start[b]) + off for b, off in rows)
                xb = [(int(start[b]), int(lens[b]), pr) if b >= 0 else (s0 + P, 0, pr) for b, pr in t.xbranches]
                owners.append(Owner(job_id, len(sel) - n0, job_end - s0, [], [pl.n_opts for pl in t.plans], row_start, t.plans, s0, P, xb))
            else:
                first, plan, n0 = {}, [], len(sel)
                for b, off, tgt, c, side in t.reads:      # one row per distinct position (packer.py:338-350)
                    qpos = int(start[b]) + off
                    if qpos not in first:
                        first[qpos] = len(sel) - n0
                        sel.append(qpos)
                    plan.append((first[qpos], tgt, c, side))
                owners.append(Owner(job_id, len(sel) - n0, job_end - s0, plan, t.n_options, start=s0))
            cursor = _up(job_end) if self.align else job_end
        return Batch(ids, pos, seg, art, np.asarray(sel, np.int64), owners, real, [], None, end, prev)
