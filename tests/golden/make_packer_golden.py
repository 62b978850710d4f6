"""Writes tests/golden/packer_golden.json.gz: input trees and the stream metadata, block tables and recurrent-layer plans
that the reference's host code produces for them.

Run once, in the build container only (the reference tree is not present anywhere else):

    python tests/golden/make_packer_golden.py /root/reference

It imports spinf_serve.packer (numpy only) and spinf_serve.models.qwen35.qwen.tree_plan (host numpy code, device "cpu")
from the path given and stores plain integers.  The parts of those functions that the reference's own tests pin only by
invariants (the exact first-fit-decreasing stream order of Packer._flush, block_tables' full/partial split on arbitrary
input, tree_plan's call partition and slot numbering) are what these vectors add.
"""

import gzip
import json
import os
import random
import sys

import numpy as np


def main(ref):
    sys.path.insert(0, ref)
    from spinf_serve.packer import Packer, ReadPlan, block_tables, build_grouped_tree, build_tree, GroupedTree

    try:
        from spinf_serve.models.qwen35.qwen import tree_plan
    except Exception as e:  # noqa: BLE001
        print("tree_plan not importable:", repr(e))
        tree_plan = None

    rng = random.Random(20261125)
    cases = []

    def rand_tree(two_level=False, aligned=False):
        P = rng.randrange(1, 400)
        prefix = [rng.randrange(5, 90) for _ in range(P)]
        if two_level:
            branches, parents = [], []
            for _ in range(rng.randrange(1, 5)):
                node = len(branches)
                branches.append([rng.randrange(5, 90) for _ in range(rng.randrange(1, 40))])
                parents.append(-1)
                for _ in range(rng.randrange(0, 6)):
                    leaf = len(branches)
                    branches.append([rng.randrange(5, 90) for _ in range(rng.randrange(1, 12))])
                    parents.append(node)
                    if rng.random() < 0.3:
                        branches.append([rng.randrange(5, 90) for _ in range(rng.randrange(1, 5))])
                        parents.append(leaf)
        else:
            branches = [[rng.randrange(5, 90) for _ in range(rng.randrange(1, 30))] for _ in range(rng.randrange(1, 20))]
            parents = [-1] * len(branches)
        al = []
        if aligned:
            roots = [b for b, p in enumerate(parents) if p < 0]
            al = sorted(rng.sample(roots, min(len(roots), 2)))
        return GroupedTree(prefix, branches, [], [], parents=parents, aligned=al)

    def dump_batch(b, window):
        full, sliding = block_tables(b.art, b.end, b.pos, window, always_window=True)

        def tabs(t):
            pn, pi, fn, fi = t
            return {"partial": [pi[i, : pn[i]].tolist() for i in range(len(pn))], "full": [fi[i, : fn[i]].tolist() for i in range(len(fn))]}

        out = {
            "ids": b.ids.tolist(), "pos": b.pos.tolist(), "seg": b.seg.tolist(), "art": b.art.tolist(), "end": b.end.tolist(),
            "prev": b.prev.tolist(), "n_tokens": int(b.n_tokens), "owners": [[int(o.job_id), int(o.start), int(o.n_tokens), int(o.prefix_len)] for o in b.owners],
            "window": window, "tables_full": tabs(full), "tables_sliding": tabs(sliding) if sliding is not None else None,
        }
        if tree_plan is not None:
            real = b.art >= 0
            for short, call_tokens in ((64, 8192), (4, 300)):
                pl = tree_plan(b.prev, real, "cpu", path="indexed", short=short, call_tokens=call_tokens)
                lv = []
                for calls in pl.levels:
                    lv.append([{"kind": c.kind, "idx": c.idx.tolist(), "cu": c.cu.tolist(),
                                "h0_idx": None if c.h0_idx is None else c.h0_idx.tolist(),
                                "ht_idx": None if c.ht_idx is None else c.ht_idx.tolist()} for c in calls])
                out[f"plan_short{short}_ct{call_tokens}"] = {"levels": lv, "n_keep": [int(x) for x in pl.n_keep], "n_segments": int(pl.n_segments),
                                                           "conv": pl.conv.tolist()}
        return out

    for trial in range(6):
        align = trial % 2 == 0
        trees = [rand_tree(two_level=(trial >= 2), aligned=(trial >= 4)) for _ in range(rng.randrange(2, 7))]
        pk = Packer(2048, 4096, align=align, min_stream=1024 if trial == 0 else 0)
        batches = []
        for k, t in enumerate(trees):
            batches += list(pk.push(k, t, window=4))
        batches += list(pk.flush())
        cases.append({
            "align": align, "budget": 2048, "max_tokens": 4096, "min_stream": 1024 if trial == 0 else 0, "push_window": 4,
            "trees": [{"prefix": t.prefix, "branches": t.branches, "parents": t.parents, "aligned": list(t.aligned)} for t in trees],
            "batches": [dump_batch(b, window=(256, 512, 100)[trial % 3]) for b in batches],
        })
    # the flat Tree path (build_tree) with reads
    t = build_tree([[1, 5, 6, 7], [1, 5, 6, 8, 9]], [[[10], [11]], [[12], [13, 14]]])
    flat = {"prefix": t.prefix, "branches": t.branches, "reads": [list(r) for r in t.reads], "n_options": t.n_options}
    gt = build_grouped_tree([[1, 2, 5, 6, 7, 8], [1, 2, 5, 6, 7, 9], [1, 2, 4]],
                            [ReadPlan.build([[30], [31]]), ReadPlan.build([[30], [31]]), ReadPlan.build([[20], [21, 22], [21, 23]])])
    grouped = {"prefix": gt.prefix, "branches": gt.branches, "parents": gt.parents, "prompt_rows": [[list(x) for x in r] for r in gt.prompt_rows]}
    here = os.path.dirname(os.path.abspath(__file__))
    with gzip.open(os.path.join(here, "packer_golden.json.gz"), "wt") as f:
        json.dump({"cases": cases, "build_tree": flat, "build_grouped_tree": grouped}, f, separators=(",", ":"))
    print("wrote", len(cases), "cases,", sum(len(c["batches"]) for c in cases), "batches")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
