"""Benchmark of the tree-mask packed-prefill attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K=200] [--warmup W=100] [--workload C2|C2_stream|C3|C4|C5|XDEC|LM|LM_head|copy|mfma_peak|mfma_valu ...] [--seed S] [--no-cpu]

A step is one pass of the attention op (one layer's call through the C ABI) over one packed synthetic stream already
resident in HBM; the tile plan is compiled once per stream, outside the timed region, as the reference builds its block
masks once per forward for all layers.  Prints ONE JSON line: packed query tokens/s, the useful-FLOP roofline fraction of
the kernel (events on the launch stream around every step) and the CPU baseline (dense-mask attention on the host cores).
Before the W warm-up steps the step is run untimed for SPINUP_S seconds, so that the timed steps see the GPU's sustained clocks.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "spinf-serve_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA (published)
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E (published)

WORKLOADS = {
    "C2": "C2: 24 contents x (470-token trunk + 56 branches of U{8..16} tokens) in one varlen pass, 16 query / 8 KV heads, head_dim 256, scale 1/16, Q/K/V ~ 0.5 N(0,1), global layer",
    "C2_512": "C2's stream at the head geometry of the Gemma-4 full-attention layers: 16 query heads / 1 KV head, head_dim 512, global layer",
    "C3": "C3: 512 contents, trunk lognormal(median 800, sigma 0.6) clipped 64..4096, U{8..64} branches of U{4..24}, passes <= 65,536 tokens, 16/8 heads, head_dim 256, one sliding (W=1024) + one global layer per pass",
    "C4": "C4: contents x (8192-token trunk + 16 nodes x 32 + 192 leaves of U{6..10}), 32/16 heads, head_dim 128, one varlen pass",
    "C2_stream": "C2's byte pattern with nothing computed: the same work items on the same static schedule, query loads, every K / V tile through the LDS ring by the same DMA requests (four in flight), output stores in the kernel's pattern; no MFMA, no softmax, no mask (spinf_diag_attn_stream)",
    "copy": "plain device copy of 1 GiB (reads 1 GiB, writes 1 GiB per launch): the yardstick the FETCH_SIZE / WRITE_SIZE counters are scaled by",
    "C5": "C5: Gated DeltaNet, contents x (2048-token trunk + 32 branches x 12), 16 qk / 32 v heads, 128 x 128 fp32 state",
    "C5_prologue": "C5's stream through the Gated DeltaNet layer's prologue: path convolution (4 taps) + silu + q/k l2 norm + beta + g from the input projection's rows",
    "C5_gate": "C5's stream through the Gated DeltaNet layer's output gate: per-head rms norm x norm_w x silu(z)",
    "XDEC": "extraction-decode attention step: 24 groups x (470-token prefix + 8 slots with templates of U{8..16} tokens) x 6 beams = 48 queries per group, 33 generated entries per query all written (step 32), 16 query / 8 KV heads, head_dim 256, scale 1/16, global layer",
    "XDEC_long": "extraction-decode attention step: 64 groups x (U{1024..4096}-token prefix + 8 slots with templates of U{8..16} tokens) x 6 beams, 33 generated entries (step 32), 16 / 8 heads, head_dim 256, global layer",
    "XDEC_qwen": "XDEC's step at the Qwen-hybrid attention geometry: 24 query heads / 4 KV heads, head_dim 256 (288 rows per (group, kv head): three row chunks)",
    "XDEC_512": "XDEC's step at the head geometry of the Gemma-4 full-attention layers: 16 query heads / 1 KV head, head_dim 512 (output computed 256 head dims at a time, two launches)",
    "mfma_valu": "rounds of one v_mfma_f32_32x32x16_bf16 and nv independent vector instructions per wave, one, two and four waves per SIMD: clocks per round of a wave and of its SIMD (spinf_diag_mfma_valu)",
    "mfma_peak": "pure v_mfma_f32_32x32x16_bf16 loop, one workgroup of eight waves on every compute unit, operands in registers: the yardstick for what the matrix cores sustain on this part",
    "LM_head": "lm head of one chunk of 1,024 read rows gathered from a 65,536-row stream: h[sel] W^T (hidden 2,560, vocabulary 262,144, bf16 MFMA, fp32 logits) + soft-capping (30) + log-softmax + 8 option columns in one pass, no logits matrix",
    "LM": "lm head read-out of one chunk of 1,024 read rows: soft-capping (30) + log-softmax over 262,144 fp32 logits + 8 option columns",
}


# HBM bytes per launch of the dominant kernel(s), from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of this file (KiB per
# dispatch), each scaled by what the same counter reads for `--workload copy` (whose traffic is known).  The figures and the
# commands are in profiles/*_counters.md; a workload without a counter run has None.
TRAFFIC_BYTES = {"C2": 786_454_852, "C2_512": 1_301_296_466, "C3": 49_766_912_684, "C4": 22_633_866_199, "C5": 8_754_360_320, "C5_prologue": 10_777_077_760, "C5_gate": 7_650_867_200,
                 "XDEC": 525_321_216, "XDEC_long": 2_324_807_680}


SPINUP_S = 0.3    # untimed, before the warm-up steps: keeps the GPU busy until its clocks have come up from idle


def timed(fn, steps, warmup, torch):
    """-> (wall seconds of the `steps` timed steps, [event milliseconds per step] * steps).  The timed steps follow each other
    with nothing between them: ONE pair of events around all of them, on the stream they are launched on (an event recorded
    between two launches costs the GPU ~5 us of idling, which is 4 % of a C2 step if every step is bracketed).  The shortest
    single step, from a second, untimed pass that does bracket every step, is left in timed.min_ms."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < SPINUP_S:
        fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per_step = a.elapsed_time(b) / steps
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(min(steps, 20))]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    timed.min_ms = min(a.elapsed_time(b) for a, b in ev)
    return wall, [per_step] * steps


def mfma_rate(torch, steps=20, warmup=5, iters=4000):
    """-> (TFLOP/s, ms per launch) of the library's pure MFMA loop, events on the launch stream"""
    import ctypes as C

    import numpy as np

    from spinf_serve_amd import _lib

    lib = _lib.load_library()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.empty(cus * 512, dtype=torch.float32, device="cuda:0")
    flops = C.c_double()

    def fn():
        _lib.check(lib.spinf_diag_mfma_rate(iters, out.data_ptr(), out.numel(), C.byref(flops), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "spinf_diag_mfma_rate")

    _, kern = timed(fn, steps, warmup, torch)
    ms = float(np.mean(kern))
    return flops.value / (ms * 1e-3) / 1e12, ms


def gdn_record(sa, synth, torch, np, args, steps, warmup):
    """C5 through the Gated DeltaNet tree scan -> (record, cfg, tensors)"""
    cfg = synth.gdn_config("C5", seed=args.seed, contents=args.contents if args.workload == "C5" else None)
    t = synth.gdn_inputs(cfg, seed=args.seed, device=torch.device("cuda:0"))
    plan = cfg.plan(torch.device("cuda:0"))
    wall, kern = timed(lambda: sa.gdn_tree(t["q"], t["k"], t["v"], t["g"], t["beta"], plan), steps, warmup, torch)
    ms = float(np.mean(kern))
    gbs = cfg.bytes() / (ms * 1e-3) / 1e9
    whole = args.workload != "C5" or args.contents is None
    rec = {"metric": "packed tokens/s, Gated DeltaNet tree scan", "value": cfg.n_real * steps / wall, "unit": "tokens/s", "ms_per_step": 1e3 * wall / steps,
           "steps": steps, "warmup": warmup, "dtype": "bf16 (fp32 state)", "config": {"workload": WORKLOADS["C5"], "contents": len(cfg.trees), "tokens": cfg.n_real},
           "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                        "traffic": TRAFFIC_BYTES["C5"] if whole else None, "kernel_ms": ms, "algorithmic_bytes": cfg.bytes()}}
    return rec, cfg, t


def attn_record(sa, synth, torch, np, workload, seed, steps, warmup):
    """one of the other attention configurations, whole (every pass, every layer of a step), inputs drawn on the device -> record"""
    dev = torch.device("cuda:0")
    cfg = synth.attention_config(workload, seed=seed)
    layers = [None] if cfg.window is None else [cfg.window, None]
    work = []
    for b in cfg.batches:
        masks = sa.block_masks(b, sliding_window=cfg.window, device=dev)
        work.append((synth.qkv_device(cfg, b, seed=seed, device=dev), masks))
    torch.cuda.synchronize()

    def step():
        out = None
        for (q, k, v), masks in work:
            for w in layers:
                out = sa.tree_attn(q, k, v, masks["sliding_attention" if w else "full_attention"], cfg.scale)
        return out

    wall, kern = timed(step, steps, warmup, torch)
    ms = float(np.mean(kern))
    flops = sum(cfg.flops(w) for w in layers)
    nbytes = cfg.bytes() * len(layers)
    tfl = flops / (ms * 1e-3) / 1e12
    return {"metric": "packed query tokens/s + % bf16 MFMA peak (useful FLOPs), tree-mask attn", "value": cfg.n_real * len(layers) * steps / wall, "unit": "tokens/s",
            "ms_per_step": 1e3 * wall / steps, "steps": steps, "warmup": warmup, "dtype": "bf16", "data": "synthetic (seeded numpy trees; Q/K/V from the device generator)",
            "config": {"workload": WORKLOADS[workload], "contents": len(cfg.trees), "packed_tokens": cfg.n_real, "stream_tokens": sum(b.length for b in cfg.batches),
                       "passes": len(cfg.batches), "layers_per_step": len(layers), "visible_pairs": [cfg.pairs(w) for w in layers]},
            "roofline": {"bound": "mfma", "achieved": tfl, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tfl / PEAK_BF16_TFLOPS, "traffic": TRAFFIC_BYTES.get(workload),
                         "kernel_ms": ms, "useful_flops": flops, "algorithmic_bytes": nbytes,
                         "mfma_floor_ms": flops / (PEAK_BF16_TFLOPS * 1e12) * 1e3, "hbm_floor_ms": nbytes / (PEAK_HBM_GBS * 1e9) * 1e3}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the defaults measure the sustained rate: after idle the GPU takes about a hundred launches of this size to reach its
    # clocks (C2: 0.30 ms per launch over the first 50, 0.26 ms from the hundredth on)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="C2", choices=sorted(WORKLOADS))
    ap.add_argument("--contents", type=int, default=None, help="override the number of contents (C4 / C5 memory)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--variant", type=int, default=0)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-big", action="store_true", help="C2 only: skip the C3 / C4 sub-records")
    ap.add_argument("--parts-only", action="store_true", help="C2_stream only: time the whole pattern alone, none of its parts and variants (for a profile of one kernel shape)")
    ap.add_argument("--nsplit", type=int, default=None, help="XDEC workloads: splits of a (group, kv head) key stream (default: the library's choice)")
    ap.add_argument("--rows", default="stream", choices=["stream", "compact", "scatter"],
                    help="attention workloads: stream layout (default); compact = real rows only, read through the kernel's row map; "
                         "scatter = real rows only, scattered into stream layout and gathered back around the call (the reference's way). "
                         "The timed region then is the whole call, copies included; no CPU leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU's throughput; contents shard across GPUs with no exchange, run one process per GPU (--gpus 1)")

    import numpy as np
    import torch

    import spinf_serve_amd as sa
    from spinf_serve_amd import synth

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible (the attention op has no CPU path)")
    sa.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    line = {"metric": "packed query tokens/s + % bf16 MFMA peak (useful FLOPs), tree-mask attn", "unit": "tokens/s", "n_gpus": 1,
            "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "data": "synthetic (seeded, numpy default_rng / torch generator)", "seed": args.seed, "spinup_s": SPINUP_S}

    if args.workload == "copy":
        n = 1 << 30
        src = torch.arange(n // 4, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        wall, kern = timed(lambda: dst.copy_(src), args.steps, args.warmup, torch)
        ms = float(np.mean(kern))
        line.update(metric="device copy", unit="GB/s", value=2 * n / (ms * 1e-3) / 1e9, ms_per_step=1e3 * wall / args.steps, dtype="u8",
                    config={"workload": WORKLOADS["copy"], "bytes_read": n, "bytes_written": n},
                    roofline={"bound": "hbm", "achieved": 2 * n / (ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                              "frac": 2 * n / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": 2 * n, "kernel_ms": ms})
        print(json.dumps(line))
        return

    if args.workload == "C2_stream":
        # the floor that data movement alone sets for C2 on its schedule, and the product kernel beside it in the same run
        from spinf_serve_amd import attention

        cfg = synth.attention_config("C2", seed=args.seed, contents=args.contents)
        b = cfg.batches[0]
        mask = sa.block_masks(b, sliding_window=None, device=dev)["full_attention"]
        q, k, v = synth.qkv(cfg, b, seed=args.seed, device=dev)
        out = torch.empty_like(q)
        status = torch.zeros(2, dtype=torch.int32, device=dev)
        want = sa.tree_attn(q, k, v, mask, cfg.scale)   # (uploads the schedule)
        wall, kern = timed(lambda: attention.tree_attn_byte_pattern(q, k, v, mask, out, status), args.steps, args.warmup, torch)
        ms, ms_min = float(np.mean(kern)), float(timed.min_ms)
        gave_up = int(status[0])
        assert gave_up == 0 and bool((out == 1).all()), "the yardstick did not run to its end"
        if args.parts_only:
            line.update(metric="tree-mask attn byte pattern, nothing computed", unit="ms", value=ms, higher_is_better=False, ms_per_step=1e3 * wall / args.steps,
                        dtype="bf16", config={"workload": WORKLOADS["C2_stream"], "contents": len(cfg.trees), "packed_tokens": cfg.n_real, "stream_tokens": b.length},
                        roofline={"bound": "hbm", "achieved": cfg.bytes() / (ms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                  "frac": cfg.bytes() / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None, "kernel_ms": ms, "kernel_ms_min": ms_min})
            print(json.dumps(line))
            return
        _, kern2 = timed(lambda: sa.tree_attn(q, k, v, mask, cfg.scale), args.steps, args.warmup, torch)
        ms2 = float(np.mean(kern2))
        ms_tiles = float(np.mean(timed(lambda: attention.tree_attn_byte_pattern(q, k, v, mask, out, status, parts=1), args.steps, args.warmup, torch)[1]))
        ms_rows = float(np.mean(timed(lambda: attention.tree_attn_byte_pattern(q, k, v, mask, out, status, parts=2), args.steps, args.warmup, torch)[1]))
        by_slots = {n: float(np.mean(timed(lambda: attention.tree_attn_byte_pattern(q, k, v, mask, out, status, parts=1, nslot=n), args.steps, args.warmup, torch)[1]))
                    for n in (1, 2, 3)}
        by_slots[4] = ms_tiles
        dealt = {n: float(np.mean(timed(lambda: attention.tree_attn_byte_pattern(q, k, v, mask, out, status, parts=5, nslot=n), args.steps, args.warmup, torch)[1]))
                 for n in (1, 2, 4)}
        out.zero_()
        ms_dealt = float(np.mean(timed(lambda: attention.tree_attn_byte_pattern(q, k, v, mask, out, status, parts=7), args.steps, args.warmup, torch)[1]))
        assert int(status[0]) == 0 and bool((out == 1).all())
        plan = mask.for_head_dim(cfg.d, ring=True).plan
        tile_bytes = len(plan.kv_idx) * (cfg.hq // 2) * 32 * cfg.d * 2 * 2   # K and V of every 32-key tile of every work item: what goes into LDS
        gbs = cfg.bytes() / (ms * 1e-3) / 1e9
        line.update(metric="tree-mask attn byte pattern, nothing computed", unit="ms", value=ms, higher_is_better=False, ms_per_step=1e3 * wall / args.steps,
                    dtype="bf16", config={"workload": WORKLOADS["C2_stream"], "contents": len(cfg.trees), "packed_tokens": cfg.n_real, "stream_tokens": b.length},
                    roofline={"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS, "traffic": None,
                              "kernel_ms": ms, "kernel_ms_min": ms_min, "algorithmic_bytes": cfg.bytes(), "bytes_into_lds": tile_bytes,
                              "lds_fill_gbs": tile_bytes / (ms * 1e-3) / 1e9, "tiles_only_ms": ms_tiles, "tiles_only_ms_by_requests_in_flight": by_slots, "tiles_only_ms_requests_dealt_over_the_waves": dealt, "kernel_ms_requests_dealt_over_the_waves": ms_dealt, "queries_and_outputs_only_ms": ms_rows, "product_kernel_ms": ms2, "product_over_floor": ms2 / ms,
                              "frac_of_bf16_peak_if_the_product_ran_at_this_floor": cfg.flops(None) / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS})
        assert torch.equal(sa.tree_attn(q, k, v, mask, cfg.scale), want)
        print(json.dumps(line))
        return

    if args.workload == "mfma_valu":
        import ctypes as C

        from spinf_serve_amd import _lib

        lib = _lib.load_library()
        iters = 20000
        table = {}
        for kind, kname in ((0, "v_fma_f32"), (1, "v_exp_f32")):
            for wps in (1, 2, 4):
                for nv in (0, 2, 4, 6, 8, 12, 16):
                    out = torch.zeros(2 * 4 * wps, dtype=torch.int64, device=dev)
                    _lib.check(lib.spinf_diag_mfma_valu(nv, kind, wps, iters, out.data_ptr(), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "spinf_diag_mfma_valu")
                    torch.cuda.synchronize()
                    t = out.cpu().view(-1, 2)
                    simd0 = t[0::4]   # the waves of SIMD 0: wave 0 (the oldest, favoured by the arbiter), 4, 8, 12
                    table[f"{kname} nv={nv} waves_per_simd={wps}"] = {
                        "clocks_per_round_oldest_wave": round(float(simd0[0, 1] - simd0[0, 0]) / iters, 1),
                        "clocks_per_mfma_simd": round(float(simd0[:, 1].max() - simd0[:, 0].min()) / (iters * wps), 1)}
        for wps in (1, 2, 4):   # rounds shaped like an attention block at head dim 128 (16 MFMAs; 48 v_fma_f32 + 16 v_exp_f32 at nv = 16)
            for nv in (0, 8, 16):
                out = torch.zeros(2 * 4 * wps, dtype=torch.int64, device=dev)
                _lib.check(lib.spinf_diag_mfma_valu(nv, 2, wps, iters // 8, out.data_ptr(), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "spinf_diag_mfma_valu")
                torch.cuda.synchronize()
                simd0 = out.cpu().view(-1, 2)[0::4]
                table[f"block-shaped rounds nv={nv} waves_per_simd={wps}"] = {
                    "clocks_per_block_oldest_wave": round(float(simd0[0, 1] - simd0[0, 0]) / (iters // 8), 1),
                    "clocks_per_block_simd": round(float(simd0[:, 1].max() - simd0[:, 0].min()) / ((iters // 8) * wps), 1)}
        line.update(metric="clocks per MFMA of a SIMD, MFMA + nv vector instructions per round", unit="clocks", value=table["v_fma_f32 nv=6 waves_per_simd=2"]["clocks_per_mfma_simd"],
                    higher_is_better=False, ms_per_step=None, dtype="bf16", config={"workload": WORKLOADS["mfma_valu"], "iters": iters}, table=table)
        print(json.dumps(line))
        return

    if args.workload == "mfma_peak":
        tfl, ms = mfma_rate(torch, args.steps, args.warmup)
        line.update(metric="bf16 MFMA rate, pure loop", unit="TFLOP/s", value=tfl, ms_per_step=ms, dtype="bf16", config={"workload": WORKLOADS["mfma_peak"]},
                    roofline={"bound": "mfma", "achieved": tfl, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tfl / PEAK_BF16_TFLOPS, "traffic": None,
                              "kernel_ms": ms, "reachable_peak": tfl})
        print(json.dumps(line))
        return

    if args.workload == "LM_head":
        rows, stream, hidden, vocab, cap = 1024, 65536, 2560, 262144, 30.0
        gen = torch.Generator(device=dev).manual_seed(args.seed)
        h = torch.randn((stream, hidden), generator=gen, device=dev).to(torch.bfloat16)
        w = (torch.randn((vocab, hidden), generator=gen, device=dev) * 0.05).to(torch.bfloat16)
        sel = torch.randperm(stream, generator=gen, device=dev)[:rows].sort().values
        cols = torch.randint(0, vocab, (8,), generator=gen, device=dev)
        if args.rows == "scatter":   # the reference's own lines (scorer.py:247-254, :345-353), for comparison
            step = lambda: torch.log_softmax(torch.tanh(torch.mm(h[sel], w.t(), out_dtype=torch.float32) / cap) * cap, dim=-1)[:, cols]  # noqa: E731
        else:
            step = lambda: sa.lm_head_logprobs(h, sel, w, cols, cap)  # noqa: E731
        wall, kern = timed(step, args.steps, args.warmup, torch)
        ms = float(np.mean(kern))
        flops = 2.0 * rows * vocab * hidden
        nbytes = (vocab + rows) * hidden * 2 + rows * 8 * 4
        tfl = flops / (ms * 1e-3) / 1e12
        peak_now, _ = mfma_rate(torch)
        line.update(metric="read rows/s, lm head (GEMM + read-out in one pass)", value=rows * args.steps / wall, unit="rows/s", ms_per_step=1e3 * wall / args.steps,
                    dtype="bf16 (fp32 accumulation and read-out)",
                    config={"workload": WORKLOADS["LM_head"], "rows": rows, "vocab": vocab, "hidden": hidden, "way": "torch ops" if args.rows == "scatter" else "kernel"},
                    roofline={"bound": "mfma", "achieved": tfl, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tfl / PEAK_BF16_TFLOPS, "traffic": None,
                              "kernel_ms": ms, "useful_flops": flops, "reachable_peak": peak_now, "algorithmic_bytes": nbytes,
                              "hbm_frac_at_algorithmic_bytes": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS})
        print(json.dumps(line))
        return

    if args.workload == "LM":
        rows, vocab, cap = 1024, 262144, 30.0
        gen = torch.Generator(device=dev).manual_seed(args.seed)
        logits = torch.randn((rows, vocab), generator=gen, device=dev) * 12
        cols = torch.randint(0, vocab, (8,), generator=gen, device=dev)
        if args.rows == "scatter":   # the reference's own lines (scorer.py:351-353, :254), for comparison
            step = lambda: torch.log_softmax((torch.tanh(logits / cap) * cap).float(), dim=-1)[:, cols]  # noqa: E731
        else:
            step = lambda: sa.lm_logprobs(logits, cols, cap)  # noqa: E731
        wall, kern = timed(step, args.steps, args.warmup, torch)
        ms = float(np.mean(kern))
        nbytes = rows * vocab * 4 + rows * 8 * 4
        gbs = nbytes / (ms * 1e-3) / 1e9
        line.update(metric="read rows/s, lm head read-out", value=rows * args.steps / wall, unit="rows/s", ms_per_step=1e3 * wall / args.steps,
                    dtype="f32", config={"workload": WORKLOADS["LM"], "rows": rows, "vocab": vocab, "way": "torch ops" if args.rows == "scatter" else "kernel"},
                    roofline={"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS, "traffic": None,
                              "kernel_ms": ms, "algorithmic_bytes": nbytes})
        print(json.dumps(line))
        return

    if args.workload in ("XDEC", "XDEC_long", "XDEC_512", "XDEC_qwen"):
        from oracle import xdecode as ox

        long = args.workload == "XDEC_long"
        G = args.contents or (64 if long else 24)
        xH, xh, xd = {"XDEC_512": (16, 1, 512), "XDEC_qwen": (24, 4, 256)}.get(args.workload, (16, 8, 256))
        q, c = synth.xdecode_case(G=G, H=xH, h=xh, d=xd, slots=8, beam=6, S=33, prefix=(1024, 4096) if long else (470, 470), template=(8, 16),
                                  step=32, seed=args.seed, device=dev)
        Q, scale = q.shape[2], 1 / 16
        if args.rows == "scatter":   # the reference's own way (decode.py:81-103: three einsums, masks, one softmax, three einsums), for comparison
            kp, vp, kt, vt, gk, gv = (t[0] for t in (c.kp, c.vp, c.kt, c.vt, c.gk, c.gv))
            mp = (c.pos_p[0] >= 0)[:, None, None, None, :]
            mt = (c.own_t[:, None, :] == (torch.arange(Q, device=dev) // c.beam)[None, :, None])[:, None, None]
            mg = (torch.arange(33, device=dev) > c.step_t)
            ninf = torch.finfo(torch.float32).min

            def step():
                qq = q.reshape(G, xh, xH // xh, Q, xd)
                sp = (torch.einsum("ghrqd,ghkd->ghrqk", qq, kp).float() * scale).masked_fill(~mp, ninf)
                st = (torch.einsum("ghrqd,ghkd->ghrqk", qq, kt).float() * scale).masked_fill(~mt, ninf)
                sg = (torch.einsum("ghrqd,ghqsd->ghrqs", qq, gk).float() * scale).masked_fill(mg, ninf)
                a = torch.softmax(torch.cat([sp, st, sg], -1), -1).to(vp.dtype)
                Lp, Lt = sp.shape[-1], st.shape[-1]
                out = torch.einsum("ghrqk,ghkd->ghrqd", a[..., :Lp], vp).float()
                out += torch.einsum("ghrqk,ghkd->ghrqd", a[..., Lp : Lp + Lt], vt).float()
                out += torch.einsum("ghrqs,ghqsd->ghrqd", a[..., Lp + Lt :], gv).float()
                return out.reshape(G, xH, Q, xd).transpose(1, 2).contiguous().to(q.dtype)
        else:
            step = lambda: sa.xdecode_attn(q, c, 0, scale, nsplit=args.nsplit)  # noqa: E731
        wall, kern = timed(step, args.steps, args.warmup, torch)
        ms = float(np.mean(kern))
        nbytes = synth.xdecode_bytes(c, 0, H=xH)
        gbs = nbytes / (ms * 1e-3) / 1e9
        cpu = None
        if not args.no_cpu and args.rows != "scatter":   # the float64 oracle on the first groups, one core
            ng = min(G, 2)
            sub = [t[0][:ng].float().cpu().numpy() for t in (c.kp, c.vp, c.kt, c.vt, c.gk, c.gv)]
            t0 = time.perf_counter()
            ox.x_attention(q[:ng].float().cpu().numpy(), sub[0], sub[1], c.pos_p[0][:ng].cpu().numpy(), sub[2], sub[3], c.pos_t[:ng].cpu().numpy(),
                           c.own_t[:ng].cpu().numpy(), sub[4], sub[5], c.qpos[:ng].cpu().numpy(), 32, c.beam, scale)
            dt = time.perf_counter() - t0
            cpu = {"value": ng * Q / dt, "unit": "queries/s", "cores": 1, "kind": "port", "sample": f"{ng} of {G} groups through the numpy float64 oracle"}
        line.update(metric="decoded queries/s, extraction-decode attention step (one layer)", value=G * Q * args.steps / wall, unit="queries/s",
                    ms_per_step=1e3 * wall / args.steps, dtype="bf16",
                    config={"workload": WORKLOADS[args.workload], "groups": G, "queries": G * Q, "nsplit": args.nsplit or (next(iter(c._plans.values()))[0] if c._plans else None),
                            "way": "torch ops" if args.rows == "scatter" else "kernel"},
                    roofline={"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                              "traffic": TRAFFIC_BYTES.get(args.workload) if args.contents is None and args.rows != "scatter" and not args.nsplit else None,
                              "kernel_ms": ms, "algorithmic_bytes": nbytes},
                    cpu_baseline=cpu)
        print(json.dumps(line))
        return

    if args.workload in ("C5_prologue", "C5_gate"):
        cfg = synth.gdn_config("C5", seed=args.seed, contents=args.contents)
        plan = cfg.plan(dev)
        T, h, hv, dk, dv = cfg.batch.length, 16, 32, 128, 128
        kd, vd = h * dk, hv * dv
        cd = 2 * kd + vd
        gen = torch.Generator(device=dev).manual_seed(args.seed)
        y = torch.randn((T, cd + vd + 2 * hv), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
        if args.workload == "C5_prologue":
            conv_w = torch.randn((cd, 4), generator=gen, device=dev) * 0.5
            a_log = torch.rand(hv, generator=gen, device=dev)
            dt_bias = torch.randn(hv, generator=gen, device=dev)
            step = lambda: sa.gdn_prologue(y, plan.conv, conv_w, a_log, dt_bias, h, hv, dk, dv, True)  # noqa: E731
            nbytes = T * ((cd + 2 * hv) * 2 + 32 + cd * 2 + hv * 6)     # q k v b a columns + taps in; q k v, g, beta out
        else:
            o = torch.randn((T, hv, dv), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
            norm_w = torch.rand(dv, generator=gen, device=dev).to(torch.bfloat16) + 0.5
            z = y[:, cd : cd + vd]
            step = lambda: sa.gdn_gate(o, z, norm_w, 1e-6)  # noqa: E731
            nbytes = T * 3 * vd * 2                                        # o, z in; out
        wall, kern = timed(step, args.steps, args.warmup, torch)
        ms = float(np.mean(kern))
        gbs = nbytes / (ms * 1e-3) / 1e9
        line.update(metric="stream rows/s, Gated DeltaNet layer element-wise kernel", value=T * args.steps / wall, unit="rows/s",
                    ms_per_step=1e3 * wall / args.steps, dtype="bf16 (fp32 arithmetic)",
                    config={"workload": WORKLOADS[args.workload], "contents": len(cfg.trees), "rows": T},
                    roofline={"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS,
                              "traffic": TRAFFIC_BYTES[args.workload] if args.contents is None else None, "kernel_ms": ms,
                              "algorithmic_bytes": nbytes})
        print(json.dumps(line))
        return

    if args.workload == "C5":
        rec, cfg, t = gdn_record(sa, synth, torch, np, args, args.steps, args.warmup)
        line.update({k: rec[k] for k in ("metric", "value", "ms_per_step", "dtype", "config", "roofline")})
        if not args.no_cpu:
            from oracle import cpu_baseline

            tps, n, dt, _ = cpu_baseline.gdn_tokens_per_s(*(t[x].cpu() for x in ("q", "k", "v", "g", "beta")), cfg.batch.prev, cfg.batch.art >= 0)
            line["cpu_baseline"] = {"value": tps, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                    "sample": f"fp32 token-by-token recurrence on the first {n} real tokens of the stream ({dt:.1f} s)"}
        print(json.dumps(line))
        return

    cfg = synth.attention_config(args.workload, seed=args.seed, contents=args.contents)
    layers = [None] if cfg.window is None else [cfg.window, None]   # C3 alternates sliding and global layers
    t0 = time.perf_counter()
    work = []
    for b in cfg.batches:
        masks = sa.block_masks(b, sliding_window=cfg.window, device=dev)
        work.append((synth.qkv(cfg, b, seed=args.seed, device=dev), masks))
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t0
    tp0 = time.perf_counter()
    for b in cfg.batches:
        sa.TilePlan.build(b.art, b.end, b.pos, None)
    plan_ms = 1e3 * (time.perf_counter() - tp0)

    if args.rows != "stream":
        args.no_cpu = True
        # compact rows (the Qwen stack's call, spinf_serve/models/qwen35/qwen.py:613-622): q, k, v hold the real tokens only
        compact = []
        for b, ((q, k, v), masks) in zip(cfg.batches, work):
            sidx = torch.from_numpy(np.flatnonzero(b.art >= 0)).to(dev)
            compact.append((tuple(t[sidx].contiguous() for t in (q, k, v)), masks, sidx, b.length))
        work = None

    def step():
        out = None
        if args.rows == "stream":
            for (q, k, v), masks in work:
                for w in layers:
                    out = sa.tree_attn(q, k, v, masks["sliding_attention" if w else "full_attention"], cfg.scale, variant=args.variant)
        elif args.rows == "compact":   # the kernel goes through the row map
            for (q, k, v), masks, sidx, _ in compact:
                for w in layers:
                    out = sa.tree_attn(q, k, v, masks["sliding_attention" if w else "full_attention"], cfg.scale, variant=args.variant, sidx=sidx)
        else:                          # "scatter": the reference's three zero-filled scatters and the gather around the stream-layout call
            for (q, k, v), masks, sidx, length in compact:
                for w in layers:
                    up = [t.new_zeros(length, t.shape[1], t.shape[2]).index_copy_(0, sidx, t) for t in (q, k, v)]
                    o = sa.tree_attn(*up, masks["sliding_attention" if w else "full_attention"], cfg.scale, variant=args.variant)
                    out = q.new_zeros(q.shape)
                    out[: sidx.shape[0]] = o.index_select(0, sidx)
        return out

    wall, kern = timed(step, args.steps, args.warmup, torch)
    ms = float(np.mean(kern))
    flops = sum(cfg.flops(w) for w in layers)
    tokens = cfg.n_real * len(layers)
    tfl = flops / (ms * 1e-3) / 1e12
    line.update(value=tokens * args.steps / wall, ms_per_step=1e3 * wall / args.steps, dtype="bf16",
                config={"workload": WORKLOADS[args.workload], "contents": len(cfg.trees), "packed_tokens": cfg.n_real,
                        "stream_tokens": sum(b.length for b in cfg.batches), "passes": len(cfg.batches), "layers_per_step": len(layers),
                        "visible_pairs": [cfg.pairs(w) for w in layers], "variant": args.variant, "rows": args.rows},
                roofline={"bound": "mfma", "achieved": tfl, "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": tfl / PEAK_BF16_TFLOPS,
                          "traffic": TRAFFIC_BYTES.get(args.workload) if args.contents is None and args.rows == "stream" else None, "kernel_ms": ms,
                          "kernel_ms_min": float(timed.min_ms), "useful_flops": flops,
                          "algorithmic_bytes": cfg.bytes() * len(layers), "hbm_frac_at_algorithmic_bytes": cfg.bytes() * len(layers) / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                          # the two roofs at the published peaks: whichever floor is higher binds the workload
                          "mfma_floor_ms": flops / (PEAK_BF16_TFLOPS * 1e12) * 1e3, "hbm_floor_ms": cfg.bytes() * len(layers) / (PEAK_HBM_GBS * 1e9) * 1e3},
                plan_build_ms_host=plan_ms, setup_s=setup_s)
    if args.workload == "C2" and args.rows == "stream" and args.variant == 0:
        # the same work items with nothing computed (spinf_diag_attn_stream, --workload C2_stream): what moving this pass's bytes in the
        # kernel's pattern takes on this box right now
        from spinf_serve_amd import attention

        (q, k, v), masks = work[0]
        ybuf, ystat = torch.empty_like(q), torch.zeros(2, dtype=torch.int32, device=dev)
        _, ykern = timed(lambda: attention.tree_attn_byte_pattern(q, k, v, masks["full_attention"], ybuf, ystat), args.steps, args.warmup, torch)
        if int(ystat[0]) == 0 and bool((ybuf == 1).all()):
            line["roofline"]["byte_pattern_ms"] = float(np.mean(ykern))
            line["roofline"]["kernel_ms_over_byte_pattern_ms"] = ms / line["roofline"]["byte_pattern_ms"]
        del ybuf
    # what a pure MFMA loop sustains on this part right now, next to the published constant the fraction is priced against
    line["roofline"]["reachable_peak"] = mfma_rate(torch)[0]
    line["roofline"]["frac_of_reachable_peak"] = tfl / line["roofline"]["reachable_peak"]
    if not args.no_cpu:
        from oracle import cpu_baseline

        (q, k, v), _ = work[0]
        b = cfg.batches[0]
        w = layers[0]
        qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
        tps, done, done_tok, dt, outs = cpu_baseline.attention_tokens_per_s(qc, kc, vc, b.art, b.end, b.pos, cfg.scale, window=w)
        reps = 1
        while dt < 10.0 and reps < 64:   # a sample of about 10 - 30 s of CPU work: repeat the same pass
            t2, d2, k2, s2, _ = cpu_baseline.attention_tokens_per_s(qc, kc, vc, b.art, b.end, b.pos, cfg.scale, window=w, max_seconds=25.0 - dt)
            done_tok, dt, reps = done_tok + k2, dt + s2, reps + 1
            tps = done_tok / dt
        gpu = sa.tree_attn(q, k, v, work[0][1]["sliding_attention" if w else "full_attention"], cfg.scale).float().cpu()
        err = max(float((gpu[a:bb] - o).abs().max()) for (a, bb), o in outs.items())
        line["cpu_baseline"] = {"value": tps, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
                                "sample": f"{done} of {len(cfg.trees) if len(cfg.batches) == 1 else 'the first pass'} contents x {reps} repeats ({done_tok} packed tokens), fp32 torch scaled_dot_product_attention with an explicit dense tree mask per content, {dt:.1f} s; os.cpu_count()={os.cpu_count()}",
                                "max_abs_err_gpu_vs_cpu_fp32": err}
    if args.workload == "C2" and args.contents is None and args.rows == "stream":
        # the other half of the hot path, timed in the same run: C5 through the Gated DeltaNet tree scan
        work = None
        line["gdn"] = gdn_record(sa, synth, torch, np, args, max(10, args.steps // 4), max(5, args.warmup // 4))[0]
        # and the two bigger attention configurations, whole, a few steps each (C3: 13 passes x 2 layers a step; C4: one launch of 659,200 tokens)
        if not args.no_big:
            for name, key in (("C3", "c3"), ("C4", "c4")):
                torch.cuda.empty_cache()
                line[key] = attn_record(sa, synth, torch, np, name, args.seed, 4, 1)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
