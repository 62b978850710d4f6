"""Hardware assumptions that the kernels lean on, checked on the GPU itself (no counterpart in the reference)."""

import ctypes as C

import pytest
import torch

from spinf_serve_amd import _lib

pytestmark = pytest.mark.gpu


def test_lds_reads_of_mixed_kinds_return_in_issue_order(dev, lib):
    """Every s_waitcnt lgkmcnt(n) in the attention and scan kernels assumes that a wave's LDS reads return in the order
    they were issued, also when transposing 8-byte reads and 16-byte reads alternate.  1024 workgroups of four waves
    (four per compute unit, all hammering LDS) run 200 rounds of six interleavings of eight reads with the partial waits
    an in-order LDS allows; each result is compared with the same read done alone behind a full wait."""
    out = torch.zeros(7, dtype=torch.int32, device=dev)
    wgs, iters = 1024, 200
    _lib.check(lib.spinf_diag_lds_order(iters, wgs, out.data_ptr(), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "spinf_diag_lds_order")
    torch.cuda.synchronize()
    got = out.cpu().tolist()
    assert got[6] == wgs, got
    assert got[:6] == [0] * 6, f"LDS reads returned out of order: mismatches per interleaving {got[:6]} of {wgs * 256 * iters * 8} reads each"


def test_an_mfma_needs_one_instruction_after_a_vector_write_of_its_operands(dev, lib):
    """The ring kernel issues its MFMAs from inline assembly, where the compiler's hazard recogniser does not look, so the gap
    the hardware wants between a vector write of an MFMA's A / B registers and the MFMA must come from the source (the build
    scans the generated assembly for it).  Measured here: with the MFMA in the very next issue cycle it multiplies the
    registers' OLD contents (v_mov as well as v_exp -> v_cvt_pk writers); with one instruction or more in between, or with
    the write behind the MFMA, every product is right."""
    out = torch.zeros(21, dtype=torch.int32, device=dev)
    wgs, iters = 1024, 20
    _lib.check(lib.spinf_diag_mfma_hazard(iters, wgs, out.data_ptr(), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "spinf_diag_mfma_hazard")
    torch.cuda.synchronize()
    got = out.cpu().tolist()
    lanes = wgs * 512 * iters
    assert got[20] == wgs, got
    write_then_mfma, mfma_then_write, cvt_then_mfma, other_gaps = got[0:5], got[5:10], got[10:15], got[15:20]
    print(f"lanes with wrong products of {lanes} per case, gaps of 0 1 2 4 8 instructions: v_mov -> MFMA {write_then_mfma}, MFMA -> v_mov "
          f"{mfma_then_write}, v_exp -> v_cvt_pk -> MFMA {cvt_then_mfma}; s_waitcnt x1, x2, vmcnt, v_nop, s_waitcnt + s_nop in the gap {other_gaps}")
    assert write_then_mfma[1:] == [0] * 4 and cvt_then_mfma[1:] == [0] * 4, got
    assert mfma_then_write == [0] * 5, got
    assert other_gaps[3:] == [0] * 2, got
    assert write_then_mfma[0] > 0 and cvt_then_mfma[0] > 0, f"no wrong product without a gap any more: {got} (the assembly scan of the build could go)"


def test_a_waves_vector_instructions_do_not_run_in_the_shadow_of_its_own_mfmas(dev, lib):
    """What bounds the attention kernels at head dim 128 (16 MFMAs and about as many clocks of softmax per 32 x 32 block and wave):
    a wave that issues { MFMA 32x32x16, nv independent v_fma_f32 } per round needs 36 + 4 nv clocks per round, not max(36, 4 nv):
    its vector instructions wait for its MFMA.  Only another wave of the SIMD fills the gap: with two waves per SIMD and 4 vector
    instructions per MFMA the matrix pipe is busy all the time (32 clocks per MFMA of the SIMD)."""
    iters = 20000

    def run(nv, wps):
        out = torch.zeros(2 * 4 * wps, dtype=torch.int64, device=dev)
        _lib.check(lib.spinf_diag_mfma_valu(nv, 0, wps, iters, out.data_ptr(), C.c_void_p(torch.cuda.current_stream().cuda_stream)), "spinf_diag_mfma_valu")
        torch.cuda.synchronize()
        t = out.cpu().view(-1, 2)[0::4]   # the waves of SIMD 0
        return float(t[0, 1] - t[0, 0]) / iters, float(t[:, 1].max() - t[:, 0].min()) / (iters * wps)

    alone = {nv: run(nv, 1)[0] for nv in (0, 8, 16)}
    pair = run(4, 2)[1]
    print(f"clocks per round of a wave alone on its SIMD: {alone}; clocks per MFMA of a SIMD with two waves, 4 vector instructions per MFMA: {pair:.1f}")
    assert 30 <= alone[0] <= 36, alone            # the counter counts core clocks: a 32x32x16 MFMA chain is 32 per link
    assert alone[8] >= alone[0] + 0.8 * 32, f"vector instructions now run under a wave's own MFMA: {alone} (the two-block pipeline of the lockstep kernel would pay)"
    assert alone[16] >= alone[0] + 0.8 * 64, alone
    assert pair <= 36, f"a second wave no longer fills the matrix pipe: {pair}"


def test_byte_pattern_yardstick_moves_every_tile_and_writes_every_row(dev, lib):
    """spinf_diag_attn_stream on a scaled-down C2: every tile of every work item is seen landed (the count equals the plan
    entries of the 32-key plan x head groups), no wait is given up, and every row of the stream is written"""
    import spinf_serve_amd as sa
    from spinf_serve_amd import attention, synth

    cfg = synth.attention_config("C2", contents=3)
    b = cfg.batches[0]
    q, k, v = synth.qkv(cfg, b, seed=1, device=dev)
    mask = sa.TreeMask.build(b.art, b.end, b.pos, device=dev)
    plan = mask.for_head_dim(cfg.d, ring=True).plan
    for parts in (3, 7):   # a tile's requests made by one wave, as in the kernel; dealt out over the eight waves
        out = torch.zeros_like(q)
        status = torch.zeros(2, dtype=torch.int32, device=dev)
        attention.tree_attn_byte_pattern(q, k, v, mask, out, status, parts=parts)
        torch.cuda.synchronize()
        gave_up, tiles = status.cpu().tolist()
        assert gave_up == 0, parts
        assert tiles == len(plan.kv_idx) * (cfg.hq // 2), parts
        assert (out == 1).all(), parts
