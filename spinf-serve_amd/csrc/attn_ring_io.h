// How a 32-key K / V tile gets into a slot of the ring kernel's LDS ring (tree_attn_ring.hip): whole-wave DMA requests
// (global_load_lds_dwordx4), the last of which writes the slot's "landed" flag.  Shared with the byte-pattern yardstick in
// diag.hip, which moves the same tiles the same way and computes nothing.
#pragma once
#include <hip/hip_runtime.h>

#include "attn_kernels.h"

// A tile's "landed" flag is written by the DMA engine itself: the last request of a tile copies ring_seq[generation % 64] from
// global memory into the flag words of the slot (the fourth 256 bytes of its key metadata).  The loads of a wave return in
// order, so when the flag shows the tile's generation the tile's data is there; the wave that made the requests never waits.
static __device__ const int ring_seq[64] = {0,  1,  2,  3,  4,  5,  6,  7,  8,  9,  10, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20, 21,
                                     22, 23, 24, 25, 26, 27, 28, 29, 30, 31, 32, 33, 34, 35, 36, 37, 38, 39, 40, 41, 42, 43,
                                     44, 45, 46, 47, 48, 49, 50, 51, 52, 53, 54, 55, 56, 57, 58, 59, 60, 61, 62, 63};

// NREG requests of 1 KiB each in a row: region r comes from base + r * stride + lane_off (bytes; base and stride wave-uniform)
// and goes to LDS bytes lds + r * PITCH.  Three instructions per request (the request, the LDS address in m0, the lane offset):
// the wave that recycles a slot is the one the others are waiting for, and address arithmetic left to the compiler took a dozen.
template <int NREG, int PITCH>
__device__ __forceinline__ void dma_regions(const char* base, unsigned stride, unsigned lane_off, unsigned lds) {
    base = uniform_ptr(base);
    stride = __builtin_amdgcn_readfirstlane(stride);
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\t"
                 ".rept %c4\n\t"
                 "global_load_lds_dwordx4 %0, %1\n\t"
                 "s_add_u32 m0, m0, %c5\n\t"
                 "v_add_u32_e32 %0, %3, %0\n\t"
                 ".endr"
                 : "+v"(lane_off)
                 : "s"(base), "s"(lds), "s"(stride), "n"(NREG), "n"(PITCH)
                 : "memory", "m0", "scc");
}

// One wave requests a whole tile of TK keys (32; 64 at head dim 128): K and V regions, art / end / pos of the keys, then the flag
// (generation gen).
template <int D, bool WIN, int TK = 32>
__device__ __forceinline__ void issue_tile_wave(const AttnParams& p, unsigned buf, int kt, int kvh, int gen, int lane, unsigned lane_k, unsigned lane_v) {
    using GK = Geo<D, TK>;
    constexpr int KTILEB = GK::KTILEB, VTILEB = GK::VTILEB;
    const char* kbase = (const char*)(p.k + (long)kvh * p.k_head);
    const char* vbase = (const char*)(p.v + (long)kvh * p.v_head);
    if (kt * TK + TK <= p.n) {
        const long first = (long)kt * TK;
        dma_regions<GK::NREG, GK::KRS>(kbase + first * p.k_tok * 2, (unsigned)(p.k_tok * 2), lane_k, buf);
        dma_regions<GK::NREG, GK::VRS>(vbase + first * p.v_tok * 2, (unsigned)(p.v_tok * 2), lane_v, buf + KTILEB);
        const int key = kt * TK + (lane & (TK - 1));
        dma4_lane(p.art + key, buf + KTILEB + VTILEB);
        dma4_lane(p.end + key, buf + KTILEB + VTILEB + 256);
        if (WIN) dma4_lane(p.pos + key, buf + KTILEB + VTILEB + 512);
    } else {   // the stream's last, partial tile: rows clamped per lane
        auto row_at = [&](const int reg, const int slot) {
            const long grow = (long)kt * TK + reg + GK::NREG * slot;
            return grow < p.n ? grow : (long)p.n - 1;
        };
#pragma unroll 1   // (rolled: unrolled, the 32 per-lane addresses are all computed up front and take 64 registers)
        for (int reg = 0; reg < GK::NREG; reg++)
            dma16_lane(kbase + row_at(reg, lane / GK::CPR) * p.k_tok * 2 + (lane % GK::CPR) * 16, buf + reg * GK::KRS);
#pragma unroll 1
        for (int reg = 0; reg < GK::NREG; reg++)
            dma16_lane(vbase + row_at(reg, lane / GK::CPR) * p.v_tok * 2 + (lane % GK::CPR) * 16, buf + KTILEB + reg * GK::VRS);
        int key = kt * TK + (lane & (TK - 1));
        key = key < p.n ? key : p.n - 1;
        dma4_lane(p.art + key, buf + KTILEB + VTILEB);
        dma4_lane(p.end + key, buf + KTILEB + VTILEB + 256);
        if (WIN) dma4_lane(p.pos + key, buf + KTILEB + VTILEB + 512);
    }
    dma4_lane(ring_seq + (gen & 63), buf + KTILEB + VTILEB + 768);   // every lane the same word: 64 copies of the flag
}
