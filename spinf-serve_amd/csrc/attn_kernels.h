// Pieces shared by the attention kernels of tree_attn.hip and tree_attn_ring.hip: the kernel argument block, the LDS tile buffer,
// the tile DMA, a wave's fragment addresses, the per-element mask (spinf_serve/scorer.py:173-177).
#pragma once
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"
#include "attn_tiles.h"

constexpr int NLIST = 8;       // work lists (XCDs of an MI355X)
constexpr int LAND_CAP = 4096;  // most item lists of a static schedule (a schedule has one list per compute unit)
constexpr int ENT_CAP = 256;   // plan entries of a query tile kept in LDS at a time

struct AttnParams {
    const __bf16* q; const __bf16* k; const __bf16* v; __bf16* o;
    long q_tok, q_head, k_tok, k_head, v_tok, v_head, o_tok, o_head;
    int n, group;
    float c;              // scale * log2(e)
    int window;
    const int* art; const int* end; const int* pos;
    const int* kv_idx; const unsigned* kv_bits;
    const int4* items;    // work items {query tile, first entry, entries | head group << 20, first key tile}, list by list
    const int* list_ptr;  // [NLIST + 1] offsets of the lists in items
    int* counters;        // [0..NLIST) next item of each list, [NLIST] workgroups done, [NLIST+1] items awaiting the exact pass,
                          // [NLIST+2] exact-pass workgroups done; each kernel's last workgroup resets what it used; running totals:
                          // [NLIST+3] items recomputed exactly, [NLIST+4] waves of the ring kernel that gave up a wait
    int* redo;            // indices (into items) of the work items the fast pass handed to the exact pass (the ring kernel: entries
                          // list_ptr[b] .. of workgroup b's own hand-overs, which it recomputes itself)
    // compact rows (ROWS kernels): q, k, v, o hold the real tokens only; row_of[stream position] = row, -1 for a pad position;
    // kv_row0[entry] = row of the entry's first key if its 64 keys are 64 consecutive rows, else -1
    const int* row_of; const int* kv_row0;
    const int* grp;       // image groups (GRP kernels): -1 none; the tokens of a group see each other both ways
    bool static_lists;    // list_ptr delimits one item list per workgroup (a static schedule) instead of the eight shared lists
    bool clear_first;     // host side only: zero the cursors and counts in front of the pass (the entry point that allocates nothing)
    int spin_limit;       // ring kernel: polls of one wait before the wave gives up and its workgroup lands in the barrier-paced pass (a healthy
                          // wait takes a handful; tests set it to 1 to force the landing)
};

// Softmax reference point.  The fast pass fixes each row's reference at the maximum of the first 32-key block in which
// the row sees a key and never rescales the accumulators: probabilities are exp2(t - ref) and stay below 2^TAU_FAST, well
// inside fp32 / bf16 range.  If any row of a tile meets scores so far above its reference that a lane's 16 probabilities of a
// block sum to more than 2^TAU_FAST (at the latest when one score lies TAU_FAST above the reference), the whole tile is
// recomputed by the exact pass: classic online softmax, reference raised and accumulators rescaled whenever a block
// maximum exceeds the reference by more than TAU_LAZY.  Which pass produced a row depends on the rows of its own
// 128-token tile only, so it does not depend on what the job is packed with.
constexpr float TAU_FAST = 60.f;
constexpr float VIOL_SUM = 1152921504606846976.f;   // 2^TAU_FAST: a lane's 16 probabilities of a block summing above it send the tile to the exact pass
constexpr float TAU_LAZY = 8.f;


// A tile buffer: the K tile at the key head dim D, the V tile at DV head dims (DV = D, except at head dim 512, where O^T is
// computed 256 dims at a time: see launch_d512), then art, end, pos, grp of the keys.
template <int D, int TK, int DV>
struct TileGeo {
    using K = Geo<D, TK>;
    using V = Geo<DV, TK>;
    static constexpr int KTILEB = K::KTILEB, VTILEB = V::VTILEB;
    static constexpr int BUFB = KTILEB + VTILEB + K::METAB;
    static constexpr int KSUB = K::KSUB, VSUB = V::VSUB;
};


// Starts the DMA of key tile kt (64 keys of kv head kvh) into the LDS buffer at byte address `buf`.  Wave w of NW copies regions
// w*IPW .. w*IPW+IPW-1; lane -> (slot = which row of the region, 16-byte chunk of the row).  For a tile that lies fully inside
// the stream every address is a wave-uniform base plus a per-lane constant (lane_k / lane_v, bytes), so the loop spends no
// vector ALU on addressing; the last, partial tile clamps its rows per lane.
// ROWS (compact rows): row0 >= 0 says that the tile's keys are rows row0 .. row0 + 63; otherwise every lane looks its row up.
template <int D, int NW = 4, bool ROWS = false, int GRP = 0, int TK = 64, int DV = D>
__device__ __forceinline__ void issue_tile(const AttnParams& p, unsigned buf, int kt, int row0, int kvh, int w, int lane, unsigned lane_k, unsigned lane_v) {
    using G = TileGeo<D, TK, DV>;
    using GK = typename G::K;
    using GV = typename G::V;
    constexpr int IPWK = GK::NREG / NW, IPWV = GV::NREG / NW;   // DMA instructions per wave and tile
    static_assert(IPWK >= 1 && IPWK * NW == GK::NREG && IPWV >= 1 && IPWV * NW == GV::NREG, "the tile's regions must divide among the waves");
    const char* kbase = (const char*)(p.k + (long)kvh * p.k_head);
    const char* vbase = (const char*)(p.v + (long)kvh * p.v_head);
    if (ROWS ? row0 >= 0 : kt * TK + TK <= p.n) {
        const long first = ROWS ? (long)row0 : (long)kt * TK;
#pragma unroll
        for (int i = 0; i < IPWK; i++) {
            const int reg = w * IPWK + i;
            dma16_uniform(kbase + (first + reg) * p.k_tok * 2, lane_k, buf + reg * GK::KRS);
        }
#pragma unroll
        for (int i = 0; i < IPWV; i++) {
            const int reg = w * IPWV + i;
            dma16_uniform(vbase + (first + reg) * p.v_tok * 2, lane_v, buf + G::KTILEB + reg * GV::VRS);
        }
        if (w < (GRP ? 4 : 3)) {   // wave 0: art, wave 1: end, wave 2: pos, wave 3: grp of the 64 keys
            const int* src = (w == 0 ? p.art : w == 1 ? p.end : w == 2 ? p.pos : p.grp) + (long)kt * TK;
            dma4_lane(src + (TK < 64 ? lane % TK : lane), buf + G::KTILEB + G::VTILEB + w * 256);   // (64 lanes: a 32-key tile's twice)
        }
    } else {
        auto row_at = [&](const int reg, const int nreg, const int slot) {
            long grow = (long)kt * TK + reg + nreg * slot;
            grow = grow < p.n ? grow : p.n - 1;
            if (ROWS) {   // a pad position has no row: any row will do, its keys are visible to nobody but pad rows
                const int r = p.row_of[grow];
                grow = r < 0 ? 0 : r;
            }
            return grow;
        };
#pragma unroll
        for (int i = 0; i < IPWK; i++) {
            const int reg = w * IPWK + i;
            dma16_lane(kbase + row_at(reg, GK::NREG, lane / GK::CPR) * p.k_tok * 2 + (lane % GK::CPR) * 16, buf + reg * GK::KRS);
        }
#pragma unroll
        for (int i = 0; i < IPWV; i++) {
            const int reg = w * IPWV + i;
            dma16_lane(vbase + row_at(reg, GV::NREG, lane / GV::CPR) * p.v_tok * 2 + (lane % GV::CPR) * 16, buf + G::KTILEB + reg * GV::VRS);
        }
        if (w < (GRP ? 4 : 3)) {
            long gk = (long)kt * TK + (TK < 64 ? lane % TK : lane);
            gk = gk < p.n ? gk : p.n - 1;
            dma4_lane((w == 0 ? p.art : w == 1 ? p.end : w == 2 ? p.pos : p.grp) + gk, buf + G::KTILEB + G::VTILEB + w * 256);
        }
    }
}

// Everything a wave needs to know about its place in the workgroup and its LDS fragment addresses.
template <int D, int TK = 64, int DV = D>
struct Lane {
    using GK = Geo<D, TK>;
    using GV = Geo<DV, TK>;
    int lane, m, g, w;
    int wr, wh;                  // row group (tokens 32 wr ..) and head set of this wave
    int k_lane, v_lane;          // byte offsets of this lane's K fragment row / V^T fragment address inside a tile
    unsigned lane_k, lane_v;     // per-lane part of the DMA source addresses
    __device__ __forceinline__ Lane(const AttnParams& p) {
        lane = threadIdx.x & 63;
        m = lane & 31;
        g = lane >> 5;
        w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
        wh = w >> 2;
        // waves w and w + 4 share a SIMD: the second head set takes the row groups in reverse order, so that a SIMD's two waves
        // together see about the same number of key blocks near the diagonal (row group k sees k + 1 of 4, or only its own branch)
        wr = wh ? 3 - (w & 3) : (w & 3);
        // K fragment: row m of the 32-key block, 16-byte chunk g of each 32-byte step.  V^T fragment
        // (ds_read_b64_tr_b16): inside its 16-lane group a lane supplies the address of key row 4g + tr_j, head dims
        // 16 tr_mb + 4 tr_a .. +3 of the 32-wide slice, and receives head dim lane%32 of 4 consecutive keys.
        const int tr_a = lane & 3, tr_j = (lane >> 2) & 3, tr_mb = (lane >> 4) & 1;
        k_lane = GK::k_off(m) + 16 * g;
        v_lane = GV::v_off(4 * g + tr_j) + 32 * tr_mb + 8 * tr_a;
        lane_k = (unsigned)((lane / GK::CPR) * GK::NREG * p.k_tok * 2 + (lane % GK::CPR) * 16);
        lane_v = (unsigned)((lane / GV::CPR) * GV::NREG * p.v_tok * 2 + (lane % GV::CPR) * 16);
    }
};

// mask of one 32-key block: register i of the S^T tile holds key 8*(i/4) + 4g + i%4 of the block
// GRP 1: a key of the row's image group is visible whatever the rest says; GRP 2: if it also lies within the window
// STEPWISE: the four groups of four keys one after the other (a scheduling barrier between them), so that only one group's
// metadata is in registers at a time; otherwise the compiler requests all of it up front (up to 64 registers)
template <int RT, bool WIN, int GRP = 0, int TK = 64, bool STEPWISE = false>
__device__ __forceinline__ void apply_mask(f32x16 (&s_acc)[RT], const int* meta, int kt, int sub, int g, int tok, int art_q, int pos_q, int window,
                                           int grp_q = -1) {
#pragma unroll
    for (int i4 = 0; i4 < 4; i4++) {
        if (STEPWISE && i4 > 0) __builtin_amdgcn_sched_barrier(0);
        const int ko = 32 * sub + 8 * i4 + 4 * g;
        const int4 ka = *(const int4*)(meta + ko);
        const int4 ke = *(const int4*)(meta + 64 + ko);
        int4 kp = make_int4(0, 0, 0, 0), kgr = make_int4(-1, -1, -1, -1);
        if (WIN) kp = *(const int4*)(meta + 128 + ko);
        if (GRP) kgr = *(const int4*)(meta + 192 + ko);
        const int kg = kt * TK + ko;
        const int kav[4] = {ka.x, ka.y, ka.z, ka.w};
        const int kev[4] = {ke.x, ke.y, ke.z, ke.w};
        const int kpv[4] = {kp.x, kp.y, kp.z, kp.w};
        const int kgv[4] = {kgr.x, kgr.y, kgr.z, kgr.w};
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            const int kk = kg + jj;
            bool vis = (kk <= tok) & (art_q >= 0) & (kav[jj] == art_q) & (tok < kev[jj]);
            if (GRP == 1 && WIN) vis = vis & ((pos_q - kpv[jj]) < window);   // the group term below is not windowed
            if (GRP) vis = vis | ((grp_q >= 0) & (kgv[jj] == grp_q));
            vis = vis | (kk == tok);
            if (WIN && GRP != 1) vis = vis & ((pos_q - kpv[jj]) < window);
#pragma unroll
            for (int rt = 0; rt < RT; rt++) s_acc[rt][4 * i4 + jj] = vis ? s_acc[rt][4 * i4 + jj] : -INFINITY;
        }
    }
}

// The lane index, recomputed on the spot (two instructions).  For the code between two items (output rows, the next item's
// queries): a lane-dependent value kept in a register across the tile loop is spilled at head dim 256, and its reload is a
// memory operation whose wait also waits for every output store issued before it, one store at a time.
__device__ __forceinline__ int fresh_lane_id() {
    int lane;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane));
    return lane;
}

// tree_attn_ring.hip: the pass with decoupled waves over a static schedule (p.list_ptr delimits n_wg item lists, one per
// workgroup; plan entries of 32 keys), the exact recomputation of the items that need it included.  Stream-ordered launch on `stream`.
int spinf_launch_ring(const AttnParams& p, int d, bool win, int n_wg, hipStream_t stream);
