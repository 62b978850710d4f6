// Gated DeltaNet, chunked WY form, one fused kernel: stands in for gdn.chunked (spinf_serve/models/qwen35/gdn.py:109-133),
// i.e. for fla's cumsum -> intra-chunk WY solve -> state recurrence (gdn.py:21-106) -> output pipeline, without writing
// the per-chunk state snapshots or the w / u / v_new intermediates to memory; it also serves the recurrent entry point
// (gdn.py:197-235) for value head dim 128, where the leaves that fork from one state are taken two to a chunk.
//
// One workgroup (4 waves) owns one (segment, value head) and walks its 32-token chunks (two 16-token tiles) in order;
// wave w owns value columns 32w .. 32w+31 of the state S [K=128, V=128], which never leaves its
// fp32 accumulator registers.  Per chunk, with G = cumsum(g), D_ij = e^{G_i - G_j}:
//     A   = -strict_tril(beta_i (K K^T)_ij D_ij)         T = (I - A)^-1      (fp32: 16 x 16 blocks solved by substitution in
//                                                                             registers, merged with fp32 MFMAs)
//     U   = T diag(beta) V          -W = -T diag(beta e^G) K                 (bf16 MFMA, fp32 accumulate)
//     V'  = U - W S                 O = s e^{G_i} (Q S)_i + tril(s (Q K^T) D) V'
//     S  <- e^{G_L} S + (K e^{G_L - G})^T V'
// The token x token and token x key quantities (A, P, T, W) are the same for all value columns: the waves split them (one
// 16 x 16 tile of A and P per wave, the triangular solve on wave 0, two key tiles of W per wave) and exchange them through
// LDS; everything that touches value columns is private to a wave, and every product leaves its result in the register
// layout the next product takes as an operand (see gdn_tiles.h), so of those only the output rows pass through LDS (for
// 16-byte stores).  The kernels are bound by instruction issue, not by the matrix cores: what is shared is not recomputed.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"
#include "gdn_tiles.h"

using namespace gdn_tiles;

namespace {

constexpr int KD = 128;        // key head dim
constexpr int VD = 128;        // value head dim
// Row strides of the LDS tiles, chosen by how a tile is read most.  A tile read row-wise in 8- or 16-byte pieces (Q, -W: lane c
// takes row c) wants a stride of 4 banks (mod 64): 16 rows then start in 16 different groups of four banks.  A tile read through
// ds_read_b64_tr_b16 (K, V: 16 lanes take a 4 rows x 32 bytes block, the next 16 lanes the four rows below) wants 8 banks
// (mod 64): eight rows x 32 bytes then cover the 64 banks once.  Measured LDS clocks per instruction of a workgroup (stride in
// banks mod 64): 8-byte row reads 2.8 at 4 or 20, 4.0 at 2, 8, 18; transposing reads 2.9 at 8 or 24, 4.0 at 4, 12, 16, 20;
// 16-byte row reads 4.0 at 8, 8.0 at 4, 20, 36.
constexpr int LD = 136;        // row stride (elements) of the Q tile: 68 banks
constexpr int LDT = 144;       // row stride of the K and V tiles: 72 banks
constexpr int LW = 136;        // row stride of the -W tile
constexpr int LP = 40;         // row stride of the token x token bf16 tiles (P, T diag(beta), -T diag(beta e^G))
constexpr int LA = 36;         // row stride (floats) of A
constexpr int LX = 20;         // row stride (floats) of the 16 x 16 blocks of T and of the merge scratch

// element offset of a row: one 32 x 32 -> 64 bit multiply (rows and strides are below 2^31; the launch checks the strides)
__device__ __forceinline__ long row_offset(int row, long stride) { return (long)((unsigned long)(unsigned)row * (unsigned)stride); }
__device__ __forceinline__ bf16x4 zero_bf4() {
    bf16x4 z;
#pragma unroll
    for (int r = 0; r < 4; r++) z[r] = (__bf16)0.f;
    return z;
}
}  // namespace

template <bool PAIRS>
__device__ __forceinline__ void gdn_wy_body(const GdnParams& p) {
    constexpr int NT = 2;                           // 16-token tiles per chunk
    constexpr int CH = 16 * NT;
    constexpr int LO = CH + 4;                      // row stride (elements) of a wave's transposed output tile [32 values][CH tokens]; 64-byte rows
                                                    // put the 8-byte stores of 16 lanes into four banks (32 clocks per store instead of 7)
    constexpr int NTILES = NT * (NT + 1) / 2;       // 16 x 16 tiles of A / P on or below the diagonal
    typedef bf16x8 tok_op;                          // operand of a product that contracts over the chunk's 32 tokens
    __shared__ __attribute__((aligned(16))) __bf16 Ks[CH * LDT];
    __shared__ __attribute__((aligned(16))) __bf16 Qs[CH * LD];
    __shared__ __attribute__((aligned(16))) __bf16 Vs[CH * LDT];     // V; later the waves' output tiles
    __shared__ __attribute__((aligned(16))) char solve[32 * LA * 4 + 32 * LX * 4 + 16 * LX * 4 + 256];   // A, T blocks, merge scratch; later -W
    __shared__ __attribute__((aligned(16))) __bf16 Ps[CH * LP];
    __shared__ __attribute__((aligned(16))) __bf16 Tus[CH * LP];
    __shared__ __attribute__((aligned(16))) __bf16 Tws[CH * LP];
    __shared__ __attribute__((aligned(16))) float Gs[CH];
    __shared__ __attribute__((aligned(16))) float Bs[CH];
    __shared__ int Rs[CH];
    float* As = (float*)solve;
    float* Ts = As + 32 * LA;          // T_00 in rows 0..15, T_11 in rows 16..31
    float* Xs = Ts + 32 * LX;
    __bf16* Wn = (__bf16*)solve;       // -W [CH][LW], written when A and T are dead
    static_assert(32 * LW * 2 <= (int)sizeof(solve), "-W must fit the region it shares");
    static_assert(4 * 32 * LO <= CH * LDT, "the output tiles must fit the V tile");

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c = lane & 15, q4 = lane >> 4;
    // Workgroups go round the 8 XCDs (each with its own L2) in launch order.  Two value heads that share a key head read the
    // same q and k rows: they get launch slots 8 apart, i.e. the same XCD at about the same time, so the second read hits L2.
    long slot = blockIdx.x;
    if (p.hv == 2 * p.h && gridDim.x % 16 == 0) slot = (slot / 16) * 16 + (slot % 8) * 2 + (slot % 16) / 8;
    const int hv = (int)(slot % p.hv);
    const int hk = hv / (p.hv / p.h);
    // Pairs (the recurrent entry point).  Consecutive segments that start from the same stored state, have at most 16 tokens
    // and leave no state behind (the leaves that fork from one trunk) never change the state registers: they form a run that
    // is taken TWO segments per chunk (one per 16-token tile: A, P and T are then block diagonal, the tiles do not see each
    // other), with the state loaded once and the row prefetch running from one pair into the next.  The instructions of a
    // chunk hardly depend on how many of its rows are in use, so this halves the work per leaf.  A workgroup owns a group of
    // p.run consecutive segments (launching one workgroup per leaf would cost more in dispatch than the leaves in compute)
    // and walks it run by run; any segment that is not such a leaf is a run of its own, walked chunk by chunk.
    const long group = PAIRS ? p.run : 1;
    const long s_begin = (slot / p.hv) * group, s_end = PAIRS ? min(p.n_seg, s_begin + group) : s_begin + 1;
    // The group's segments are described once, by one thread each: first call row, length, and whether the segment continues
    // the run of the one before it (both leaves of the same state); the bit mask of the latter gives the run lengths.
    __shared__ long g_base[16];
    __shared__ int g_len[16];
    __shared__ unsigned g_follows;
    if (PAIRS) {
        if (tid < 16) {
            const long s_ = s_begin + tid;
            bool fol = false;
            if (s_ < s_end) {
                const long b0 = p.cu[s_], b1 = p.cu[s_ + 1];
                g_base[tid] = b0;
                g_len[tid] = (int)(b1 - b0);
                if (tid > 0) {
                    const bool keeps = p.ht != nullptr && p.ht_idx != nullptr && (p.ht_idx[s_] >= 0 || p.ht_idx[s_ - 1] >= 0);
                    const bool same = (p.h0 != nullptr && p.h0_idx != nullptr) ? p.h0_idx[s_] == p.h0_idx[s_ - 1] : true;
                    fol = b1 - b0 <= 16 && b0 - p.cu[s_ - 1] <= 16 && !keeps && same;
                }
            }
            const unsigned long m = __builtin_amdgcn_ballot_w64(fol);     // lanes 0..15 of wave 0
            if (tid == 0) g_follows = (unsigned)m;
        }
        lds_barrier();
    }
    const unsigned fol_mask = PAIRS ? (unsigned)__builtin_amdgcn_readfirstlane((int)g_follows) : 0u;
  for (long seg = s_begin; seg < s_end; seg++) {
    const int sl = (int)(seg - s_begin);
    if (PAIRS && ((fol_mask >> sl) & 1u)) continue;     // taken by the run it belongs to
    // the run: this segment and the followers right after it
    const int run_len = PAIRS ? 1 + __builtin_ctz(~(fol_mask >> (sl + 1)) | (1u << 16)) : 1;
    const bool run_mode = PAIRS && run_len > 1;
    const long bos = PAIRS ? g_base[sl] : p.cu[seg];
    const int T = PAIRS ? g_len[sl] : (int)(p.cu[seg + 1] - bos);
    const int n_chunks = run_mode ? (run_len + 1) / 2 : (T + CH - 1) / CH;
    // token tile cc of chunk j: its first call row and its number of rows (0: there is no such tile)
    auto tile_of = [&](int j, int cc, long& base, int& len) __attribute__((always_inline)) {
        if (run_mode) {
            const bool there = 2 * j + cc < run_len;
            base = there ? g_base[sl + 2 * j + cc] : 0;
            len = there ? g_len[sl + 2 * j + cc] : 0;
        } else {
            base = bos + (long)j * CH + 16 * cc;
            len = max(0, min(16, T - j * CH - 16 * cc));
        }
    };
    __bf16* Ow = Vs + w * 32 * LO;

    // ---- state: S[kt][vt][r] = S[16 kt + 4 q4 + r][32 w + 16 vt + c]
    f32x4 S[8][2];
#pragma unroll
    for (int kt = 0; kt < 8; kt++)
#pragma unroll
        for (int vt = 0; vt < 2; vt++) S[kt][vt] = zero4();
    if (p.h0 != nullptr && p.h0_idx != nullptr) {
        const long src = p.h0_idx[seg];
        if (src >= 0) {
            const float* hp = p.h0 + ((src * p.hv + hv) * KD + 4 * q4) * VD + 32 * w + c;
#pragma unroll
            for (int kt = 0; kt < 8; kt++)
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int vt = 0; vt < 2; vt++) S[kt][vt][r] = hp[(16 * kt + r) * VD + 16 * vt];
        }
    }
    const bool keep = p.ht != nullptr && p.ht_idx != nullptr && p.ht_idx[seg] >= 0;

    // The next chunk's rows are fetched into registers while the current chunk is computed, and the stream rows (idx) of
    // the chunk after that one chunk earlier still, so that no load ever waits for the load of its own address.
    // Thread -> 16-byte piece tid%16 of chunk rows tid/16 (+ 16); threads 0..CH-1 also -> g, beta and the stream row of chunk
    // row tid.
    bf16x8 pk[NT], pq[NT], pv[NT];
    int pr32 = -1;
    float pg = 0.f;
    __bf16 pbeta = (__bf16)0.f;   // (kept as loaded: converting here would make the wave wait for the load at once)
    int ra[NT], rb = -1;          // stream rows (< 2^31) of the chunk fetched next: this thread's K / Q / V rows; chunk row tid
    // Only the low half of an index is loaded: the register of an unused high half would be handed out again at once, and
    // whoever writes it first has to wait for the load (and with it for every load in flight).
    const int* idx_lo = (const int*)p.idx;
    auto fetch_rows = [&](const int j) __attribute__((always_inline)) {
        long base[NT];
        int len[NT];
#pragma unroll
        for (int cc = 0; cc < NT; cc++) {
            tile_of(j, cc, base[cc], len[cc]);
            ra[cc] = -1;
            if ((tid >> 4) < len[cc]) {       // this thread's row of tile cc
                const long t = base[cc] + (tid >> 4);
                ra[cc] = p.idx ? idx_lo[2 * t] : (int)t;
            }
        }
        rb = -1;
        if (tid < CH) {                       // chunk row tid = row tid % 16 of tile tid / 16
            const bool hi = tid >= 16;
            const int r = tid & 15;
            if (r < (hi ? len[NT - 1] : len[0])) {
                const long t = (hi ? base[NT - 1] : base[0]) + r;
                rb = p.idx ? idx_lo[2 * t] : (int)t;
            }
        }
    };
    auto fetch_data = [&]() __attribute__((always_inline)) {
        const int col = (tid & 15) * 8;
#pragma unroll
        for (int cc = 0; cc < NT; cc++) {
#pragma unroll
            for (int j = 0; j < 8; j++) { pk[cc][j] = (__bf16)0.f; pq[cc][j] = (__bf16)0.f; pv[cc][j] = (__bf16)0.f; }
            if (ra[cc] >= 0) {
                pk[cc] = *(const bf16x8*)(p.k + row_offset(ra[cc], p.q_tok) + hk * KD + col);
                pq[cc] = *(const bf16x8*)(p.q + row_offset(ra[cc], p.q_tok) + hk * KD + col);
                pv[cc] = *(const bf16x8*)(p.v + row_offset(ra[cc], p.v_tok) + hv * VD + col);
            }
        }
        pr32 = rb;
        pg = 0.f;
        pbeta = (__bf16)0.f;
        if (rb >= 0) {
            pg = p.g[row_offset(rb, p.g_tok) + hv];
            pbeta = p.beta[row_offset(rb, p.g_tok) + hv];
        }
    };
    fetch_rows(0);
    fetch_data();
    fetch_rows(1);

    for (int j = 0; j < n_chunks; j++) {
        lds_barrier();   // every wave is done with the previous chunk's tiles
        // ---- stage the chunk from the prefetch registers (rows >= L are zero): cumulative g, beta, stream rows, K / Q / V
        if (tid < CH) {
            float x = row_prefix_sum(pg);
            // row_bcast:15 -> lanes 16..31 (not for a pair: the second tile is another segment)
            if (!run_mode) x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, false));
            Gs[tid] = x;
            Bs[tid] = (float)pbeta;
            Rs[tid] = pr32;
        }
        {
            const int col = (tid & 15) * 8;
#pragma unroll
            for (int cc = 0; cc < NT; cc++) {
                const int row = (tid >> 4) + 16 * cc;
                *(bf16x8*)(Ks + row * LDT + col) = pk[cc];
                *(bf16x8*)(Qs + row * LD + col) = pq[cc];
                *(bf16x8*)(Vs + row * LDT + col) = pv[cc];
            }
        }
        lds_barrier();

        // Token tiles: tile t = chunk rows 16 t .. 16 t + 15.  In a transposed token x token result the lane owns row
        // i = 16 it + c and its registers hold columns j = 16 jt + 4 q4 + r.
        // ---- (K K^T)^T and (Q K^T)^T: wave x < NTILES takes tile (jt, it) = (0,0), (0,1), (1,1); (1,0) lies above the diagonal.
        // A[i][j] goes to LDS in fp32, P[i][j] = s Q_i.K_j e^{G_i - G_j} (j <= i) in bf16.
        if (w < NTILES) {
            const int jt = w >> 1, it = (w + 1) >> 1;
            f32x4 kk = zero4(), qk = zero4();
#pragma unroll
            for (int s = 0; s < KD / 32; s++) {
                const bf16x8 kj = *(const bf16x8*)(Ks + (16 * jt + c) * LDT + 32 * s + 8 * q4);
                const bf16x8 ki = *(const bf16x8*)(Ks + (16 * it + c) * LDT + 32 * s + 8 * q4);
                const bf16x8 qi = *(const bf16x8*)(Qs + (16 * it + c) * LD + 32 * s + 8 * q4);
                kk = mfma32(kj, ki, kk);
                qk = mfma32(kj, qi, qk);
            }
            const int i = 16 * it + c;
            const bool apart = run_mode && jt != it;     // a pair's tiles are different segments
            const float Gi = Gs[i], bi = Bs[i];
            const f32x4 Gj = *(const f32x4*)(Gs + 16 * jt + 4 * q4);
            f32x4 a4;
            bf16x4 p4;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int j = 16 * jt + 4 * q4 + r;
                const float d = __expf(Gi - Gj[r]);
                a4[r] = (j < i && !apart) ? -bi * kk[r] * d : 0.f;
                p4[r] = (__bf16)((j <= i && !apart) ? p.scale * qk[r] * d : 0.f);
            }
            *(f32x4*)(As + i * LA + 16 * jt + 4 * q4) = a4;
            *(bf16x4*)(Ps + i * LP + 16 * jt + 4 * q4) = p4;
        }
        lds_barrier();

        // ---- T = (I - A)^-1 on wave 0: rows of the diagonal blocks by substitution in registers (lane groups 0 and 2 the
        // upper-left block, 1 and 3 the lower-right one, in the same instructions), then the lower-left block
        // T_lo = T_11 A_lo T_00, computed transposed (T_lo^T = T_00^T (A_lo^T T_11^T)) so that the lane again holds a row.
        // Leaves T diag(beta) and -T diag(beta e^G) in LDS as bf16, tile by tile.
        if (w == 0) {
            float t[16];
            const int blk = q4 & 1;
            unit_lower_inverse_row<true>(As + blk * (16 * LA + 16), LA, c, t);
            // the rows pass through LDS to reach the lanes in operand order (row c, columns 4 q4 ..+3)
#pragma unroll
            for (int j4 = 0; j4 < 4; j4++) *(f32x4*)(Ts + (16 * blk + c) * LX + 4 * j4) = f32x4{t[4 * j4], t[4 * j4 + 1], t[4 * j4 + 2], t[4 * j4 + 3]};
            wave_lds_order();
            const f32x4 G0 = *(const f32x4*)(Gs + 4 * q4), B0 = *(const f32x4*)(Bs + 4 * q4);
            const f32x4 t00 = *(const f32x4*)(Ts + c * LX + 4 * q4);
            f32x4 e0;
            bf16x4 u4, w4;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                e0[r] = B0[r] * __expf(G0[r]);
                u4[r] = (__bf16)(t00[r] * B0[r]);
                w4[r] = (__bf16)(-t00[r] * e0[r]);
            }
            *(bf16x4*)(Tus + c * LP + 4 * q4) = u4;
            *(bf16x4*)(Tws + c * LP + 4 * q4) = w4;
            {
                const float* T1s = Ts + 16 * LX;
                const f32x4 G1 = *(const f32x4*)(Gs + 16 + 4 * q4), B1 = *(const f32x4*)(Bs + 16 + 4 * q4);
                const f32x4 t11 = *(const f32x4*)(T1s + c * LX + 4 * q4);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    u4[r] = (__bf16)(t11[r] * B1[r]);
                    w4[r] = (__bf16)(-t11[r] * B1[r] * __expf(G1[r]));
                }
                *(bf16x4*)(Tus + (16 + c) * LP + 16 + 4 * q4) = u4;
                *(bf16x4*)(Tws + (16 + c) * LP + 16 + 4 * q4) = w4;
                f32x4 tlo = zero4();
                if (!run_mode) {      // (a pair's tiles are different segments: A_lo = 0, so is T_lo)
                    f32x4 x = zero4();
#pragma unroll
                    for (int s4 = 0; s4 < 4; s4++)        // X[j][i] = sum_m A_lo[m][j] T_11[i][m]
                        x = mfma4(As[(16 + 4 * s4 + q4) * LA + c], T1s[c * LX + 4 * s4 + q4], x);
#pragma unroll
                    for (int r = 0; r < 4; r++) Xs[(4 * q4 + r) * LX + c] = x[r];
                    wave_lds_order();
#pragma unroll
                    for (int s4 = 0; s4 < 4; s4++)        // T_lo[16 + i][j'] = sum_j T_00[j][j'] X[j][i]
                        tlo = mfma4(Ts[(4 * s4 + q4) * LX + c], Xs[(4 * s4 + q4) * LX + c], tlo);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    u4[r] = (__bf16)(tlo[r] * B0[r]);
                    w4[r] = (__bf16)(-tlo[r] * e0[r]);
                }
                *(bf16x4*)(Tus + (16 + c) * LP + 4 * q4) = u4;
                *(bf16x4*)(Tws + (16 + c) * LP + 4 * q4) = w4;
            }
        }
        lds_barrier();   // T visible; A and the T blocks are dead, -W may take their place

        // ---- U[i][v] = sum_j Tu[i][j] V[j][v] for this wave's columns (lane = column v, registers = rows i), and this wave's
        // share of -W^T[k][i] = sum_j K[j][k] Tw[i][j]: key tiles 2w and 2w + 1, stored as -W[i][k]
        f32x4 vp[NT][2], qs[NT][2];
        {
            tok_op tu[NT], tw[NT];
#pragma unroll
            for (int it = 0; it < NT; it++) {
                const __bf16* up = Tus + (16 * it + c) * LP + 4 * q4;
                const __bf16* wp = Tws + (16 * it + c) * LP + 4 * q4;
                tu[it] = join(*(const bf16x4*)up, it ? *(const bf16x4*)(up + 16) : zero_bf4());
                tw[it] = join(*(const bf16x4*)wp, it ? *(const bf16x4*)(wp + 16) : zero_bf4());
            }
#pragma unroll
            for (int vt = 0; vt < 2; vt++) {
                const tok_op vB = join(frag_tr4(Vs, LDT, 0, 32 * w + 16 * vt, lane), frag_tr4(Vs, LDT, 16, 32 * w + 16 * vt, lane));
#pragma unroll
                for (int it = 0; it < NT; it++) {
                    vp[it][vt] = mfma32(tu[it], vB, zero4());
                    qs[it][vt] = zero4();
                }
            }
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int kt = 2 * w + h;
                const tok_op kT = join(frag_tr4(Ks, LDT, 0, 16 * kt, lane), frag_tr4(Ks, LDT, 16, 16 * kt, lane));
#pragma unroll
                for (int it = 0; it < NT; it++) *(bf16x4*)(Wn + (16 * it + c) * LW + 16 * kt + 4 * q4) = round4(mfma32(kT, tw[it], zero4()));
            }
        }
        lds_barrier();   // -W visible; every wave has read its V columns
        // The next chunk's rows are requested here: the registers they land in are free since the staging, and from here no phase
        // needs more registers than there are (one phase earlier the solve spills).  They have the three value-column phases
        // (about 4 k cycles) to arrive; requested after the V' phase (2 k cycles) the next chunk's staging waited for them.
        fetch_data();          // chunk j + 1, whose rows are known since the previous chunk
        fetch_rows(j + 2);

        // ---- V' = U + (-W) S and Q S over the 128 key rows, 32 at a time (the state tiles 2s and 2s + 1 are the B operand)
#pragma unroll
        for (int s = 0; s < KD / 32; s++) {
            bf16x8 wA[NT], qA[NT];
#pragma unroll
            for (int it = 0; it < NT; it++) {
                const __bf16* wp = Wn + (16 * it + c) * LW + 32 * s + 4 * q4;
                const __bf16* qp = Qs + (16 * it + c) * LD + 32 * s + 4 * q4;
                wA[it] = join(*(const bf16x4*)wp, *(const bf16x4*)(wp + 16));
                qA[it] = join(*(const bf16x4*)qp, *(const bf16x4*)(qp + 16));
            }
#pragma unroll
            for (int vt = 0; vt < 2; vt++) {
                const bf16x8 sb = join(round4(S[2 * s][vt]), round4(S[2 * s + 1][vt]));
#pragma unroll
                for (int it = 0; it < NT; it++) {
                    vp[it][vt] = mfma32(wA[it], sb, vp[it][vt]);
                    qs[it][vt] = mfma32(qA[it], sb, qs[it][vt]);
                }
            }
        }
        // ---- O[i][v] = s e^{G_i} (Q S)[i][v] + sum_j P[i][j] V'[j][v], rows i = 16 it + 4 q4 + r; through LDS for 16-byte stores
        f32x4 Gj[NT];
#pragma unroll
        for (int it = 0; it < NT; it++) Gj[it] = *(const f32x4*)(Gs + 16 * it + 4 * q4);
        {
            tok_op pA[NT];
#pragma unroll
            for (int it = 0; it < NT; it++) {
                const __bf16* pp = Ps + (16 * it + c) * LP + 4 * q4;
                pA[it] = join(*(const bf16x4*)pp, it ? *(const bf16x4*)(pp + 16) : zero_bf4());
            }
#pragma unroll
            for (int vt = 0; vt < 2; vt++) {
                const tok_op vb = join(round4(vp[0][vt]), round4(vp[NT - 1][vt]));
#pragma unroll
                for (int it = 0; it < NT; it++) {
                    f32x4 o = mfma32(pA[it], vb, zero4());
#pragma unroll
                    for (int r = 0; r < 4; r++) o[r] = __builtin_fmaf(p.scale * __expf(Gj[it][r]), qs[it][vt][r], o[r]);
                    *(bf16x4*)(Ow + (16 * vt + c) * LO + 16 * it + 4 * q4) = round4(o);      // O^T[v][i]
                }
            }
        }
        wave_lds_order();
        // row i = 16 it + lane%16, values 8 (lane/16) ..+7 of this wave's 32: two transposing reads, one 16-byte store
#pragma unroll
        for (int it = 0; it < NT; it++) {
            const int row = 16 * it + c;
            const __bf16* op = Ow + (8 * q4 + (c >> 2)) * LO + 16 * it + 4 * (c & 3);
            const bf16x4 lo = __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)op));
            const bf16x4 hi = __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(op + 4 * LO)));
            const int orow = Rs[row];      // -1: no such row in this chunk
            if (orow >= 0) *(bf16x8*)(p.o + row_offset(orow, p.o_tok) + hv * VD + 32 * w + 8 * q4) = join(lo, hi);
        }
        // ---- S[k][v] = e^{G_L} S[k][v] + sum_j K[j][k] (V' e^{G_L - G_j})[j][v]; skipped when nothing reads the state again
        if (!run_mode && (j + 1 < n_chunks || keep)) {
            const float GL = Gs[CH - 1];
            const float eg = __expf(GL);
            tok_op vd[2];
#pragma unroll
            for (int vt = 0; vt < 2; vt++) {
                bf16x4 d[2];
#pragma unroll
                for (int it = 0; it < NT; it++)
#pragma unroll
                    for (int r = 0; r < 4; r++) d[it][r] = (__bf16)(vp[it][vt][r] * __expf(GL - Gj[it][r]));
                vd[vt] = join(d[0], d[NT - 1]);
            }
#pragma unroll
            for (int kt = 0; kt < 8; kt++) {
                const tok_op kT = join(frag_tr4(Ks, LDT, 0, 16 * kt, lane), frag_tr4(Ks, LDT, 16, 16 * kt, lane));
#pragma unroll
                for (int vt = 0; vt < 2; vt++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) S[kt][vt][r] *= eg;
                    S[kt][vt] = mfma32(kT, vd[vt], S[kt][vt]);
                }
            }
        }
    }

    if (keep) {
        float* hp = p.ht + ((p.ht_idx[seg] * p.hv + hv) * KD + 4 * q4) * VD + 32 * w + c;
#pragma unroll
        for (int kt = 0; kt < 8; kt++)
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int vt = 0; vt < 2; vt++) hp[(16 * kt + r) * VD + 16 * vt] = S[kt][vt][r];
    }
  }
}

// 32-token chunks, 254 registers, two workgroups per compute unit; the recurrent entry point's kernel also pairs up leaves.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gdn_wy32_kernel(const GdnParams p) { gdn_wy_body<false>(p); }
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gdn_wy_pairs_kernel(const GdnParams p) { gdn_wy_body<true>(p); }

// pairs: the recurrent entry point (short segments, leaves two to a chunk)
int gdn_wy_launch(GdnParams p, bool pairs, hipStream_t stream) {
    if (p.dv != VD) return spinf_fail(SPINF_E_ARG, "gdn: value head dim %d, the chunked kernel is built for 128", p.dv);
    // segments per workgroup: as many as leave about eight workgroups per compute unit (of 256), 16 at most
    p.run = 1;
    while (pairs && p.run < 16 && (p.n_seg + 2 * p.run - 1) / (2 * p.run) * p.hv >= 2048) p.run *= 2;
    const long blocks = (p.n_seg + p.run - 1) / p.run * p.hv;
    if (blocks > INT32_MAX) return spinf_fail(SPINF_E_ARG, "gdn: too many segments");
    if (!pairs) hipLaunchKernelGGL(gdn_wy32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(gdn_wy_pairs_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}
