// Gated DeltaNet, chunked WY form, one fused kernel: stands in for gdn.chunked (spinf_serve/models/qwen35/gdn.py:109-133),
// i.e. for fla's cumsum -> intra-chunk WY solve -> state recurrence (gdn.py:21-106) -> output pipeline, without writing
// the per-chunk state snapshots or the w / u / v_new intermediates to memory.
//
// One workgroup (4 waves) owns one (segment, value head) and walks its 32-token chunks in order; wave w owns value columns
// 32w .. 32w+31 of the state S [K=128, V=128], which never leaves its fp32 accumulator registers.  The four waves share
// only the staged K / Q / V rows of the chunk: each wave forms the (small) token x token quantities itself, so between two
// chunks there are two workgroup barriers (rows consumed, rows staged) and none inside a chunk, and three workgroups fit a
// compute unit (44 KB of LDS, <= 168 registers) and fill each other's latencies.  Per chunk, G = cumsum(g), D_ij = e^{G_i - G_j}:
//     A   = -strict_tril(beta_i (K K^T)_ij D_ij)         T = (I - A)^-1      (fp32: two 16 x 16 blocks solved by substitution
//                                                                             in registers, merged with fp32 MFMAs)
//     U   = T diag(beta) V          -W = -T diag(beta e^G) K                 (bf16 MFMA, fp32 accumulate)
//     V'  = U - W S                 O = s e^{G_i} (Q S)_i + tril(s (Q K^T) D) V'
//     S  <- e^{G_L} S + (K e^{G_L - G})^T V'
// Every product leaves its result in the register layout the next product takes as an operand (see gdn_tiles.h), so only
// the output rows pass through LDS again (for 16-byte stores).
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"
#include "gdn_tiles.h"

using namespace gdn_tiles;

#ifdef SPINF_TRACE
__device__ long g_gdn_trace[16];
extern "C" int spinf_debug_gdn_trace(long* out) { return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_gdn_trace), sizeof(long) * 16, 0, hipMemcpyDeviceToHost); }
#define GT_CLK(v) const long v = clock64()
#define GT_ADD(slot, val) do { if (threadIdx.x == 64 && blockIdx.x == 7) g_gdn_trace[slot] += (val); } while (0)
#else
#define GT_CLK(v) do { } while (0)
#define GT_ADD(slot, val) do { } while (0)
#endif

namespace {

constexpr int CH = 32;         // chunk
constexpr int KD = 128;        // key head dim
constexpr int VD = 128;        // value head dim
constexpr int LD = 136;        // row stride (elements) of the [32, 128] bf16 tiles
constexpr int LA = 36;         // row stride (floats) of the fp32 [32, 32] matrix A
constexpr int LX = 20;         // row stride (floats) of the 16 x 16 merge scratch
constexpr int LO = 40;         // row stride (elements) of a wave's [32, 32] output tile

}  // namespace

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gdn_chunk_kernel(const GdnParams p) {
    __shared__ __attribute__((aligned(16))) __bf16 Ks[CH * LD];
    __shared__ __attribute__((aligned(16))) __bf16 Qs[CH * LD];
    __shared__ __attribute__((aligned(16))) __bf16 Vs[CH * LD];
    // A, the upper-left block of T and the merge intermediate are written by all four waves with identical values (each
    // wave reads back what it wrote itself or the same number from another wave)
    __shared__ __attribute__((aligned(16))) float As[CH * LA];
    __shared__ __attribute__((aligned(16))) float Ts[32 * LX];     // T_00 (rows 0..15) and T_11 (rows 16..31)
    __shared__ __attribute__((aligned(16))) float Xs[16 * LX];
    __shared__ __attribute__((aligned(16))) __bf16 Os[4 * CH * LO];
    __shared__ __attribute__((aligned(16))) float Gs[CH];
    __shared__ __attribute__((aligned(16))) float Bs[CH];
    __shared__ long Rs[CH];

    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), c = lane & 15, q4 = lane >> 4;
    const long seg = blockIdx.x / p.hv;
    const int hv = (int)(blockIdx.x % p.hv);
    const int hk = hv / (p.hv / p.h);
    const long bos = p.cu[seg], eos = p.cu[seg + 1];
    const int T = (int)(eos - bos);
    __bf16* Ow = Os + w * CH * LO;

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
                    for (int vt = 0; vt < 2; vt++) S[kt][vt][r] = hp[(long)(16 * kt + r) * VD + 16 * vt];
        }
    }
    const bool keep = p.ht != nullptr && p.ht_idx != nullptr && p.ht_idx[seg] >= 0;

    // The next chunk's rows are fetched into registers while the current chunk is computed, and the stream rows (idx) of
    // the chunk after that one chunk earlier still, so that no load ever waits for the load of its own address.
    // Thread -> 16-byte piece tid%16 of chunk rows tid/16 and tid/16 + 16 (one load instruction of a wave covers four whole
    // rows); threads 0..31 also -> g, beta and the stream row of chunk row tid.
    bf16x8 pk[2], pq[2], pv[2];
    long pr64 = -1;
    float pg = 0.f;
    __bf16 pbeta = (__bf16)0.f;   // (kept as loaded: converting here would make the wave wait for the load at once)
    long ra[2] = {-1, -1}, rb = -1;
    auto fetch_rows = [&](const int c0) __attribute__((always_inline)) {
        const int L = min(CH, T - c0);      // <= 0: there is no such chunk
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
            const int row = (tid >> 4) + 16 * cc;
            ra[cc] = -1;
            if (row < L) {
                const long t = bos + c0 + row;
                ra[cc] = p.idx ? p.idx[t] : t;
            }
        }
        rb = -1;
        if (tid < CH && tid < L) {
            const long t = bos + c0 + tid;
            rb = p.idx ? p.idx[t] : t;
        }
    };
    auto fetch_data = [&]() __attribute__((always_inline)) {
        const int col = (tid & 15) * 8;
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
#pragma unroll
            for (int j = 0; j < 8; j++) { pk[cc][j] = (__bf16)0.f; pq[cc][j] = (__bf16)0.f; pv[cc][j] = (__bf16)0.f; }
            if (ra[cc] >= 0) {
                pk[cc] = *(const bf16x8*)(p.k + ra[cc] * p.q_tok + (long)hk * KD + col);
                pq[cc] = *(const bf16x8*)(p.q + ra[cc] * p.q_tok + (long)hk * KD + col);
                pv[cc] = *(const bf16x8*)(p.v + ra[cc] * p.v_tok + (long)hv * VD + col);
            }
        }
        pr64 = rb;
        pg = 0.f;
        pbeta = (__bf16)0.f;
        if (rb >= 0) {
            pg = p.g[rb * p.g_tok + hv];
            pbeta = p.beta[rb * p.g_tok + hv];
        }
    };
    fetch_rows(0);
    fetch_data();
    fetch_rows(CH);

    for (int c0 = 0; c0 < T; c0 += CH) {
        const int L = min(CH, T - c0);
        GT_CLK(g0);
        lds_barrier();   // every wave is done with the previous chunk's rows
        // ---- stage the chunk from the prefetch registers (rows >= L are zero): cumulative g, beta, stream rows, K / Q / V
        if (tid < CH) {
            float x = row_prefix_sum(pg);
            x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, false));  // row_bcast:15 -> lanes 16..31
            Gs[tid] = x;
            Bs[tid] = (float)pbeta;
            Rs[tid] = pr64;
        }
        {
            const int col = (tid & 15) * 8;
#pragma unroll
            for (int cc = 0; cc < 2; cc++) {
                const int row = (tid >> 4) + 16 * cc;
                *(bf16x8*)(Ks + row * LD + col) = pk[cc];
                *(bf16x8*)(Qs + row * LD + col) = pq[cc];
                *(bf16x8*)(Vs + row * LD + col) = pv[cc];
            }
        }
        lds_barrier();
        GT_CLK(g1);

        // Token tiles: tile 0 = chunk rows 0..15, tile 1 = rows 16..31.  Index [it] = tile of the row i = 16 it + c this lane
        // owns in a transposed result, [jt] = tile of the columns j = 16 jt + 4 q4 + r its registers hold.
        const float GL = Gs[CH - 1];
        float Gi[2], bi[2];
        f32x4 Gj[2], Bj[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
            Gi[t] = Gs[16 * t + c];
            bi[t] = Bs[16 * t + c];
            Gj[t] = *(const f32x4*)(Gs + 16 * t + 4 * q4);
            Bj[t] = *(const f32x4*)(Bs + 16 * t + 4 * q4);
        }
        // ---- (K K^T)^T and (Q K^T)^T, tiles (jt, it) = (0,0), (0,1), (1,1); (1,0) lies above the diagonal
        f32x4 kk[3], qk[3];
#pragma unroll
        for (int x = 0; x < 3; x++) { kk[x] = zero4(); qk[x] = zero4(); }
#pragma unroll
        for (int s = 0; s < KD / 32; s++) {
            const bf16x8 k0 = *(const bf16x8*)(Ks + c * LD + 32 * s + 8 * q4);
            const bf16x8 k1 = *(const bf16x8*)(Ks + (16 + c) * LD + 32 * s + 8 * q4);
            const bf16x8 q0 = *(const bf16x8*)(Qs + c * LD + 32 * s + 8 * q4);
            const bf16x8 q1 = *(const bf16x8*)(Qs + (16 + c) * LD + 32 * s + 8 * q4);
            kk[0] = mfma32(k0, k0, kk[0]);
            kk[1] = mfma32(k0, k1, kk[1]);
            kk[2] = mfma32(k1, k1, kk[2]);
            qk[0] = mfma32(k0, q0, qk[0]);
            qk[1] = mfma32(k0, q1, qk[1]);
            qk[2] = mfma32(k1, q1, qk[2]);
        }
        // A[i][j] (fp32, to LDS) and P[i][j] = s Q_i.K_j e^{G_i - G_j}, j <= i (kept as the A operand of O = P V')
        bf16x8 pA[2];
        {
            bf16x4 pT[3];
#pragma unroll
            for (int x = 0; x < 3; x++) {
                const int jt = x >> 1, it = (x + 1) >> 1;     // (0,0), (0,1), (1,1)
                const int i = 16 * it + c;
                f32x4 a4;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int j = 16 * jt + 4 * q4 + r;
                    const float d = __expf(Gi[it] - Gj[jt][r]);
                    a4[r] = j < i ? -bi[it] * kk[x][r] * d : 0.f;
                    pT[x][r] = (__bf16)(j <= i ? p.scale * qk[x][r] * d : 0.f);
                }
                *(f32x4*)(As + i * LA + 16 * jt + 4 * q4) = a4;
            }
            bf16x4 z;
#pragma unroll
            for (int r = 0; r < 4; r++) z[r] = (__bf16)0.f;
            pA[0] = join(pT[0], z);
            pA[1] = join(pT[1], pT[2]);
        }
        wave_lds_order();
        GT_CLK(g2);

        // ---- T = (I - A)^-1: rows c of the two diagonal blocks in registers, then the lower-left block
        // T_lo = T_11 A_lo T_00, computed transposed (T_lo^T = T_00^T (A_lo^T T_11^T)) so that the lane again holds row 16 + c.
        f32x4 t00, t11, tlo;
        {
            const float* T1s = Ts + 16 * LX;
            // the rows pass through LDS to reach the lanes in operand order (row c, columns 4 q4 ..+3; single elements for the
            // fp32 products); all four groups of 16 lanes write the same values
            // lane groups 0 and 2 solve the upper-left block, groups 1 and 3 the lower-right one, in the same instructions
            float t[16];
            const int blk = q4 & 1;
            unit_lower_inverse_row(As + blk * (16 * LA + 16), LA, c, t);
#pragma unroll
            for (int j4 = 0; j4 < 4; j4++) *(f32x4*)(Ts + (16 * blk + c) * LX + 4 * j4) = f32x4{t[4 * j4], t[4 * j4 + 1], t[4 * j4 + 2], t[4 * j4 + 3]};
            wave_lds_order();
            t00 = *(const f32x4*)(Ts + c * LX + 4 * q4);
            t11 = *(const f32x4*)(T1s + c * LX + 4 * q4);
            f32x4 x = zero4();
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++)        // X[j][i] = sum_m A_lo[m][j] T_11[i][m]
                x = mfma4(As[(16 + 4 * s4 + q4) * LA + c], T1s[c * LX + 4 * s4 + q4], x);
#pragma unroll
            for (int r = 0; r < 4; r++) Xs[(4 * q4 + r) * LX + c] = x[r];
            wave_lds_order();
            tlo = zero4();
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++)        // T_lo[16 + i][j'] = sum_j T_00[j][j'] X[j][i]
                tlo = mfma4(Ts[(4 * s4 + q4) * LX + c], Xs[(4 * s4 + q4) * LX + c], tlo);
        }
        // T diag(beta) and -T diag(beta e^G): row 16 it + c, columns in the order of the contraction slots
        bf16x8 tu[2], tw[2];
        {
            bf16x4 u00, w00, u10, w10, u11, w11, z;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float e0 = Bj[0][r] * __expf(Gj[0][r]), e1 = Bj[1][r] * __expf(Gj[1][r]);
                u00[r] = (__bf16)(t00[r] * Bj[0][r]);
                w00[r] = (__bf16)(-t00[r] * e0);
                u10[r] = (__bf16)(tlo[r] * Bj[0][r]);
                w10[r] = (__bf16)(-tlo[r] * e0);
                u11[r] = (__bf16)(t11[r] * Bj[1][r]);
                w11[r] = (__bf16)(-t11[r] * e1);
                z[r] = (__bf16)0.f;
            }
            tu[0] = join(u00, z);
            tw[0] = join(w00, z);
            tu[1] = join(u10, u11);
            tw[1] = join(w10, w11);
        }
        GT_CLK(g3);

        // ---- U[i][v] = sum_j Tu[i][j] V[j][v]   (lane = column v, registers = rows i)
        f32x4 vp[2][2], qs[2][2];
#pragma unroll
        for (int vt = 0; vt < 2; vt++) {
            const bf16x8 vB = join(frag_tr4(Vs, LD, 0, 32 * w + 16 * vt, lane), frag_tr4(Vs, LD, 16, 32 * w + 16 * vt, lane));
#pragma unroll
            for (int it = 0; it < 2; it++) {
                vp[it][vt] = mfma32(tu[it], vB, zero4());
                qs[it][vt] = zero4();
            }
        }
        // ---- -W^T[k][i] = sum_j K[j][k] Tw[i][j]; then V' = U + (-W) S and Q S over the 128 key rows, 32 at a time
#pragma unroll
        for (int s = 0; s < KD / 32; s++) {
            const bf16x8 kT0 = join(frag_tr4(Ks, LD, 0, 32 * s, lane), frag_tr4(Ks, LD, 16, 32 * s, lane));
            const bf16x8 kT1 = join(frag_tr4(Ks, LD, 0, 32 * s + 16, lane), frag_tr4(Ks, LD, 16, 32 * s + 16, lane));
            bf16x8 wA[2], qA[2];
#pragma unroll
            for (int it = 0; it < 2; it++) {
                wA[it] = join(round4(mfma32(kT0, tw[it], zero4())), round4(mfma32(kT1, tw[it], zero4())));
                const __bf16* qp = Qs + (16 * it + c) * LD + 32 * s + 4 * q4;
                qA[it] = join(*(const bf16x4*)qp, *(const bf16x4*)(qp + 16));
            }
#pragma unroll
            for (int vt = 0; vt < 2; vt++) {
                const bf16x8 sb = join(round4(S[2 * s][vt]), round4(S[2 * s + 1][vt]));
#pragma unroll
                for (int it = 0; it < 2; it++) {
                    vp[it][vt] = mfma32(wA[it], sb, vp[it][vt]);
                    qs[it][vt] = mfma32(qA[it], sb, qs[it][vt]);
                }
            }
        }
        GT_CLK(g4);
        // the next chunk's rows are requested here, where few registers are live; they arrive during the state update
        fetch_data();          // chunk c0 + CH, whose rows are known since the previous chunk
        fetch_rows(c0 + 2 * CH);
        // ---- O[i][v] = s e^{G_i} (Q S)[i][v] + sum_j P[i][j] V'[j][v], rows i = 16 it + 4 q4 + r; through LDS for 16-byte stores
        bf16x8 vb[2];
#pragma unroll
        for (int vt = 0; vt < 2; vt++) {
            vb[vt] = join(round4(vp[0][vt]), round4(vp[1][vt]));
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const f32x4 o = mfma32(pA[it], vb[vt], zero4());
#pragma unroll
                for (int r = 0; r < 4; r++)
                    Ow[(16 * it + 4 * q4 + r) * LO + 16 * vt + c] = (__bf16)__builtin_fmaf(p.scale * __expf(Gj[it][r]), qs[it][vt][r], o[r]);
            }
        }
        wave_lds_order();
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
            const int row = (lane >> 2) + 16 * cc;
            if (row < L) *(bf16x8*)(p.o + Rs[row] * p.o_tok + (long)hv * VD + 32 * w + (lane & 3) * 8) = *(const bf16x8*)(Ow + row * LO + (lane & 3) * 8);
        }
        GT_CLK(g5);
        // ---- S[k][v] = e^{G_L} S[k][v] + sum_j K[j][k] (V' e^{G_L - G_j})[j][v]; skipped when nothing reads the state again
        if (c0 + CH < T || keep) {
            const float eg = __expf(GL);
            bf16x8 vd[2];
#pragma unroll
            for (int vt = 0; vt < 2; vt++) {
                bf16x4 d0, d1;
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    d0[r] = (__bf16)(vp[0][vt][r] * __expf(GL - Gj[0][r]));
                    d1[r] = (__bf16)(vp[1][vt][r] * __expf(GL - Gj[1][r]));
                }
                vd[vt] = join(d0, d1);
            }
#pragma unroll
            for (int kt = 0; kt < 8; kt++) {
                const bf16x8 kT = join(frag_tr4(Ks, LD, 0, 16 * kt, lane), frag_tr4(Ks, LD, 16, 16 * kt, lane));
#pragma unroll
                for (int vt = 0; vt < 2; vt++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) S[kt][vt][r] *= eg;
                    S[kt][vt] = mfma32(kT, vd[vt], S[kt][vt]);
                }
            }
        }
        GT_CLK(g6);
        GT_ADD(0, g1 - g0); GT_ADD(1, g2 - g1); GT_ADD(2, g3 - g2); GT_ADD(3, g4 - g3); GT_ADD(4, g5 - g4); GT_ADD(5, g6 - g5); GT_ADD(8, 1);
    }

    if (keep) {
        float* hp = p.ht + ((p.ht_idx[seg] * p.hv + hv) * KD + 4 * q4) * VD + 32 * w + c;
#pragma unroll
        for (int kt = 0; kt < 8; kt++)
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int vt = 0; vt < 2; vt++) hp[(long)(16 * kt + r) * VD + 16 * vt] = S[kt][vt][r];
    }
}

int gdn_chunked_launch(const GdnParams& p, long max_len, hipStream_t stream) {
    (void)max_len;
    if (p.dv != VD) return spinf_fail(SPINF_E_ARG, "gdn chunked: value head dim %d, only 128 is built", p.dv);
    const long blocks = p.n_seg * p.hv;
    if (blocks > INT32_MAX) return spinf_fail(SPINF_E_ARG, "gdn chunked: too many segments");
    hipLaunchKernelGGL(gdn_chunk_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn chunked: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}
