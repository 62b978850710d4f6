// Gated DeltaNet scan for gfx950 (MI355X).
//
// Stands in for gdn.recurrent / gdn.chunked (spinf_serve/models/qwen35/gdn.py:197-235, :109-133).  The recurrence per value
// head, state S [K, V] in fp32 (gdn.py:176-186):
//     S <- exp(g_t) S ;  d = beta_t (v_t - S^T k_t) ;  S <- S + k_t d^T ;  o_t = S^T (scale q_t)
// value head hv reads query/key head hv / (HV / H) (gdn.py:167); segment s starts from h0[h0_idx[s]] (or zero) and leaves
// its final state in ht[ht_idx[s]] when that index is >= 0 (gdn.py:172-175,187-190).
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

#include "gdn_tiles.h"

using namespace gdn_tiles;

// ---------------------------------------------------------------------------------------------- short segments
// The recurrent entry point for value head dims other than 128 (128 runs the workgroup kernel of gdn_chunk.hip, leaves two
// to a chunk): meant for the short segments of a trie (a handful of tokens after a fork), thousands per call.
// One wave per (segment, value head, 32 value columns) and no workgroup barrier anywhere.  The wave walks its segment in
// mini-chunks of 16 tokens with the same WY algebra as the workgroup kernel of gdn_chunk.hip (A = -strict_tril(beta_i K_i.K_j e^{G_i-G_j}),
// T = (I - A)^-1, U = T diag(beta) V, -W = -T diag(beta e^G) K, V' = U - W S, O = s e^G Q S + P V', S <- e^{G_L} S +
// K^T (V' e^{G_L-G})), on 16x16 MFMA tiles laid out so that every product's result is already the next product's operand:
//   * the state slice S[128][32] stays in fp32 accumulator layout (lane = value column, 4 consecutive key rows per tile): two
//     key tiles side by side are the B operand of a 16x16x32 product over a permuted contraction index, and K and Q rows are
//     fetched in that same permutation, so S is never moved, only rounded to bf16 on the way into the matrix core;
//   * Q.K^T and K.K^T are computed transposed (lane = row i, registers = columns j), which is the A operand layout of P in
//     O = P V' and the row layout (I - A)^-1 is solved in; every lane solves row i = lane % 16 by substitution in registers;
//   * -W^T and V' come out of their products as the A and B operands of the products that consume them.
// The state is kept and accumulated in fp32; products take bf16 operands, as in the workgroup kernel.
namespace {
constexpr int MC = 16;      // tokens per mini-chunk
constexpr int LDK = 136;    // row stride (elements) of the K tile in LDS
constexpr int LDV = 40;     // row stride of the V and O tiles
constexpr int LDA = 20;     // row stride (floats) of A
}  // namespace

__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(3, 3))) void gdn_short_kernel(const GdnParams p) {
    constexpr int K = 128;
    __shared__ __attribute__((aligned(16))) __bf16 Ksm[MC * LDK];
    __shared__ __attribute__((aligned(16))) __bf16 Vsm[MC * LDV];
    __shared__ __attribute__((aligned(16))) __bf16 Osm[MC * LDV];
    __shared__ __attribute__((aligned(16))) float As[MC * LDA];
    __shared__ __attribute__((aligned(16))) float Gs[MC];
    __shared__ __attribute__((aligned(16))) float Bs[MC];

    const int nvb = p.dv / 32;
    const long b = blockIdx.x;
    const int iv = (int)(b % nvb);
    const long nh = b / nvb;
    const long n = nh / p.hv;
    const int hv = (int)(nh % p.hv);
    const int hk = hv / (p.hv / p.h);
    const int lane = threadIdx.x, c = lane & 15, q4 = lane >> 4;
    const int vrow = lane >> 2, vcol = (lane & 3) * 8;      // this lane's 16-byte piece of the V and O tiles

    // state: S[kt][vt][r] = S[16 kt + 4 q4 + r][32 iv + 16 vt + c]
    f32x4 S[8][2];
#pragma unroll
    for (int kt = 0; kt < 8; kt++)
#pragma unroll
        for (int vt = 0; vt < 2; vt++) S[kt][vt] = zero4();
    if (p.h0 != nullptr && p.h0_idx != nullptr) {
        const long src = p.h0_idx[n];
        if (src >= 0) {
            const float* hp = p.h0 + ((src * p.hv + hv) * K + 4 * q4) * p.dv + 32 * iv + c;
#pragma unroll
            for (int kt = 0; kt < 8; kt++)
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int vt = 0; vt < 2; vt++) S[kt][vt][r] = hp[(long)(16 * kt + r) * p.dv + 16 * vt];
        }
    }
    const bool keep = p.ht != nullptr && p.ht_idx != nullptr && p.ht_idx[n] >= 0;
    const long bos = p.cu[n], eos = p.cu[n + 1];
    const int T = (int)(eos - bos);

    for (int c0 = 0; c0 < T; c0 += MC) {
        const int L = min(MC, T - c0);
        // ---- fetch: lane (c, q4) takes row c of K and Q in the contraction order of the state operand (per 32 columns: 4 q4 ..+3
        // and 16 + 4 q4 ..+3), g and beta of row c; lane (vrow, vcol) a 16-byte piece of V.  Rows >= L are zero.
        long rc = -1, rv = -1;
        if (c < L) { const long t = bos + c0 + c; rc = p.idx ? p.idx[t] : t; }
        if (vrow < L) { const long t = bos + c0 + vrow; rv = p.idx ? p.idx[t] : t; }
        bf16x4 klo[4], khi[4], qlo[4], qhi[4];
#pragma unroll
        for (int s = 0; s < 4; s++)
#pragma unroll
            for (int j = 0; j < 4; j++) { klo[s][j] = (__bf16)0.f; khi[s][j] = (__bf16)0.f; qlo[s][j] = (__bf16)0.f; qhi[s][j] = (__bf16)0.f; }
        float gv = 0.f, bv = 0.f;
        if (rc >= 0) {
            const __bf16* kp = p.k + rc * p.q_tok + (long)hk * K + 4 * q4;
            const __bf16* qp = p.q + rc * p.q_tok + (long)hk * K + 4 * q4;
#pragma unroll
            for (int s = 0; s < 4; s++) {
                klo[s] = *(const bf16x4*)(kp + 32 * s);
                khi[s] = *(const bf16x4*)(kp + 32 * s + 16);
                qlo[s] = *(const bf16x4*)(qp + 32 * s);
                qhi[s] = *(const bf16x4*)(qp + 32 * s + 16);
            }
            gv = p.g[rc * p.g_tok + hv];
            bv = (float)p.beta[rc * p.g_tok + hv];
        }
        bf16x8 vv;
#pragma unroll
        for (int j = 0; j < 8; j++) vv[j] = (__bf16)0.f;
        if (rv >= 0) vv = *(const bf16x8*)(p.v + rv * p.v_tok + (long)hv * p.dv + 32 * iv + vcol);

        wave_lds_order();   // the previous mini-chunk's reads come first
#pragma unroll
        for (int s = 0; s < 4; s++) {
            *(bf16x4*)(Ksm + c * LDK + 32 * s + 4 * q4) = klo[s];
            *(bf16x4*)(Ksm + c * LDK + 32 * s + 16 + 4 * q4) = khi[s];
        }
        *(bf16x8*)(Vsm + vrow * LDV + vcol) = vv;
        // G_c = g_0 + .. + g_c: every group of 16 lanes holds the same 16 values
        const float Gi = row_prefix_sum(gv);
        Gs[c] = Gi;
        Bs[c] = bv;
        wave_lds_order();
        const f32x4 Gj = *(const f32x4*)(Gs + 4 * q4), Bj = *(const f32x4*)(Bs + 4 * q4);
        const float GL = Gs[MC - 1];

        // ---- (K K^T)^T and (Q K^T)^T: lane = row i = c, registers = columns j = 4 q4 + r
        f32x4 kk = {0.f, 0.f, 0.f, 0.f}, qk = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const bf16x8 kf = join(klo[s], khi[s]);
            kk = mfma32(kf, kf, kk);
            qk = mfma32(kf, join(qlo[s], qhi[s]), qk);
        }
        bf16x4 pA;     // P[i][j] = s Q_i.K_j e^{G_i - G_j}, j <= i
        {
            f32x4 a4;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int j = 4 * q4 + r;
                const float d = __expf(Gi - Gj[r]);
                a4[r] = j < c ? -bv * kk[r] * d : 0.f;
                pA[r] = (__bf16)(j <= c ? p.scale * qk[r] * d : 0.f);
            }
            *(f32x4*)(As + c * LDA + 4 * q4) = a4;
        }
        wave_lds_order();
        // ---- row c of T = (I - A)^-1, solved by every group of 16 lanes alike
        float t[MC];
        unit_lower_inverse_row<false>(As, LDA, c, t);
        // T diag(beta) and -T diag(beta e^G), columns 4 q4 + r of row c
        bf16x4 tuA, twB;
        const f32x4 tq = pick4(t, q4);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float tb = tq[r] * Bj[r];
            tuA[r] = (__bf16)tb;
            twB[r] = (__bf16)(-tb * __expf(Gj[r]));
        }
        // ---- U[i][v] = sum_j Tu[i][j] V[j][v]   (lane = column v, registers = rows i)
        f32x4 vp[2], qs[2];
#pragma unroll
        for (int vt = 0; vt < 2; vt++) {
            vp[vt] = mfma16(tuA, frag_tr4(Vsm, LDV, 0, 16 * vt, lane), zero4());
            qs[vt] = zero4();
        }
        // ---- -W^T[k][i] = sum_j K[j][k] Tw[i][j]; then V' = U + (-W) S and Q S over the 128 key rows, 32 at a time
#pragma unroll
        for (int s = 0; s < 4; s++) {
            const f32x4 w0 = mfma16(frag_tr4(Ksm, LDK, 0, 32 * s, lane), twB, zero4());
            const f32x4 w1 = mfma16(frag_tr4(Ksm, LDK, 0, 32 * s + 16, lane), twB, zero4());
            const bf16x8 wA = join(round4(w0), round4(w1));
            const bf16x8 qA = join(qlo[s], qhi[s]);
#pragma unroll
            for (int vt = 0; vt < 2; vt++) {
                const bf16x8 sb = join(round4(S[2 * s][vt]), round4(S[2 * s + 1][vt]));
                vp[vt] = mfma32(wA, sb, vp[vt]);
                qs[vt] = mfma32(qA, sb, qs[vt]);
            }
        }
        // ---- O[i][v] = s e^{G_i} (Q S)[i][v] + sum_j P[i][j] V'[j][v], rows i = 4 q4 + r; through LDS for 16-byte stores
        bf16x4 vb[2];
#pragma unroll
        for (int vt = 0; vt < 2; vt++) {
            vb[vt] = round4(vp[vt]);
            const f32x4 o = mfma16(pA, vb[vt], zero4());
#pragma unroll
            for (int r = 0; r < 4; r++)
                Osm[(4 * q4 + r) * LDV + 16 * vt + c] = (__bf16)__builtin_fmaf(p.scale * __expf(Gj[r]), qs[vt][r], o[r]);
        }
        wave_lds_order();
        if (rv >= 0) *(bf16x8*)(p.o + rv * p.o_tok + (long)hv * p.dv + 32 * iv + vcol) = *(const bf16x8*)(Osm + vrow * LDV + vcol);
        // ---- S[k][v] = e^{G_L} S[k][v] + sum_j K[j][k] (V' e^{G_L - G_j})[j][v]; skipped when nothing reads the state again
        if (c0 + MC < T || keep) {
            const float eg = __expf(GL);
            bf16x4 vd[2];
#pragma unroll
            for (int vt = 0; vt < 2; vt++)
#pragma unroll
                for (int r = 0; r < 4; r++) vd[vt][r] = (__bf16)(vp[vt][r] * __expf(GL - Gj[r]));
#pragma unroll
            for (int kt = 0; kt < 8; kt++) {
                const bf16x4 kT = frag_tr4(Ksm, LDK, 0, 16 * kt, lane);
#pragma unroll
                for (int vt = 0; vt < 2; vt++) {
#pragma unroll
                    for (int r = 0; r < 4; r++) S[kt][vt][r] *= eg;
                    S[kt][vt] = mfma16(kT, vd[vt], S[kt][vt]);
                }
            }
        }
    }
    if (keep) {
        float* hp = p.ht + ((p.ht_idx[n] * p.hv + hv) * K + 4 * q4) * p.dv + 32 * iv + c;
#pragma unroll
        for (int kt = 0; kt < 8; kt++)
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int vt = 0; vt < 2; vt++) hp[(long)(16 * kt + r) * p.dv + 16 * vt] = S[kt][vt][r];
    }
}

int gdn_wy_launch(GdnParams p, bool pairs, hipStream_t stream);   // gdn_chunk.hip

extern "C" int spinf_gdn_fwd(const spinf_gdn_args* a, void* stream) {
    if (!a) return spinf_fail(SPINF_E_ARG, "gdn: null args");
    if (a->n_seg <= 0) return SPINF_OK;
    if (!a->q || !a->k || !a->v || !a->g || !a->beta || !a->o || !a->cu) return spinf_fail(SPINF_E_ARG, "gdn: null pointer");
    if (a->dk != 128) return spinf_fail(SPINF_E_ARG, "gdn: key head dim %d, only 128 is built", a->dk);
    if (a->dv <= 0 || a->dv % 32) return spinf_fail(SPINF_E_ARG, "gdn: value head dim %d not a multiple of 32", a->dv);
    if (a->h <= 0 || a->hv <= 0 || a->hv % a->h) return spinf_fail(SPINF_E_ARG, "gdn: hv %d not a multiple of h %d", a->hv, a->h);
    if (a->q_tok % 8) return spinf_fail(SPINF_E_ARG, "gdn: q/k row stride must be a multiple of 8 elements");
    if (((uintptr_t)a->q | (uintptr_t)a->k) % 16) return spinf_fail(SPINF_E_ARG, "gdn: q/k must be 16-byte aligned");
    if ((a->h0 == nullptr) != (a->h0_idx == nullptr) && a->h0 == nullptr) return spinf_fail(SPINF_E_ARG, "gdn: h0_idx without h0");
    if (a->ht_idx != nullptr && a->ht == nullptr) return spinf_fail(SPINF_E_ARG, "gdn: ht_idx without ht");
    if (a->q_tok <= 0 || a->v_tok <= 0 || a->g_tok <= 0 || a->o_tok <= 0 || (a->q_tok | a->v_tok | a->g_tok | a->o_tok) >> 31)
        return spinf_fail(SPINF_E_ARG, "gdn: row strides must be positive and below 2^31 elements");
    if (a->v_tok % 8 || a->o_tok % 8) return spinf_fail(SPINF_E_ARG, "gdn: v/o row stride must be a multiple of 8 elements");
    if (((uintptr_t)a->v | (uintptr_t)a->o) % 16) return spinf_fail(SPINF_E_ARG, "gdn: v/o must be 16-byte aligned");
    GdnParams p;
    p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v; p.g = a->g; p.beta = (const __bf16*)a->beta;
    p.o = (__bf16*)a->o;
    p.q_tok = a->q_tok; p.v_tok = a->v_tok; p.g_tok = a->g_tok; p.o_tok = a->o_tok;
    p.h = a->h; p.hv = a->hv; p.dk = a->dk; p.dv = a->dv; p.scale = a->scale;
    p.cu = (const long*)a->cu; p.idx = (const long*)a->idx; p.n_seg = a->n_seg;
    p.h0 = a->h0; p.h0_idx = (const long*)a->h0_idx; p.ht = a->ht; p.ht_idx = (const long*)a->ht_idx;
    p.run = 1;
    hipStream_t s = (hipStream_t)stream;
    if (a->mode == 1) return gdn_wy_launch(p, false, s);
    if (a->mode != 0) return spinf_fail(SPINF_E_ARG, "gdn: unknown mode %d", a->mode);
    if (a->dv == 128) return gdn_wy_launch(p, true, s);   // the workgroup kernel shares the per-head work of the four 32-column waves
    const long blocks = a->n_seg * a->hv * (a->dv / 32);
    if (blocks > INT32_MAX) return spinf_fail(SPINF_E_ARG, "gdn: too many segments");
    hipLaunchKernelGGL(gdn_short_kernel, dim3((unsigned)blocks), dim3(64), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}
