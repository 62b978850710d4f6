// Gated DeltaNet, chunk-64 WY form, one fused kernel: stands in for gdn.chunked (spinf_serve/models/qwen35/gdn.py:109-133),
// i.e. for fla's cumsum -> intra-chunk WY solve -> state recurrence (gdn.py:21-106) -> output pipeline, without writing
// the per-chunk state snapshots or the w / u / v_new intermediates to memory.
//
// One workgroup (8 waves) owns one (segment, value head) and walks its 64-token chunks in order.  The state S [K=128, V=128]
// lives in fp32 MFMA accumulators (a wave owns 32 key rows x 64 value columns) and is mirrored once per chunk as bf16 S^T in LDS,
// where it serves as an MFMA operand.  Per chunk, with G = cumsum(g), D_ij = exp(G_i - G_j):
//     A   = -strict_tril(beta_i (K K^T)_ij D_ij)         T = (I - A)^-1        (fp32, blocked forward substitution)
//     U   = T diag(beta) V          W = T diag(beta e^G) K                     (bf16 MFMA, fp32 accumulate)
//     V'  = U - W S                 O = s e^{G_i} (Q S)_i + tril(s (Q K^T) D) V'
//     S  <- e^{G_L} S + (K e^{G_L - G})^T V'
// Every product is computed in the orientation whose result has the token index on the lanes, so results go to LDS or to
// memory as 8-byte row-major vectors; operands whose contraction index is their row index are read with
// ds_read_b64_tr_b16.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

struct GdnParams {
    const __bf16* q; const __bf16* k; const __bf16* v; const float* g; const __bf16* beta; __bf16* o;
    long q_tok, v_tok, g_tok, o_tok;
    int h, hv, dk, dv; float scale;
    const long* cu; const long* idx; long n_seg;
    const float* h0; const long* h0_idx; float* ht; const long* ht_idx;
};

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

constexpr int C = 64;          // chunk
constexpr int KD = 128;        // key head dim
constexpr int VD = 128;        // value head dim
constexpr int LD = 136;        // row stride (elements) of the [*, 128] bf16 tiles: 272 B, b128 row reads hit 16 distinct bank groups
constexpr int LT = 72;         // row stride of the [64, 64] bf16 tiles
constexpr int LA = 68;         // row stride (floats) of the fp32 [64, 64] matrix

// LDS map (bytes)
constexpr int OFF_K = 0;                         // K   [64][LD] bf16
constexpr int OFF_Q = OFF_K + C * LD * 2;        // Q   [64][LD]
constexpr int OFF_V = OFF_Q + C * LD * 2;        // V, later V' [64][LD]
constexpr int OFF_A = OFF_V + C * LD * 2;        // A / T fp32 [64][LA]; later V' e^{G_L - G} bf16 [64][LD] (same size)
constexpr int OFF_TU = OFF_A + C * LD * 2;       // T diag(beta)            bf16 [64][LT]
constexpr int OFF_TW = OFF_TU + C * LT * 2;      // -T diag(beta e^G)       bf16 [64][LT]
constexpr int OFF_P = OFF_TW + C * LT * 2;       // tril(s Q K^T D)         bf16 [64][LT]
constexpr int OFF_W = OFF_P + C * LT * 2;        // -W  [64][LD] bf16
constexpr int OFF_ST = OFF_W + C * LD * 2;       // S^T [128][LD] bf16
constexpr int OFF_G = OFF_ST + VD * LD * 2;      // G [64] fp32, beta [64] fp32, idx rows [64] int64
constexpr int OFF_X = OFF_G + 64 * 4 * 2 + 64 * 8;   // scratch fp32 [32][36] for the block merges
constexpr int LDS_BYTES = OFF_X + 32 * 36 * 4;
static_assert(C * LA * 4 <= C * LD * 2, "fp32 A must fit the region it shares");
static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");

__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int i = 0; i < 16; i++) z[i] = 0.f;
    return z;
}
// rows row0 + lane%32, contraction elements k0 + 8 (lane/32) .. +7, from a tile whose contraction index is contiguous
__device__ __forceinline__ bf16x8 frag_nt(const __bf16* base, int stride, int row0, int k0, int lane) {
    return *(const bf16x8*)(base + (row0 + (lane & 31)) * stride + k0 + 8 * (lane >> 5));
}
// column n0 + lane%32, contraction rows k0 + 8 (lane/32) .. +7, from a tile whose contraction index is its ROW index
__device__ __forceinline__ bf16x8 frag_tr(const __bf16* base, int stride, int k0, int n0, int lane) {
    const int tr_a = lane & 3, tr_j = (lane >> 2) & 3, tr_mb = (lane >> 4) & 1, g = lane >> 5;
    const __bf16* p = base + (k0 + 8 * g + tr_j) * stride + n0 + 16 * tr_mb + 4 * tr_a;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(p + 4 * stride));
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}
// Workgroup barrier for LDS traffic only: waits for this wave's LDS operations, not for its global loads.  __syncthreads()
// carries a memory fence in front of which the compiler drains every load in flight, the next chunk's prefetch included.
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}
__device__ __forceinline__ f32x16 mfma(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }

}  // namespace

__global__ __launch_bounds__(512) void gdn_chunk_kernel(const GdnParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    __bf16* Ks = (__bf16*)(smem + OFF_K);
    __bf16* Qs = (__bf16*)(smem + OFF_Q);
    __bf16* Vs = (__bf16*)(smem + OFF_V);
    float* As = (float*)(smem + OFF_A);
    __bf16* Vd = (__bf16*)(smem + OFF_A);
    __bf16* Tu = (__bf16*)(smem + OFF_TU);
    __bf16* Tw = (__bf16*)(smem + OFF_TW);
    __bf16* Pm = (__bf16*)(smem + OFF_P);
    __bf16* Wn = (__bf16*)(smem + OFF_W);
    __bf16* St = (__bf16*)(smem + OFF_ST);
    float* Gs = (float*)(smem + OFF_G);
    float* Bs = Gs + 64;
    long* Rs = (long*)(Bs + 64);
    float* Xs = (float*)(smem + OFF_X);

    // Eight waves, two per SIMD: every phase below is a short dependent chain (LDS reads -> MFMAs -> conversions -> LDS
    // writes -> barrier), and a second wave on the SIMD is what fills the gaps of the first.  Wave w = (wq, wh): quarter
    // wq = w % 4 of whatever a phase splits four ways (32 of 128 rows, a 32x32 tile of a 64x64 matrix), half wh = w / 4.
    const int tid = threadIdx.x, lane = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6), wq = w & 3, wh = w >> 2, n32 = lane & 31, g = lane >> 5;
    const long seg = blockIdx.x / p.hv;
    const int hv = (int)(blockIdx.x % p.hv);
    const int hk = hv / (p.hv / p.h);
    const long bos = p.cu[seg], eos = p.cu[seg + 1];
    const int T = (int)(eos - bos);

    // ---- state: S[k][v]; wave (wq, wh) owns k rows 32wq..32wq+31 of v columns 64wh..64wh+63 as two 32x32 tiles (tile j:
    // v columns 64wh + 32j ..); lane = v column, reg r = k row
    f32x16 S[2];
#pragma unroll
    for (int j = 0; j < 2; j++) S[j] = zero16();
    long src = -1;
    if (p.h0 != nullptr && p.h0_idx != nullptr) src = p.h0_idx[seg];
    if (src >= 0) {
        const float* hp = p.h0 + (src * p.hv + hv) * (long)KD * VD;
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) S[j][r] = hp[(long)(32 * wq + 8 * (r >> 2) + 4 * g + (r & 3)) * VD + 64 * wh + 32 * j + n32];
    }
    // S^T mirror (bf16): St[v][k]
    auto mirror = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                bf16x4 t;
#pragma unroll
                for (int jj = 0; jj < 4; jj++) t[jj] = (__bf16)S[j][4 * r4 + jj];
                *(bf16x4*)(St + (64 * wh + 32 * j + n32) * LD + 32 * wq + 8 * r4 + 4 * g) = t;
            }
    };
    mirror();

    // The next chunk's rows are fetched into registers while the current chunk is computed (global latency would otherwise
    // be exposed in front of every chunk: a workgroup walks its chunks strictly in order), and the stream rows of the chunk
    // after that (idx) one chunk earlier still, so that no load ever waits for the load of its own address.
    // Thread -> 16-byte piece tid%16 of chunk rows tid/16 and tid/16 + 32 (one load instruction of a wave covers four whole
    // rows); threads 0..63 also -> g, beta and the stream row of chunk row tid.
    bf16x8 pk[2], pq[2], pv[2];
    long pr64 = -1;
    float pg = 0.f;
    __bf16 pbeta = (__bf16)0.f;   // (kept as loaded: converting here would make the wave wait for the load at once)
    long ra[2] = {-1, -1}, rb = -1;     // stream rows (the thread's two K/Q/V rows; chunk row tid) of the chunk fetched next
    auto fetch_rows = [&](const int c0) __attribute__((always_inline)) {
        const int L = min(C, T - c0);      // <= 0: there is no such chunk
#pragma unroll
        for (int cc = 0; cc < 2; cc++) {
            const int row = (tid >> 4) + 32 * cc;
            ra[cc] = -1;
            if (row < L) {
                const long t = bos + c0 + row;
                ra[cc] = p.idx ? p.idx[t] : t;
            }
        }
        rb = -1;
        if (tid < 64 && tid < L) {
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
    fetch_rows(C);

    for (int c0 = 0; c0 < T; c0 += C) {
        const int L = min(C, T - c0);
        GT_CLK(g0);
        lds_barrier();   // previous chunk fully consumed (and St written)
        // ---- stage the chunk from the prefetch registers: rows, cumulative g, beta, then K / Q / V tiles (rows >= L are zero)
        if (tid < 64) {
            // inclusive prefix sum of g over the wave: within rows of 16 lanes by shifts, then across rows by broadcasts
            float x = pg;
            x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x111, 0xf, 0xf, true));   // row_shr:1
            x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x112, 0xf, 0xf, true));   // row_shr:2
            x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x114, 0xf, 0xf, true));   // row_shr:4
            x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x118, 0xf, 0xf, true));   // row_shr:8
            x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x142, 0xa, 0xf, false));  // row_bcast:15 -> rows 1, 3
            x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x143, 0xc, 0xf, false));  // row_bcast:31 -> rows 2, 3
            Gs[tid] = x;
            Bs[tid] = (float)pbeta;
            Rs[tid] = pr64;
        }
        {
            const int col = (tid & 15) * 8;
#pragma unroll
            for (int cc = 0; cc < 2; cc++) {
                const int row = (tid >> 4) + 32 * cc;
                *(bf16x8*)(Ks + row * LD + col) = pk[cc];
                *(bf16x8*)(Qs + row * LD + col) = pq[cc];
                *(bf16x8*)(Vs + row * LD + col) = pv[cc];
            }
        }
        fetch_data();          // chunk c0 + C, whose rows are known since the previous chunk
        fetch_rows(c0 + 2 * C);
        lds_barrier();
        const float GL = Gs[63];
        GT_CLK(g1);

        // ---- (a) A = -strict_tril(beta_i K_i.K_j D_ij) fp32 (waves with wh = 0), (b) P = tril(s Q_i.K_j D_ij) bf16 (wh = 1);
        // computed transposed so that a lane holds row i and 4 consecutive columns j per register group.  Tile (jt, it) = wq.
        {
            const int jt = wq >> 1, it = wq & 1;
            const __bf16* rhs = wh ? Qs : Ks;
            f32x16 acc = zero16();
#pragma unroll
            for (int s = 0; s < KD / 16; s++) acc = mfma(frag_nt(Ks, LD, 32 * jt, 16 * s, lane), frag_nt(rhs, LD, 32 * it, 16 * s, lane), acc);
            const int i = 32 * it + n32;
            const float Gi = Gs[i], bi = Bs[i];
#pragma unroll
            for (int r4 = 0; r4 < 4; r4++) {
                const int j0 = 32 * jt + 8 * r4 + 4 * g;
                bf16x4 pv4;
                float avv[4];
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int j = j0 + jj;
                    const float d = __expf(Gi - Gs[j]);
                    avv[jj] = j < i ? -bi * acc[4 * r4 + jj] * d : 0.f;
                    pv4[jj] = (__bf16)(j <= i ? p.scale * acc[4 * r4 + jj] * d : 0.f);
                }
                if (wh == 0) *(float4*)(As + i * LA + j0) = make_float4(avv[0], avv[1], avv[2], avv[3]);
                else *(bf16x4*)(Pm + i * LT + j0) = pv4;
            }
        }
        lds_barrier();
        GT_CLK(g2);

        // ---- T = (I - A)^-1 in place (fp32).  Stage 1: the four 16x16 diagonal blocks by forward substitution, wave b < 4 =
        // block b, lane c < 16 = column c of the block.
        if (w < 4 && lane < 16) {
            float t[16];
            const float* Ab = As + (16 * w) * LA + 16 * w;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float acc = (i == lane) ? 1.f : 0.f;
#pragma unroll
                for (int j = 0; j < i; j++) acc = __builtin_fmaf(Ab[i * LA + j], t[j], acc);
                t[i] = acc;
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): all reads of A done before the block is overwritten
#pragma unroll
            for (int i = 0; i < 16; i++) As[(16 * w + i) * LA + 16 * w + lane] = t[i];
        }
        lds_barrier();
        // Stages 2 and 3 are products of 16x16 / 32x32 fp32 blocks, done with v_mfma_f32_16x16x4_f32 (operands: lane l gives
        // A[l%16][l/16] and B[l/16][l%16] of a 16x4 by 4x16 step; result: lane l holds rows 4(l/16)..+3 of column l%16).
        // Stage 2: 32x32 diagonal blocks: T_lo = T_bb A_lo T_aa for (a, b) = (0,1) and (2,3); wave q < 2 does block q.
        {
            const int c16 = lane & 15, g4 = lane >> 4;
            if (w < 2) {
                const int rA = 32 * w, rB = rA + 16;
                f32x4 x = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s4 = 0; s4 < 4; s4++)        // X = A_lo T_aa
                    x = __builtin_amdgcn_mfma_f32_16x16x4f32(As[(rB + c16) * LA + rA + 4 * s4 + g4], As[(rA + 4 * s4 + g4) * LA + rA + c16], x, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; i++) Xs[(16 * w + 4 * g4 + i) * 36 + c16] = x[i];
                __builtin_amdgcn_s_waitcnt(0xc07f);   // this wave's own X is in LDS (nobody else reads it)
                f32x4 y = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s4 = 0; s4 < 4; s4++)        // T_lo = T_bb X
                    y = __builtin_amdgcn_mfma_f32_16x16x4f32(As[(rB + c16) * LA + rB + 4 * s4 + g4], Xs[(16 * w + 4 * s4 + g4) * 36 + c16], y, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; i++) As[(rB + 4 * g4 + i) * LA + rA + c16] = y[i];
            }
        }
        lds_barrier();
        // Stage 3: the 64x64 matrix: T_lo = T_11 A_lo T_00 with 32x32 blocks; wave w < 4 does the 16x16 tile (w>>1, w&1) of both products
        {
            const int c16 = lane & 15, g4 = lane >> 4;
            const int ti = 16 * ((w >> 1) & 1), tj = 16 * (w & 1);
            f32x4 y = {0.f, 0.f, 0.f, 0.f};
            if (w < 4) {
                f32x4 x = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s4 = 0; s4 < 8; s4++)            // X = A_lo T_00
                    x = __builtin_amdgcn_mfma_f32_16x16x4f32(As[(32 + ti + c16) * LA + 4 * s4 + g4], As[(4 * s4 + g4) * LA + tj + c16], x, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < 4; i++) Xs[(ti + 4 * g4 + i) * 36 + tj + c16] = x[i];
            }
            lds_barrier();
            if (w < 4) {
#pragma unroll
                for (int s4 = 0; s4 < 8; s4++)            // T_lo = T_11 X
                    y = __builtin_amdgcn_mfma_f32_16x16x4f32(As[(32 + ti + c16) * LA + 32 + 4 * s4 + g4], Xs[(4 * s4 + g4) * 36 + tj + c16], y, 0, 0, 0);
            }
            lds_barrier();   // every read of the A_lo block is done
            if (w < 4) {
#pragma unroll
                for (int i = 0; i < 4; i++) As[(32 + ti + 4 * g4 + i) * LA + tj + c16] = y[i];
            }
        }
        lds_barrier();
        GT_CLK(g3);
        // ---- Tu = T diag(beta), Tw = -T diag(beta e^G) (bf16).  thread: row tid/8, 8 columns
        {
            const int i = tid >> 3, jb = (tid & 7) * 8;
#pragma unroll
            for (int j4 = 0; j4 < 2; j4++) {
                const float4 t = *(const float4*)(As + i * LA + jb + 4 * j4);
                const float tv[4] = {t.x, t.y, t.z, t.w};
                bf16x4 u, ww;
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int j = jb + 4 * j4 + jj;
                    const float tb = tv[jj] * Bs[j];
                    u[jj] = (__bf16)tb;
                    ww[jj] = (__bf16)(-tb * __expf(Gs[j]));
                }
                *(bf16x4*)(Tu + i * LT + jb + 4 * j4) = u;
                *(bf16x4*)(Tw + i * LT + jb + 4 * j4) = ww;
            }
        }
        lds_barrier();
        GT_CLK(g4);

        // ---- (c) U^T[v][i] = sum_j V[j][v] Tu[i][j] (waves wh = 0, kept in registers) and -W^T[d][i] = sum_j K[j][d] Tw[i][j]
        // (waves wh = 1, written to LDS); wave: rows 32wq.. of v / d, both token tiles
        f32x16 acc[2];      // wh = 0: U^T, later V'^T; wh = 1: -W^T, later (Q S)^T.  Tile it = token columns 32 it..
        acc[0] = zero16();
        acc[1] = zero16();
        {
            const __bf16* lhs = wh ? Ks : Vs;
            const __bf16* rhs = wh ? Tw : Tu;
#pragma unroll
            for (int s = 0; s < C / 16; s++) {
                const bf16x8 a = frag_tr(lhs, LD, 16 * s, 32 * wq, lane);
#pragma unroll
                for (int it = 0; it < 2; it++) acc[it] = mfma(a, frag_nt(rhs, LT, 32 * it, 16 * s, lane), acc[it]);
            }
            if (wh) {
#pragma unroll
                for (int it = 0; it < 2; it++)
#pragma unroll
                    for (int r4 = 0; r4 < 4; r4++) {
                        bf16x4 t;
#pragma unroll
                        for (int j = 0; j < 4; j++) t[j] = (__bf16)acc[it][4 * r4 + j];
                        *(bf16x4*)(Wn + (32 * it + n32) * LD + 32 * wq + 8 * r4 + 4 * g) = t;
                    }
                acc[0] = zero16();
                acc[1] = zero16();
            }
        }
        lds_barrier();   // -W visible; V (Vs) and T (As) are dead from here
        GT_CLK(g5);

        // ---- (d) wh = 0: V'^T = U^T + S^T (-W)^T;  (e1) wh = 1: QS^T[v][i] = sum_k S^T[v][k] Q[i][k]
        {
            const __bf16* rhs = wh ? Qs : Wn;
#pragma unroll
            for (int s = 0; s < KD / 16; s++) {
                const bf16x8 a = frag_nt(St, LD, 32 * wq, 16 * s, lane);
#pragma unroll
                for (int it = 0; it < 2; it++) acc[it] = mfma(a, frag_nt(rhs, LD, 32 * it, 16 * s, lane), acc[it]);
            }
        }
        // V' and V' e^{G_L - G_i}, row-major [i][v], bf16
        if (wh == 0) {
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int i = 32 * it + n32;
                const float dec = __expf(GL - Gs[i]);
#pragma unroll
                for (int r4 = 0; r4 < 4; r4++) {
                    bf16x4 t, td;
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        t[j] = (__bf16)acc[it][4 * r4 + j];
                        td[j] = (__bf16)(acc[it][4 * r4 + j] * dec);
                    }
                    *(bf16x4*)(Vs + i * LD + 32 * wq + 8 * r4 + 4 * g) = t;
                    *(bf16x4*)(Vd + i * LD + 32 * wq + 8 * r4 + 4 * g) = td;
                }
            }
        }
        lds_barrier();
        GT_CLK(g6);

        // ---- (e2) wh = 1: O^T[v][i] = s e^{G_i} QS^T + sum_j V'[j][v] P[i][j]
        if (wh) {
            f32x16 ov[2];
            ov[0] = zero16(); ov[1] = zero16();
#pragma unroll
            for (int s = 0; s < C / 16; s++) {
                const bf16x8 a = frag_tr(Vs, LD, 16 * s, 32 * wq, lane);
#pragma unroll
                for (int it = 0; it < 2; it++) ov[it] = mfma(a, frag_nt(Pm, LT, 32 * it, 16 * s, lane), ov[it]);
            }
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int i = 32 * it + n32;
                if (i < L) {
                    const float sc = p.scale * __expf(Gs[i]);
                    __bf16* op = p.o + Rs[i] * p.o_tok + (long)hv * VD + 32 * wq + 4 * g;
#pragma unroll
                    for (int r4 = 0; r4 < 4; r4++) {
                        bf16x4 t;
#pragma unroll
                        for (int j = 0; j < 4; j++) t[j] = (__bf16)(__builtin_fmaf(sc, acc[it][4 * r4 + j], ov[it][4 * r4 + j]));
                        *(bf16x4*)(op + 8 * r4) = t;
                    }
                }
            }
        }
        GT_CLK(g7);

        // ---- (f) S[k][v] = e^{G_L} S[k][v] + sum_j K[j][k] (V' e^{G_L - G_j})[j][v]; wave: k rows 32wq.., v tiles 2wh, 2wh + 1
        {
            const float eg = __expf(GL);
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) S[j][r] *= eg;
#pragma unroll
            for (int s = 0; s < C / 16; s++) {
                const bf16x8 a = frag_tr(Ks, LD, 16 * s, 32 * wq, lane);
#pragma unroll
                for (int j = 0; j < 2; j++) S[j] = mfma(a, frag_tr(Vd, LD, 16 * s, 64 * wh + 32 * j, lane), S[j]);
            }
        }
        lds_barrier();   // every wave is done reading S^T (d, e1) before it is replaced
        mirror();
        GT_CLK(g8);
        GT_ADD(0, g1 - g0); GT_ADD(1, g2 - g1); GT_ADD(2, g3 - g2); GT_ADD(3, g4 - g3); GT_ADD(4, g5 - g4); GT_ADD(5, g6 - g5); GT_ADD(6, g7 - g6); GT_ADD(7, g8 - g7); GT_ADD(8, 1);
    }

    if (p.ht != nullptr && p.ht_idx != nullptr) {
        const long dst = p.ht_idx[seg];
        if (dst >= 0) {
            float* hp = p.ht + (dst * p.hv + hv) * (long)KD * VD;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) hp[(long)(32 * wq + 8 * (r >> 2) + 4 * g + (r & 3)) * VD + 64 * wh + 32 * j + n32] = S[j][r];
        }
    }
}

int gdn_chunked_launch(const GdnParams& p, long max_len, hipStream_t stream) {
    (void)max_len;
    if (p.dv != VD) return spinf_fail(SPINF_E_ARG, "gdn chunked: value head dim %d, only 128 is built", p.dv);
    if (p.v_tok % 8 || p.o_tok % 4) return spinf_fail(SPINF_E_ARG, "gdn chunked: v row stride must be a multiple of 8, o of 4 elements");
    static bool configured = false;
    if (!configured) {
        hipError_t e = hipFuncSetAttribute((const void*)gdn_chunk_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LDS_BYTES);
        if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn chunked: hipFuncSetAttribute: %s", hipGetErrorString(e));
        configured = true;
    }
    const long blocks = p.n_seg * p.hv;
    if (blocks > INT32_MAX) return spinf_fail(SPINF_E_ARG, "gdn chunked: too many segments");
    hipLaunchKernelGGL(gdn_chunk_kernel, dim3((unsigned)blocks), dim3(512), LDS_BYTES, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn chunked: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}
