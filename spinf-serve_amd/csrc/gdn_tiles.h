// Shared pieces of the two Gated DeltaNet kernels (gdn.hip: short segments, gdn_chunk.hip: long segments): the launch
// parameters and the 16x16 MFMA tile helpers.
//
// Both kernels keep the state slice of a wave in fp32 accumulator layout (lane = value column, 4 consecutive key rows per
// 16x16 tile) and use it in place as the B operand of v_mfma_f32_16x16x32_bf16: two tiles side by side supply the 8
// contraction slots of a lane, slot (lane/16, j) = row 4 (lane/16) + j of the first tile for j < 4 and of the second for
// j >= 4.  The other operand is read in the same permuted order, so the state never moves, it is only rounded to bf16 on
// the way into the matrix core.  The same holds for every intermediate that one product leaves in accumulator layout and the
// next one contracts over (tokens for V' and P^T, key columns for W^T).
#pragma once
#include <hip/hip_runtime.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

struct GdnParams {
    const __bf16* q; const __bf16* k; const __bf16* v; const float* g; const __bf16* beta; __bf16* o;
    long q_tok, v_tok, g_tok, o_tok;
    int h, hv, dk, dv; float scale;
    const long* cu; const long* idx; long n_seg;
    const float* h0; const long* h0_idx; float* ht; const long* ht_idx;
    int run;   // segments per workgroup of the recurrent entry point's kernel (set by its launcher)
};

namespace gdn_tiles {

// C[m][n] += sum_k A[m][k] B[k][n], 16 x 16 x 32: lane l gives A[l%16][8 (l/16) ..+7] and B[8 (l/16) ..+7][l%16] and holds
// C[4 (l/16) ..+3][l%16].
__device__ __forceinline__ f32x4 mfma32(bf16x8 a, bf16x8 b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
// 16 x 16 x 16: 4 contraction slots per lane, 4 (l/16) ..+3.
__device__ __forceinline__ f32x4 mfma16(bf16x4 a, bf16x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
}
// fp32 16 x 16 x 4: lane l gives A[l%16][l/16] and B[l/16][l%16].
__device__ __forceinline__ f32x4 mfma4(float a, float b, f32x4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }

// Operand whose contraction index is the ROW index of a row-major bf16 LDS tile: the lane gets column col0 + lane%16 of
// rows row0 + 4 (lane/16) .. +3 (each group of 16 lanes transposes a 4 x 16 block).
__device__ __forceinline__ bf16x4 frag_tr4(const __bf16* base, int stride, int row0, int col0, int lane) {
    const int t = lane & 15;
    const __bf16* p = base + (row0 + 4 * (lane >> 4) + (t >> 2)) * stride + col0 + 4 * (t & 3);
    return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)p));
}
__device__ __forceinline__ bf16x8 join(bf16x4 lo, bf16x4 hi) { return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7); }
__device__ __forceinline__ bf16x4 round4(f32x4 x) {
    bf16x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = (__bf16)x[i];
    return r;
}
__device__ __forceinline__ f32x4 zero4() { return f32x4{0.f, 0.f, 0.f, 0.f}; }
// Inclusive prefix sum inside every row of 16 lanes (zero shifted in).
__device__ __forceinline__ float row_prefix_sum(float x) {
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x111, 0xf, 0xf, true));   // row_shr:1
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x112, 0xf, 0xf, true));   // row_shr:2
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x114, 0xf, 0xf, true));   // row_shr:4
    x += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x118, 0xf, 0xf, true));   // row_shr:8
    return x;
}
// Row c of (I - A)^-1 for a strictly lower triangular 16 x 16 block A (row stride lda floats, in LDS), c = this lane's row:
// T = I + T A, so t[j] = [j == c] + sum_{m > j} t[m] A[m][j]; the highest m goes first and every step updates all j < m.
// PRELOAD: read A's rows in two batches (rows 15..8, then 7..1) ahead of the steps that use them instead of row by row: the
// steps form a chain of 15 dependent multiply-adds, and an LDS round trip inside every link is what such a solve otherwise
// waits for.
template <bool PRELOAD>
__device__ __forceinline__ void unit_lower_inverse_row(const float* A, int lda, int c, float (&t)[16]) {
    f32x4 a[16][4];
#pragma unroll
    for (int j = 0; j < 16; j++) t[j] = (j == c) ? 1.f : 0.f;
#pragma unroll
    for (int half = 1; half >= 0; half--) {
        if (PRELOAD) {
#pragma unroll
            for (int m = 8 * half + 7; m >= 8 * half; m--)
#pragma unroll
                for (int j4 = 0; 4 * j4 < m; j4++) a[m][j4] = *(const f32x4*)(A + m * lda + 4 * j4);
            __builtin_amdgcn_sched_barrier(0);
        }
#pragma unroll
        for (int m = 8 * half + 7; m >= 8 * half; m--) {
#pragma unroll
            for (int j4 = 0; 4 * j4 < m; j4++) {
                const f32x4 am = PRELOAD ? a[m][j4] : *(const f32x4*)(A + m * lda + 4 * j4);
#pragma unroll
                for (int jj = 0; jj < 4; jj++)
                    if (4 * j4 + jj < m) t[4 * j4 + jj] = __builtin_fmaf(t[m], am[jj], t[4 * j4 + jj]);
            }
        }
        if (PRELOAD) __builtin_amdgcn_sched_barrier(0);
    }
}
// t[4 q + r], r = 0..3, without indexing registers by a lane-dependent value
__device__ __forceinline__ f32x4 pick4(const float (&t)[16], int q) {
    f32x4 r;
#pragma unroll
    for (int i = 0; i < 4; i++) r[i] = q == 0 ? t[i] : q == 1 ? t[4 + i] : q == 2 ? t[8 + i] : t[12 + i];
    return r;
}
// Orders a wave's LDS writes before its later LDS reads for the compiler; the hardware runs one wave's LDS operations in order.
__device__ __forceinline__ void wave_lds_order() { asm volatile("" ::: "memory"); }
// Workgroup barrier for LDS traffic only: waits for this wave's LDS operations, not for its global loads (__syncthreads()
// carries a fence in front of which the compiler drains every load in flight, prefetches included).
__device__ __forceinline__ void lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

}  // namespace gdn_tiles
