// The lm head's read-out after the logits GEMM, for gfx950 (MI355X): final soft-capping and log-softmax over the vocabulary, and
// the selection of the option columns, in one pass over the logits (spinf_serve/scorer.py:340-355 followed by the column
// selection of scorer.py:254).  The reference writes the capped logits and the full log-probs (two more vocabulary-sized
// matrices per 1,024 read rows) and then keeps a handful of columns; here a row's logits are read once, its log-sum-exp is
// kept in registers, and only the selected columns are written (or, for the extraction rows, the full row in a second pass).
//
// Bound: HBM (4 bytes read per logit; ~12 vector ALU operations per logit stay far below that).  One workgroup per row: 256
// lanes x 16-byte loads, a running (maximum, sum) pair per lane merged across the workgroup at the end of the row.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

namespace {

struct LmParams {
    const void* logits; long ld;      // [rows, >= vocab], row stride in elements
    const long* cols; int n_cols;     // selected columns (NULL: every column)
    float* out; long out_ld;
    int rows, vocab;
    float cap, inv_cap;               // soft-capping (0: none)
};

constexpr float LOG2E = 1.4426950408889634f;

// cap * tanh(x / cap) through the hardware exp2: tanh(y) = 1 - 2 / (e^(2y) + 1)
__device__ __forceinline__ float softcap(float x, float cap, float inv_cap) {
    if (cap == 0.f) return x;
    const float e = __builtin_amdgcn_exp2f(2.0f * LOG2E * x * inv_cap);
    return cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
}

// (m, s): reference point so far and sum of exp(x - m); folding in N more values (one exponential per value, one per call)
template <int N>
__device__ __forceinline__ void fold(float& m, float& s, const float (&x)[N]) {
    float mn = m;
#pragma unroll
    for (int j = 0; j < N; j++) mn = fmaxf(mn, x[j]);
    float acc = m == -INFINITY ? 0.f : s * __builtin_amdgcn_exp2f((m - mn) * LOG2E);
#pragma unroll
    for (int j = 0; j < N; j++) acc += __builtin_amdgcn_exp2f((x[j] - mn) * LOG2E);
    s = acc;
    m = mn;
}
__device__ __forceinline__ void merge(float& m, float& s, float m2, float s2) {
    const float mn = fmaxf(m, m2);
    s = s * __builtin_amdgcn_exp2f((m - mn) * LOG2E) + s2 * __builtin_amdgcn_exp2f((m2 - mn) * LOG2E);
    m = mn;
}

template <bool BF16>
__device__ __forceinline__ float load1(const void* base, long i) {
    return BF16 ? (float)((const __bf16*)base)[i] : ((const float*)base)[i];
}

template <bool BF16>
__global__ __launch_bounds__(256) void lm_logprobs_kernel(const LmParams p) {
    constexpr int VEC = BF16 ? 8 : 4;           // elements per 16-byte load
    __shared__ float red_m[4], red_s[4];
    const int row = blockIdx.x;
    const char* base = (const char*)p.logits + (long)row * p.ld * (BF16 ? 2 : 4);
    // with soft-capping every value lies in [-cap, cap]: the reference point is cap itself and no maximum is tracked
    // (exp(-2 cap) is far inside fp32 range for any cap a model uses; the host checks cap <= 40)
    float m = p.cap > 0.f ? p.cap : -INFINITY, s = 0.f;
    const int n_vec = p.vocab / VEC;
    constexpr int UNR = 4;                      // 16-byte loads in flight per lane
    for (int i0 = threadIdx.x; i0 < n_vec; i0 += 256 * UNR) {
        float x[UNR][VEC];
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            const int i = i0 + u * 256 < n_vec ? i0 + u * 256 : i0;   // past the end: the first one again, not folded below
            if (BF16) {
                const bf16x8 v = *(const bf16x8*)(base + (long)i * 16);
#pragma unroll
                for (int j = 0; j < VEC; j++) x[u][j] = (float)v[j];
            } else {
                const float4 v = *(const float4*)(base + (long)i * 16);
                x[u][0] = v.x; x[u][1] = v.y; x[u][2] = v.z; x[u][3] = v.w;
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; u++) {
            if (i0 + u * 256 >= n_vec) break;
#pragma unroll
            for (int j = 0; j < VEC; j++) x[u][j] = softcap(x[u][j], p.cap, p.inv_cap);
            fold<VEC>(m, s, x[u]);
        }
    }
    for (int i = n_vec * VEC + threadIdx.x; i < p.vocab; i += 256) {
        const float x1[1] = {softcap(load1<BF16>(base, i), p.cap, p.inv_cap)};
        fold<1>(m, s, x1);
    }
    // across the wave, then across the four waves
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const float m2 = __shfl_xor(m, d), s2 = __shfl_xor(s, d);
        if (m2 != -INFINITY) {
            if (m == -INFINITY) { m = m2; s = s2; } else merge(m, s, m2, s2);
        }
    }
    if ((threadIdx.x & 63) == 0) { red_m[threadIdx.x >> 6] = m; red_s[threadIdx.x >> 6] = s; }
    __syncthreads();
    m = red_m[0]; s = red_s[0];
#pragma unroll
    for (int w = 1; w < 4; w++)
        if (red_m[w] != -INFINITY) {
            if (m == -INFINITY) { m = red_m[w]; s = red_s[w]; } else merge(m, s, red_m[w], red_s[w]);
        }
    const float lse = m + logf(s);
    float* out = p.out + (long)row * p.out_ld;
    if (p.cols) {
        for (int c = threadIdx.x; c < p.n_cols; c += 256) {   // a column outside the vocabulary is not read: NaN
            const long col = p.cols[c];
            out[c] = col >= 0 && col < p.vocab ? softcap(load1<BF16>(base, col), p.cap, p.inv_cap) - lse : __builtin_nanf("");
        }
    } else {
        for (int i = threadIdx.x; i < p.vocab; i += 256) out[i] = softcap(load1<BF16>(base, i), p.cap, p.inv_cap) - lse;
    }
}

}  // namespace

extern "C" int spinf_lm_logprobs(const spinf_lm_args* a, void* stream) {
    if (!a) return spinf_fail(SPINF_E_ARG, "lm_logprobs: null args");
    if (a->rows <= 0) return SPINF_OK;
    if (!a->logits || !a->out) return spinf_fail(SPINF_E_ARG, "lm_logprobs: null pointer");
    if (a->vocab <= 0 || a->vocab > (1 << 30) || a->rows > (1 << 30)) return spinf_fail(SPINF_E_ARG, "lm_logprobs: %lld rows x %lld columns out of range", (long long)a->rows, (long long)a->vocab);
    if (a->dtype != 0 && a->dtype != 1) return spinf_fail(SPINF_E_ARG, "lm_logprobs: dtype %d (0 = fp32, 1 = bf16)", a->dtype);
    const int vec = a->dtype ? 8 : 4;
    if (a->ld < a->vocab || a->ld % vec || (uintptr_t)a->logits % 16) return spinf_fail(SPINF_E_ARG, "lm_logprobs: rows must be 16-byte aligned and hold the vocabulary");
    if ((a->cols == nullptr) != (a->n_cols == 0) || a->n_cols < 0) return spinf_fail(SPINF_E_ARG, "lm_logprobs: cols and n_cols come together");
    if (a->out_ld < (a->cols ? a->n_cols : a->vocab)) return spinf_fail(SPINF_E_ARG, "lm_logprobs: output rows too short");
    if (a->softcap < 0.f || a->softcap > 40.f) return spinf_fail(SPINF_E_ARG, "lm_logprobs: softcap %g outside 0 .. 40", (double)a->softcap);
    LmParams p;
    p.logits = a->logits; p.ld = a->ld; p.cols = a->cols; p.n_cols = (int)a->n_cols; p.out = a->out; p.out_ld = a->out_ld;
    p.rows = (int)a->rows; p.vocab = (int)a->vocab; p.cap = a->softcap; p.inv_cap = a->softcap > 0.f ? 1.0f / a->softcap : 0.f;
    if (a->dtype) hipLaunchKernelGGL(lm_logprobs_kernel<true>, dim3(p.rows), dim3(256), 0, (hipStream_t)stream, p);
    else hipLaunchKernelGGL(lm_logprobs_kernel<false>, dim3(p.rows), dim3(256), 0, (hipStream_t)stream, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "lm_logprobs: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}
