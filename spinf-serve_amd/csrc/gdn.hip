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

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

struct GdnParams {
    const __bf16* q; const __bf16* k; const __bf16* v; const float* g; const __bf16* beta; __bf16* o;
    long q_tok, v_tok, g_tok, o_tok;
    int h, hv, dk, dv; float scale;
    const long* cu; const long* idx; long n_seg;
    const float* h0; const long* h0_idx; float* ht; const long* ht_idx;
};

// ---------------------------------------------------------------------------------------------- token by token
// One wave per (segment, value head, 32 values): lane (v = lane%32, half = lane/32) keeps rows 64 half .. 64 half + 63
// of column v of the state in registers.  Meant for the short segments of a trie (a handful of tokens after a fork).
__global__ __launch_bounds__(64) void gdn_recurrent_kernel(const GdnParams p) {
    constexpr int K = 128;
    const int nvb = p.dv / 32;
    const long b = blockIdx.x;
    const int iv = (int)(b % nvb);
    const long nh = b / nvb;
    const long n = nh / p.hv;
    const int hv = (int)(nh % p.hv);
    const int hk = hv / (p.hv / p.h);
    const int lane = threadIdx.x, vv = iv * 32 + (lane & 31), half = lane >> 5;
    float S[64];
#pragma unroll
    for (int i = 0; i < 64; i++) S[i] = 0.f;
    if (p.h0 != nullptr && p.h0_idx != nullptr) {
        const long src = p.h0_idx[n];
        if (src >= 0) {
            const float* hp = p.h0 + ((src * p.hv + hv) * K + 64 * half) * p.dv + vv;
#pragma unroll
            for (int i = 0; i < 64; i++) S[i] = hp[(long)i * p.dv];
        }
    }
    const long bos = p.cu[n], eos = p.cu[n + 1];
    for (long t = bos; t < eos; t++) {
        const long r = p.idx ? p.idx[t] : t;
        const __bf16* kp = p.k + r * p.q_tok + (long)hk * K + 64 * half;
        const __bf16* qp = p.q + r * p.q_tok + (long)hk * K + 64 * half;
        bf16x8 kr[8], qr[8];
#pragma unroll
        for (int c = 0; c < 8; c++) {
            kr[c] = *(const bf16x8*)(kp + 8 * c);
            qr[c] = *(const bf16x8*)(qp + 8 * c);
        }
        const float vt = (float)p.v[r * p.v_tok + (long)hv * p.dv + vv];
        const float gt = p.g[r * p.g_tok + hv];
        const float bt = (float)p.beta[r * p.g_tok + hv];
        const float eg = __expf(gt);
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < 64; i++) {
            S[i] *= eg;
            dot = __builtin_fmaf(S[i], (float)kr[i >> 3][i & 7], dot);
        }
        dot += __shfl_xor(dot, 32);
        const float dl = (vt - dot) * bt;
        float od = 0.f;
#pragma unroll
        for (int i = 0; i < 64; i++) {
            S[i] = __builtin_fmaf((float)kr[i >> 3][i & 7], dl, S[i]);
            od = __builtin_fmaf(S[i], (float)qr[i >> 3][i & 7] * p.scale, od);
        }
        od += __shfl_xor(od, 32);
        if (half == 0) p.o[r * p.o_tok + (long)hv * p.dv + vv] = (__bf16)od;
    }
    if (p.ht != nullptr && p.ht_idx != nullptr) {
        const long dst = p.ht_idx[n];
        if (dst >= 0) {
            float* hp = p.ht + ((dst * p.hv + hv) * K + 64 * half) * p.dv + vv;
#pragma unroll
            for (int i = 0; i < 64; i++) hp[(long)i * p.dv] = S[i];
        }
    }
}

int gdn_chunked_launch(const GdnParams& p, long max_len, hipStream_t stream);   // gdn_chunk.hip

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
    GdnParams p;
    p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v; p.g = a->g; p.beta = (const __bf16*)a->beta;
    p.o = (__bf16*)a->o;
    p.q_tok = a->q_tok; p.v_tok = a->v_tok; p.g_tok = a->g_tok; p.o_tok = a->o_tok;
    p.h = a->h; p.hv = a->hv; p.dk = a->dk; p.dv = a->dv; p.scale = a->scale;
    p.cu = (const long*)a->cu; p.idx = (const long*)a->idx; p.n_seg = a->n_seg;
    p.h0 = a->h0; p.h0_idx = (const long*)a->h0_idx; p.ht = a->ht; p.ht_idx = (const long*)a->ht_idx;
    hipStream_t s = (hipStream_t)stream;
    if (a->mode == 1) return gdn_chunked_launch(p, a->max_len, s);
    if (a->mode != 0) return spinf_fail(SPINF_E_ARG, "gdn: unknown mode %d", a->mode);
    const long blocks = a->n_seg * a->hv * (a->dv / 32);
    if (blocks > INT32_MAX) return spinf_fail(SPINF_E_ARG, "gdn: too many segments");
    hipLaunchKernelGGL(gdn_recurrent_kernel, dim3((unsigned)blocks), dim3(64), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}
