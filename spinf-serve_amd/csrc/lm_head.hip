// The lm head over the read rows, for gfx950 (MI355X): row gather, logits GEMM, final soft-capping, log-softmax over the
// vocabulary and column selection in one pass (spinf_serve/scorer.py:247-261 and :340-355).  The reference gathers h[sel],
// multiplies 1,024 rows at a time by W^T into a [1024, vocab] logits matrix (1 GiB in fp32 at a 262k vocabulary), writes the
// capped logits and the log-probs (two more such matrices) and keeps a handful of columns.  Here the logits exist only as
// 128 x 128 tiles in LDS: a tile's contribution to its rows' log-sum-exp and the selected columns leave it, nothing else.
//
// Kernel 1 (lm_head_tile_kernel): a workgroup of four waves computes L^T = W h^T for 128 vocabulary rows x 128 read rows with
// v_mfma_f32_32x32x16_bf16 (W and the gathered h rows staged through LDS, 64 hidden dims per step, double buffered), caps the tile,
// leaves it in LDS, and writes per read row two (reference, sum of exponentials) pairs (one per 64 vocabulary rows) and the
// selected columns' capped logits (or, for the extraction rows, the whole tile).
// Kernel 2 (lm_head_finish_kernel): per read row, the pairs are merged into the log-sum-exp, which is subtracted in place.
//
// A read row's numbers depend on nothing but that row and W: every logit is one dot product accumulated in the fixed order of the
// hidden dimension, whatever rows share its tile, and the pairs are merged in a fixed order.  That is the property the reference
// pads its last chunk to 1,024 rows for (lm_fixed_rows, spinf_serve/config.py:56-57).
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

namespace {

constexpr int TV = 128, TR = 128, BK = 64;      // tile: vocabulary rows, read rows, hidden dims per step
constexpr int PITCH = BK * 2 + 16;              // bytes of a staged row (padded: the fragment reads of 32 rows spread over the banks)
constexpr int STAGE = (TV + TR) * PITCH;        // one buffer: W rows then h rows
constexpr int LPITCH = TR + 1;                  // floats of a logits-tile row in LDS ([vocabulary][read row])
constexpr float LOG2E = 1.4426950408889634f;

struct HeadParams {
    const __bf16* h; long h_ld;
    const long* sel; int rows;
    const __bf16* w; long w_ld;
    int vocab, hidden;
    float cap, inv_cap;
    const long* cols; int n_cols;
    float* out; long out_ld;
    float2* part; int n_part;   // [rows, n_part] pairs; n_part = 2 * vocabulary tiles
};

__device__ __forceinline__ float to_bf16(float x) { return (float)(__bf16)x; }

// cap * tanh(x / cap) through the hardware exp2: tanh(y) = 1 - 2 / (e^(2y) + 1).  BF16: every step rounded to bf16, as the
// reference's bf16 logits go through torch.tanh(logits / cap) * cap
template <bool BF16>
__device__ __forceinline__ float softcap(float x, float cap, float inv_cap) {
    if (BF16) {
        const float y = to_bf16(x / cap);
        const float e = __builtin_amdgcn_exp2f(2.0f * LOG2E * y);
        const float t = to_bf16(1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
        return to_bf16(t * cap);
    }
    const float e = __builtin_amdgcn_exp2f(2.0f * LOG2E * x * inv_cap);
    return cap * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
}

template <bool CAPPED, bool BF16>
__global__ __launch_bounds__(256) void lm_head_tile_kernel(const HeadParams p) {
    static_assert(TV * LPITCH * 4 <= 2 * STAGE, "the logits tile reuses the staging buffers");
    __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, g = lane >> 5;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6), wv = w & 1, wr = w >> 1;
    const int r0 = blockIdx.x * TR, v0 = blockIdx.y * TV;   // read-row tiles fastest: the tiles that share W rows run together

    // ---- loader: a staged tile row is 64 hidden dims = 8 chunks of 16 bytes; thread t copies chunks t, t + 256, ... of W and of h
    const __bf16* src_w[4];
    const __bf16* src_h[4];
    int dst[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int c = tid + 256 * i, row = c >> 3, kc = c & 7;
        const int vr = v0 + row < p.vocab ? v0 + row : p.vocab - 1;
        int rr = r0 + row < p.rows ? r0 + row : p.rows - 1;
        const long hr = p.sel ? p.sel[rr] : (long)rr;
        src_w[i] = p.w + (long)vr * p.w_ld + kc * 8;
        src_h[i] = p.h + hr * p.h_ld + kc * 8;
        dst[i] = row * PITCH + kc * 16;
    }
    bf16x8 rw[4], rh[4];
    auto fetch = [&](const int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            rw[i] = *(const bf16x8*)(src_w[i] + k0);
            rh[i] = *(const bf16x8*)(src_h[i] + k0);
        }
    };
    auto stash = [&](char* buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *(bf16x8*)(buf + dst[i]) = rw[i];
            *(bf16x8*)(buf + TV * PITCH + dst[i]) = rh[i];
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

    const int nk = p.hidden / BK;
    fetch(0);
    stash(lds);
    __syncthreads();
    for (int kt = 0; kt < nk; kt++) {
        const char* buf = lds + (kt & 1) * STAGE;
        if (kt + 1 < nk) fetch((kt + 1) * BK);
        const char* fa = buf + (wv * 64 + m) * PITCH + 16 * g;
        const char* fb = buf + (TV + wr * 64 + m) * PITCH + 16 * g;
#pragma unroll
        for (int ks = 0; ks < BK / 16; ks++) {
            bf16x8 av[2], bv[2];
#pragma unroll
            for (int a = 0; a < 2; a++) av[a] = *(const bf16x8*)(fa + 32 * a * PITCH + 32 * ks);
#pragma unroll
            for (int b = 0; b < 2; b++) bv[b] = *(const bf16x8*)(fb + 32 * b * PITCH + 32 * ks);
#pragma unroll
            for (int a = 0; a < 2; a++)
#pragma unroll
                for (int b = 0; b < 2; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[a], bv[b], acc[a][b], 0, 0, 0);
        }
        if (kt + 1 < nk) {
            stash(lds + ((kt + 1) & 1) * STAGE);
            __syncthreads();
        }
    }
    __syncthreads();   // everyone is done with the staging buffers: the logits tile goes there

    // ---- the capped logits tile in LDS, [vocabulary row][read row].  Register i of a 32 x 32 block holds vocabulary row
    // 8 (i / 4) + 4 g + i % 4 of the block for read row m.
    float* tile = (float*)lds;
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
        for (int b = 0; b < 2; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float x = acc[a][b][i];
                if (BF16) x = to_bf16(x);
                if (CAPPED) x = softcap<BF16>(x, p.cap, p.inv_cap);
                tile[(wv * 64 + 32 * a + 8 * (i >> 2) + 4 * g + (i & 3)) * LPITCH + wr * 64 + 32 * b + m] = x;
            }
    __syncthreads();

    // ---- per read row, two (reference, sum) pairs: thread t takes read row t % 128 and vocabulary rows 64 (t / 128) .. + 63
    {
        const int row = tid & (TR - 1), half = tid >> 7;
        const int nv = p.vocab - (v0 + 64 * half) < 64 ? p.vocab - (v0 + 64 * half) : 64;   // rows of the vocabulary that exist
        const float* col = tile + 64 * half * LPITCH + row;
        float ref = CAPPED ? p.cap : -INFINITY, sum = 0.f;
        if (!CAPPED)
            for (int j = 0; j < nv; j++) ref = fmaxf(ref, col[j * LPITCH]);
        for (int j = 0; j < nv; j++) sum += __builtin_amdgcn_exp2f((col[j * LPITCH] - ref) * LOG2E);
        if (r0 + row < p.rows) p.part[(long)(r0 + row) * p.n_part + 2 * blockIdx.y + half] = make_float2(ref, sum);
    }
    // ---- what leaves the tile
    if (p.cols) {   // the selected columns: wave w looks at columns w, w + 4, ...
        for (int c = w; c < p.n_cols; c += 4) {
            const long col = p.cols[c];
            if (col < v0 || col >= v0 + TV) continue;
            for (int row = lane; row < TR; row += 64)
                if (r0 + row < p.rows) p.out[(long)(r0 + row) * p.out_ld + c] = tile[(col - v0) * LPITCH + row];
        }
    } else {        // the extraction rows: the whole tile, a read row's 128 values as two runs of 64
        for (int row = w; row < TR; row += 4) {
            if (r0 + row >= p.rows) break;
            for (int v = lane; v < TV; v += 64)
                if (v0 + v < p.vocab) p.out[(long)(r0 + row) * p.out_ld + v0 + v] = tile[v * LPITCH + row];
        }
    }
}

// per read row: merge the pairs in their fixed order, subtract the log-sum-exp
__global__ __launch_bounds__(256) void lm_head_finish_kernel(const HeadParams p) {
    __shared__ float red_m[4], red_s[4];
    const int row = blockIdx.x;
    const float2* part = p.part + (long)row * p.n_part;
    float m = -INFINITY, s = 0.f;
    for (int i = threadIdx.x; i < p.n_part; i += 256) {
        const float2 q = part[i];
        if (q.y <= 0.f) continue;   // a half tile past the end of the vocabulary
        const float mn = fmaxf(m, q.x);
        s = (m == -INFINITY ? 0.f : s * __builtin_amdgcn_exp2f((m - mn) * LOG2E)) + q.y * __builtin_amdgcn_exp2f((q.x - mn) * LOG2E);
        m = mn;
    }
    auto merge = [&](const float m2, const float s2) {
        if (m2 == -INFINITY) return;
        const float mn = fmaxf(m, m2);
        s = (m == -INFINITY ? 0.f : s * __builtin_amdgcn_exp2f((m - mn) * LOG2E)) + s2 * __builtin_amdgcn_exp2f((m2 - mn) * LOG2E);
        m = mn;
    };
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) merge(__shfl_xor(m, d), __shfl_xor(s, d));
    if ((threadIdx.x & 63) == 0) { red_m[threadIdx.x >> 6] = m; red_s[threadIdx.x >> 6] = s; }
    __syncthreads();
    m = red_m[0]; s = red_s[0];
#pragma unroll
    for (int k = 1; k < 4; k++) merge(red_m[k], red_s[k]);
    const float lse = m + logf(s);
    float* out = p.out + (long)row * p.out_ld;
    const int n = p.cols ? p.n_cols : p.vocab;
    for (int i = threadIdx.x; i < n; i += 256) {
        const bool known = !p.cols || (p.cols[i] >= 0 && p.cols[i] < p.vocab);   // no tile wrote a column outside the vocabulary
        out[i] = known ? out[i] - lse : __builtin_nanf("");
    }
}

int check(const spinf_lm_head_args* a) {
    if (!a) return spinf_fail(SPINF_E_ARG, "lm_head: null args");
    if (a->rows < 0 || a->rows > (1 << 24)) return spinf_fail(SPINF_E_ARG, "lm_head: %lld read rows out of range", (long long)a->rows);
    if (a->vocab <= 0 || a->vocab > (1 << 26)) return spinf_fail(SPINF_E_ARG, "lm_head: vocabulary %lld out of range", (long long)a->vocab);
    if (a->hidden <= 0 || a->hidden % BK) return spinf_fail(SPINF_E_ARG, "lm_head: hidden size %lld must be a multiple of %d", (long long)a->hidden, BK);
    if (a->softcap < 0.f || a->softcap > 40.f) return spinf_fail(SPINF_E_ARG, "lm_head: softcap %g outside 0 .. 40", (double)a->softcap);
    if (a->logits_dtype != 0 && a->logits_dtype != 1) return spinf_fail(SPINF_E_ARG, "lm_head: logits_dtype %d (0 = fp32, 1 = bf16)", a->logits_dtype);
    if ((a->cols == nullptr) != (a->n_cols == 0) || a->n_cols < 0) return spinf_fail(SPINF_E_ARG, "lm_head: cols and n_cols come together");
    return SPINF_OK;
}

int64_t parts_of(const spinf_lm_head_args* a) { return 2 * ((a->vocab + TV - 1) / TV); }

}  // namespace

extern "C" int spinf_lm_head_workspace(const spinf_lm_head_args* a, int64_t* bytes) {
    if (int rc = check(a)) return rc;
    if (!bytes) return spinf_fail(SPINF_E_ARG, "lm_head_workspace: null pointer");
    *bytes = a->rows * parts_of(a) * (int64_t)sizeof(float2);
    return SPINF_OK;
}

extern "C" int spinf_lm_head_fwd(const spinf_lm_head_args* a, void* stream) {
    if (int rc = check(a)) return rc;
    if (a->rows == 0) return SPINF_OK;
    if (!a->h || !a->w || !a->out || !a->workspace) return spinf_fail(SPINF_E_ARG, "lm_head: null pointer");
    if (a->h_ld < a->hidden || a->w_ld < a->hidden || a->h_ld % 8 || a->w_ld % 8 || (uintptr_t)a->h % 16 || (uintptr_t)a->w % 16)
        return spinf_fail(SPINF_E_ARG, "lm_head: h and W rows must hold the hidden size, with 16-byte aligned rows");
    if (a->out_ld < (a->cols ? a->n_cols : a->vocab)) return spinf_fail(SPINF_E_ARG, "lm_head: output rows too short");
    if (a->workspace_bytes < a->rows * parts_of(a) * (int64_t)sizeof(float2))
        return spinf_fail(SPINF_E_ARG, "lm_head: workspace of %lld bytes, %lld needed (spinf_lm_head_workspace)", (long long)a->workspace_bytes,
                          (long long)(a->rows * parts_of(a) * (int64_t)sizeof(float2)));
    HeadParams p;
    p.h = (const __bf16*)a->h; p.h_ld = a->h_ld; p.sel = a->sel; p.rows = (int)a->rows;
    p.w = (const __bf16*)a->w; p.w_ld = a->w_ld; p.vocab = (int)a->vocab; p.hidden = (int)a->hidden;
    p.cap = a->softcap; p.inv_cap = a->softcap > 0.f ? 1.0f / a->softcap : 0.f;
    p.cols = a->cols; p.n_cols = (int)a->n_cols; p.out = a->out; p.out_ld = a->out_ld;
    p.part = (float2*)a->workspace; p.n_part = (int)parts_of(a);
    const dim3 grid((unsigned)((a->rows + TR - 1) / TR), (unsigned)((a->vocab + TV - 1) / TV));
    hipStream_t s = (hipStream_t)stream;
    const bool capped = a->softcap > 0.f, bf = a->logits_dtype == 1;
    if (capped && bf) hipLaunchKernelGGL((lm_head_tile_kernel<true, true>), grid, dim3(256), 0, s, p);
    else if (capped) hipLaunchKernelGGL((lm_head_tile_kernel<true, false>), grid, dim3(256), 0, s, p);
    else if (bf) hipLaunchKernelGGL((lm_head_tile_kernel<false, true>), grid, dim3(256), 0, s, p);
    else hipLaunchKernelGGL((lm_head_tile_kernel<false, false>), grid, dim3(256), 0, s, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "lm_head: launch: %s", hipGetErrorString(e));
    hipLaunchKernelGGL(lm_head_finish_kernel, dim3((unsigned)a->rows), dim3(256), 0, s, p);
    e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "lm_head: launch (finish): %s", hipGetErrorString(e));
    return SPINF_OK;
}
