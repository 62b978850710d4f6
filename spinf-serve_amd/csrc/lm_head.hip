// The lm head over the read rows, for gfx950 (MI355X): row gather, logits GEMM, final soft-capping, log-softmax over the
// vocabulary and column selection in one pass (spinf_serve/scorer.py:247-261 and :340-355).  The reference gathers h[sel],
// multiplies 1,024 rows at a time by W^T into a [1024, vocab] logits matrix (1 GiB in fp32 at a 262k vocabulary), writes the
// capped logits and the log-probs (two more such matrices) and keeps a handful of columns.  Here the logits exist only in the
// accumulator registers of the GEMM: a tile's contribution to its rows' log-sum-exp and the selected columns leave it, nothing else.
//
// Kernel 1 (lm_head_tile_kernel): a workgroup of four waves, one per SIMD, computes L^T = W h^T for 256 vocabulary rows x 256 read
// rows with v_mfma_f32_32x32x16_bf16, each wave a 128 x 128 quarter (256 accumulator registers: with smaller wave tiles the
// fragment reads ask more of the LDS than it delivers).  W and the gathered h rows are staged through LDS, 64 hidden dims per
// step, double buffered.  The epilogue stays in registers: a lane owns one read row per 32 x 32 block, so the (reference, sum of
// exponentials) pair of a read row over the wave's 128 vocabulary rows is an in-lane reduction and one exchange with the other
// half of the wave; only blocks that hold a selected column (or, for the extraction rows, all blocks) pass through a small LDS
// tile to be written out.
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

constexpr int TV = 256, TR = 256, BK = 64;      // tile: vocabulary rows, read rows, hidden dims per step
constexpr int WT = 128;                         // a wave's quarter: 128 vocabulary rows x 128 read rows
constexpr int PITCH = BK * 2 + 16;              // bytes of a staged row (padded: the fragment reads of 32 rows spread over the banks)
constexpr int STAGE = (TV + TR) * PITCH;        // one buffer: W rows then h rows
constexpr int BP = 33;                          // floats of a row of a wave's 32 x 32 output block in LDS ([vocabulary][read row])
constexpr float LOG2E = 1.4426950408889634f;

struct HeadParams {
    const __bf16* h; long h_ld;
    const long* sel; int rows; long h_rows;
    const __bf16* w; long w_ld;
    int vocab, hidden;
    float cap, inv_cap;
    const long* cols; int n_cols;
    float* out; long out_ld;
    float2* part; int n_part;   // [rows, n_part] pairs; n_part = 2 * vocabulary tiles
    int row_tiles;
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
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void lm_head_tile_kernel(const HeadParams p) {
    __shared__ __attribute__((aligned(16))) char lds[2 * STAGE];
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, g = lane >> 5;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6), wv = w & 1, wr = w >> 1;
    // Workgroups go round the 8 XCDs (each with its own L2) in launch order.  The read-row tiles of one vocabulary tile share its
    // W rows, so they take consecutive launch slots of ONE XCD: W then comes from HBM once and from that L2 for the others (with
    // the tiles of a vocabulary tile spread over the XCDs every one of them fetched W from HBM: 4 x 1.3 GB at 1,024 read rows).
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int vtile = (slot / p.row_tiles) * 8 + xcd, rtile = slot % p.row_tiles;
    if (vtile * TV >= p.vocab) return;
    const int r0 = rtile * TR, v0 = vtile * TV;

    // ---- loader: a staged tile row is 64 hidden dims = 8 chunks of 16 bytes; thread t copies chunk t % 8 of rows t / 8 + 32 i
    const int kc = tid & 7;
    int row_h[8];   // this thread's rows of h (through the row list); its rows of W are v0 + t / 8 + 32 i, clamped to the vocabulary
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int row = (tid >> 3) + 32 * i;
        const int rr = r0 + row < p.rows ? r0 + row : p.rows - 1;
        long hr = p.sel ? p.sel[rr] : rr;           // an entry of the row list counts from the end when negative, as tensor indexing does
        hr = hr < 0 ? hr + p.h_rows : hr;
        row_h[i] = hr >= 0 && hr < p.h_rows ? (int)hr : 0;   // (an entry outside h reads row 0; the finishing kernel turns its row into NaN)
    }
    // The row list's loads end here: a value that still counts as "in flight" when the loop is entered makes the compiler wait
    // for it at every use, and such a wait also waits for every tile load issued before it.
#pragma unroll
    for (int i = 0; i < 8; i++) asm volatile("" : "+v"(row_h[i]));
    const int row_w0 = v0 + (tid >> 3), last_w = p.vocab - 1;
    auto src_w = [&](const int i, const int k0) __attribute__((always_inline)) {
        const int r = row_w0 + 32 * i < last_w ? row_w0 + 32 * i : last_w;
        return p.w + (long)r * p.w_ld + (kc * 8 + k0);
    };
    auto src_h = [&](const int i, const int k0) __attribute__((always_inline)) { return p.h + (long)row_h[i] * p.h_ld + (kc * 8 + k0); };
    const int dst = (tid >> 3) * PITCH + kc * 16;
    const int nk = p.hidden / BK;
    // Two register sets: the rows of step kt + 2 are requested while step kt is computed and are written to LDS during step
    // kt + 1, so a load has a step and a half (about 3 k cycles of MFMA work) to arrive.  The loads and the waits for them are
    // inline assembly: the compiler's own wait insertion, unsure across the loop's back edge which registers still have a load
    // in flight, waited for the set just requested whenever it touched a register of the other one.  Loads complete in order, so
    // "the older set has landed" is vmcnt(16) while a younger set is in flight and vmcnt(0) otherwise; the registers of the set
    // pass through the waiting asm, which keeps their uses behind it.
    bf16x8 rw[2][8], rh[2][8];
    auto request = [&](const int set, const int i, const int k0) __attribute__((always_inline)) {
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(rw[set][i]) : "v"(src_w(i, k0)) : "memory");
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(rh[set][i]) : "v"(src_h(i, k0)) : "memory");
    };
    auto zero_set = [&](const int set) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int j = 0; j < 8; j++) { rw[set][i][j] = (__bf16)0.f; rh[set][i][j] = (__bf16)0.f; }
    };
    auto landed = [&](const int set, const bool younger_in_flight, const int younger) __attribute__((always_inline)) {
        if (younger_in_flight && younger == 9) asm volatile("s_waitcnt vmcnt(9)" ::: "memory");
        else if (younger_in_flight) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("" : "+v"(rw[set][0]), "+v"(rw[set][1]), "+v"(rw[set][2]), "+v"(rw[set][3]), "+v"(rw[set][4]), "+v"(rw[set][5]), "+v"(rw[set][6]), "+v"(rw[set][7]));
        asm volatile("" : "+v"(rh[set][0]), "+v"(rh[set][1]), "+v"(rh[set][2]), "+v"(rh[set][3]), "+v"(rh[set][4]), "+v"(rh[set][5]), "+v"(rh[set][6]), "+v"(rh[set][7]));
    };

    f32x16 acc[4][4];   // [vocabulary block a][read-row block b]
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[a][b][i] = 0.f;

    // One step, with the memory work dealt out between the MFMAs.  The wave is alone on its SIMD: whatever it issues in one piece
    // (16 global loads, 16 LDS stores, 8 fragment reads) is time the matrix core waits, while an instruction placed between two
    // MFMAs runs in their shadow.  Sixteen groups of four MFMAs per step; groups 0 - 7 each request one W and one h piece of step
    // kt + 2 into `set`, groups 8 - 15 each move one pair of step kt + 1 (the other set) to the other LDS buffer, and every group
    // of the first three quarters reads two fragments of the next quarter.  The steps come in pairs with no branch around the
    // MFMAs (accumulators that are live across a merge of two paths cost the register allocator hundreds of copies): an odd
    // number of steps is rounded up and the extra step multiplies zeros; what the last steps move to LDS is never read.
    const int nk2 = (nk + 1) & ~1;
    auto step = [&](const int kt, const int set) __attribute__((always_inline)) {
        const char* buf = lds + (kt & 1) * STAGE;
        char* nbuf = lds + ((kt + 1) & 1) * STAGE;
        const char* fa = buf + (wv * WT + m) * PITCH + 16 * g;
        const char* fb = buf + (TV + wr * WT + m) * PITCH + 16 * g;
        const int k0 = (kt + 2) * BK;
        const bool more = kt + 2 < nk;   // wave-uniform
        if (!more) zero_set(set);
        bf16x8 av[2][4], bv[2][4];
#pragma unroll
        for (int a = 0; a < 4; a++) {
            av[0][a] = *(const bf16x8*)(fa + 32 * a * PITCH);
            bv[0][a] = *(const bf16x8*)(fb + 32 * a * PITCH);
        }
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
#pragma unroll
            for (int a = 0; a < 4; a++) {
                const int grp = 4 * ks + a;
                if (more) {   // one request per group: W pieces in the even groups, h pieces in the odd ones
                    if (grp & 1) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(rh[set][grp >> 1]) : "v"(src_h(grp >> 1, k0)) : "memory");
                    else asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(rw[set][grp >> 1]) : "v"(src_w(grp >> 1, k0)) : "memory");
                }
                if (grp >= 8) {
                    if (grp == 8) landed(set ^ 1, more, 9);   // nine of this step's requests are younger
                    *(bf16x8*)(nbuf + dst + 32 * (grp - 8) * PITCH) = rw[set ^ 1][grp - 8];
                    *(bf16x8*)(nbuf + TV * PITCH + dst + 32 * (grp - 8) * PITCH) = rh[set ^ 1][grp - 8];
                }
                if (ks < 3) {
                    av[(ks + 1) & 1][a] = *(const bf16x8*)(fa + 32 * a * PITCH + 32 * (ks + 1));
                    bv[(ks + 1) & 1][a] = *(const bf16x8*)(fb + 32 * a * PITCH + 32 * (ks + 1));
                }
#pragma unroll
                for (int b = 0; b < 4; b++) acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[ks & 1][a], bv[ks & 1][b], acc[a][b], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        __syncthreads();
    };

#pragma unroll
    for (int i = 0; i < 8; i++) request(0, i, 0);
    if (nk > 1) {
#pragma unroll
        for (int i = 0; i < 8; i++) request(1, i, BK);
    } else zero_set(1);
    landed(0, nk > 1, 16);
#pragma unroll
    for (int i = 0; i < 8; i++) {
        *(bf16x8*)(lds + dst + 32 * i * PITCH) = rw[0][i];
        *(bf16x8*)(lds + TV * PITCH + dst + 32 * i * PITCH) = rh[0][i];
    }
    __syncthreads();
    for (int kt = 0; kt < nk2; kt += 2) {
        step(kt, 0);
        step(kt + 1, 1);
    }
    __syncthreads();   // everyone is done with the staging buffers: the waves' output blocks go there

    // ---- the capped logits, in place.  Register i of block (a, b) holds vocabulary row vw0 + 32 a + 8 (i / 4) + 4 g + i % 4
    // for read row rw0 + 32 b + m.
    const int vw0 = v0 + wv * WT, rw0 = r0 + wr * WT;
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float x = acc[a][b][i];
                if (BF16) x = to_bf16(x);
                if (CAPPED) x = softcap<BF16>(x, p.cap, p.inv_cap);
                acc[a][b][i] = x;
            }
    // ---- per read row one (reference, sum) pair over the wave's 128 vocabulary rows: 64 values in this lane, 64 in lane ^ 32
    const bool tail = vw0 + WT > p.vocab;   // wave-uniform: some of the wave's vocabulary rows do not exist
#pragma unroll
    for (int b = 0; b < 4; b++) {
        float ref = CAPPED ? p.cap : -INFINITY;
        if (!CAPPED) {
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int i = 0; i < 16; i++)
                    if (!tail || vw0 + 32 * a + 8 * (i >> 2) + 4 * g + (i & 3) < p.vocab) ref = fmaxf(ref, acc[a][b][i]);
            ref = fmaxf(ref, __shfl_xor(ref, 32));
        }
        float sum = 0.f;
        if (ref != -INFINITY) {
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int i = 0; i < 16; i++)
                    if (!tail || vw0 + 32 * a + 8 * (i >> 2) + 4 * g + (i & 3) < p.vocab) sum += __builtin_amdgcn_exp2f((acc[a][b][i] - ref) * LOG2E);
        }
        const float other = __shfl_xor(sum, 32);
        sum = g == 0 ? sum + other : other + sum;   // both halves add in the same order
        const int row = rw0 + 32 * b + m;
        if (g == 0 && row < p.rows) p.part[(long)row * p.n_part + 2 * vtile + wv] = make_float2(ref, sum);
    }
    // ---- what leaves the tile: a 32 x 32 block goes through the wave's LDS tile, vocabulary-major
    float* blk = (float*)lds + w * 32 * BP;
    auto put = [&](const f32x16& x) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 16; i++) blk[(8 * (i >> 2) + 4 * g + (i & 3)) * BP + m] = x[i];
    };
    if (p.cols) {   // the selected columns: rarely one of them lies in this wave's 128 vocabulary rows
        for (int c = 0; c < p.n_cols; c++) {
            const long col = p.cols[c];
            if (col < vw0 || col >= vw0 + WT) continue;   // wave-uniform
            const int ca = (int)(col - vw0) >> 5, cv = (int)(col - vw0) & 31;
#pragma unroll
            for (int a = 0; a < 4; a++) {
                if (a != ca) continue;
#pragma unroll
                for (int b = 0; b < 4; b++) {
                    put(acc[a][b]);
                    const int row = rw0 + 32 * b + m;
                    if (g == 0 && row < p.rows) p.out[(long)row * p.out_ld + c] = blk[cv * BP + m];
                }
            }
        }
    } else {        // the extraction rows: every block, a read row's 32 values of the block as one 128-byte run
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) {
                put(acc[a][b]);
                const int vb = vw0 + 32 * a + m;
                for (int r = g; r < 32; r += 2) {
                    const int row = rw0 + 32 * b + r;
                    if (row < p.rows && vb < p.vocab) p.out[(long)row * p.out_ld + vb] = blk[m * BP + r];
                }
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
        if (q.y <= 0.f) continue;   // a wave's quarter past the end of the vocabulary
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
    const long hr = p.sel ? p.sel[row] : row;
    const bool row_known = hr >= -p.h_rows && hr < p.h_rows;   // a row list entry that names no row of h
    for (int i = threadIdx.x; i < n; i += 256) {
        const bool known = row_known && (!p.cols || (p.cols[i] >= 0 && p.cols[i] < p.vocab));   // no tile wrote a column outside the vocabulary
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
    if (a->h_rows < 0 || a->h_rows > (1ll << 31) - 1 || (a->rows > 0 && a->h_rows == 0))
        return spinf_fail(SPINF_E_ARG, "lm_head: h_rows %lld (the rows of h) out of range", (long long)a->h_rows);
    if (!a->sel && a->rows > a->h_rows) return spinf_fail(SPINF_E_ARG, "lm_head: %lld rows to read without a row list, h has %lld", (long long)a->rows, (long long)a->h_rows);
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
    p.h = (const __bf16*)a->h; p.h_ld = a->h_ld; p.sel = a->sel; p.rows = (int)a->rows; p.h_rows = a->h_rows;
    p.w = (const __bf16*)a->w; p.w_ld = a->w_ld; p.vocab = (int)a->vocab; p.hidden = (int)a->hidden;
    p.cap = a->softcap; p.inv_cap = a->softcap > 0.f ? 1.0f / a->softcap : 0.f;
    p.cols = a->cols; p.n_cols = (int)a->n_cols; p.out = a->out; p.out_ld = a->out_ld;
    p.part = (float2*)a->workspace; p.n_part = (int)parts_of(a);
    p.row_tiles = (int)((a->rows + TR - 1) / TR);
    const int64_t vtiles = (a->vocab + TV - 1) / TV;
    const dim3 grid((unsigned)(p.row_tiles * ((vtiles + 7) / 8 * 8)));
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
