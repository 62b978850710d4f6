// The element-wise work of a Gated DeltaNet layer on either side of the scan, for gfx950 (MI355X): both kernels are bound by
// HBM bandwidth (every input row is read once, every output row written once) and do their arithmetic in fp32 registers.
//
//   gdn_prologue_kernel   spinf_serve/models/qwen35/qwen.py:657-668: 4-tap convolution along each token's path through the tree
//                         (taps = rows of the 3 path predecessors and of the token itself), silu, split into q / k / v, l2 norm
//                         of q and k per head, beta = sigmoid(b), g = -exp(A_log) softplus(a + dt_bias)
//   gdn_gate_kernel       qwen.py:670-672: RMS norm of the scan's output per head, times norm_w, times silu(z)
//
// Work decomposition (both): a lane owns 8 consecutive channels (one 16-byte load / store per row), a workgroup of 256 lanes
// owns 2048 channels and walks over a range of tokens with its per-channel constants in registers; a head's channels sit
// in neighbouring lanes of one wave, so the per-head sums are a few lane exchanges.  Rows are requested eight tokens at a
// time (the walk is bound by memory latency otherwise), and consecutive tokens of a path share three of
// their four tap rows, which stay in registers: each row is read once.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

namespace {

constexpr int LANE_CH = 8;                 // channels per lane
constexpr int WG_CH = 256 * LANE_CH;       // channels per workgroup
constexpr int PF = 8;                      // tokens per batch of row requests
static_assert(PF % 4 == 0, "the tap window's slots must line up from batch to batch");

struct PreParams {
    const __bf16* y; long y_tok;
    const long* conv; const float* w; const float* a_log; const float* dt_bias;
    __bf16* q; __bf16* k; __bf16* v; float* g; __bf16* beta;
    long T; int tok_per_wg;
    int hv, kd, vd, conv_dim;   // kd = key heads x dk, vd = value heads x dv
    int head_lanes;             // lanes that share a key head (dk / 8)
    int normalize;
};

// x / (1 + e^-x) with the hardware's exp2 and reciprocal (1 ulp each; the result is rounded to bf16 anyway): the precise
// expf and division cost about as many instructions as the rest of a channel's work, and these kernels sit near the point
// where the vector ALU, not HBM, sets the pace
__device__ __forceinline__ float silu(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x)); }
// sum over the lanes of a head (aligned groups of head_lanes neighbouring lanes)
__device__ __forceinline__ float head_sum(float v, int head_lanes) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1)
        if (d < head_lanes) v += __shfl_xor(v, d);
    return v;
}
__device__ __forceinline__ float softplus(float x) { return x > 20.0f ? x : log1pf(expf(x)); }   // torch's threshold

__device__ __forceinline__ bf16x8 load_row(const __bf16* y, long y_tok, long row, long T, int c0) {
    const bool none = row < 0 || row >= T;      // "no predecessor": a zero row
    bf16x8 v = *(const bf16x8*)(y + (none ? 0 : row) * y_tok + c0);
    if (none) {
#pragma unroll
        for (int i = 0; i < LANE_CH; i++) v[i] = (__bf16)0.0f;
    }
    return v;
}

constexpr int MAX_TOK = 128;  // tokens a workgroup walks over at most

__global__ __launch_bounds__(256) void gdn_prologue_kernel(const PreParams p) {
    const int c0 = (blockIdx.y * 256 + threadIdx.x) * LANE_CH;
    const long t0 = (long)blockIdx.x * p.tok_per_wg;
    const long t1 = t0 + p.tok_per_wg < p.T ? t0 + p.tok_per_wg : p.T;
    // this range's tap rows, staged once: read from global memory inside the walk they would be vector loads (the walk's
    // stores might alias them, as far as the compiler knows), each with a wait that also drains the stores
    __shared__ int taps[MAX_TOK * 4];
    for (int e = threadIdx.x; e < (int)(t1 - t0) * 4; e += 256) {
        const long r = p.conv[t0 * 4 + e];
        taps[e] = r < 0 || r >= p.T ? -1 : (int)r;
    }
    __syncthreads();
    auto tap = [&](const long t, const int j) { return __builtin_amdgcn_readfirstlane(taps[(int)(t - t0) * 4 + j]); };
    // beta and g: 2 hv values per token (b: the hv columns after z, then a: hv more), spread over the first channel block's lanes
    if (blockIdx.y == 0) {
        const int per_tok = 2 * p.hv;
        const int total = (int)(t1 - t0) * per_tok;
        for (int e0 = 0; e0 < total; e0 += 256 * 8) {       // eight values per lane at a time: their loads go out together
            float val[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int e = e0 + i * 256 + threadIdx.x;
                val[i] = e < total ? (float)p.y[(t0 + e / per_tok) * p.y_tok + p.conv_dim + p.vd + e % per_tok] : 0.f;
            }
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int e = e0 + i * 256 + threadIdx.x;
                if (e >= total) continue;
                const long t = t0 + e / per_tok;
                const int j = e % per_tok;
                if (j < p.hv) p.beta[t * p.hv + j] = (__bf16)(1.0f / (1.0f + expf(-val[i])));
                else p.g[t * p.hv + (j - p.hv)] = -expf(p.a_log[j - p.hv]) * softplus(val[i] + p.dt_bias[j - p.hv]);
            }
        }
    }
    const bool live = c0 < p.conv_dim;       // the last channel block may be partly empty
    const int cc = live ? c0 : 0;
    float w[LANE_CH][4];
#pragma unroll
    for (int i = 0; i < LANE_CH; i++) {
        const float4 wi = *(const float4*)(p.w + (long)(cc + i) * 4);
        w[i][0] = wi.x; w[i][1] = wi.y; w[i][2] = wi.z; w[i][3] = wi.w;
    }
    // where this lane's channels go: q | k | v, each dense [T, heads x dim]
    __bf16* dst;
    long dst_tok;
    if (cc < p.kd) { dst = p.q + cc; dst_tok = p.kd; }
    else if (cc < 2 * p.kd) { dst = p.k + (cc - p.kd); dst_tok = p.kd; }
    else { dst = p.v + (cc - 2 * p.kd); dst_tok = p.vd; }
    const bool norm = p.normalize && cc < 2 * p.kd;

    // Tokens are taken PF at a time: the batch's own rows are requested together and waited for once (on this hardware a wait
    // for a load also waits for every store issued before it, so loads and stores are kept in separate phases: the batch's
    // output rows go out while the next batch's rows come in).  The three predecessor rows are the previous token's last
    // three taps wherever the path simply continues (tap j of this token = tap j + 1 of the one before), and are loaded on
    // the spot at the few tokens where it does not (the first token of a branch, of a job, of this workgroup's range).
    bf16x8 ring[PF];
    bf16x8 x[4];
    int tap1 = -2, tap2 = -2, tap3 = -2;   // the previous token's taps 1..3 (-2: none yet)
    for (long tb = t0; tb < t1; tb += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) ring[u] = load_row(p.y, p.y_tok, tb + u < t1 ? tap(tb + u, 3) : -1, p.T, cc);
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const long t = tb + u;
            if (t >= t1) break;
            const int r0 = tap(t, 0), r1 = tap(t, 1), r2 = tap(t, 2), r3 = tap(t, 3);
            // the window of four tap rows turns by one slot per token (PF is a multiple of 4: the slots are fixed registers)
            bf16x8 &x0 = x[u % 4], &x1 = x[(u + 1) % 4], &x2 = x[(u + 2) % 4], &x3 = x[(u + 3) % 4];
            if (!(r0 == tap1 && r1 == tap2 && r2 == tap3)) {   // the same for every lane
                x0 = load_row(p.y, p.y_tok, r0, p.T, cc);
                x1 = load_row(p.y, p.y_tok, r1, p.T, cc);
                x2 = load_row(p.y, p.y_tok, r2, p.T, cc);
            }
            x3 = ring[u];
            tap1 = r1; tap2 = r2; tap3 = r3;
            bf16x8 s;
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < LANE_CH; i++) {
                float acc = (float)x0[i] * w[i][0];
                acc += (float)x1[i] * w[i][1];
                acc += (float)x2[i] * w[i][2];
                acc += (float)x3[i] * w[i][3];
                s[i] = (__bf16)silu(acc);
            }
            if (__builtin_amdgcn_ballot_w64(norm) != 0) {   // (a wave of v channels skips the norm's sums altogether)
#pragma unroll
                for (int i = 0; i < LANE_CH; i++) ss += (float)s[i] * (float)s[i];
                ss = head_sum(ss, p.head_lanes);   // l2 norm over the head; every lane of the wave takes part in the exchange
            }
            if (norm) {
                const float r = rsqrtf(ss + 1e-6f);
#pragma unroll
                for (int i = 0; i < LANE_CH; i++) s[i] = (__bf16)((float)s[i] * r);
            }
            if (live) *(bf16x8*)(dst + t * dst_tok) = s;
        }
    }
}

struct GateParams {
    const __bf16* o; long o_tok;
    const __bf16* z; long z_tok;
    const __bf16* norm_w; float eps;
    __bf16* out;
    long T; int tok_per_wg;
    int vd, dv, head_lanes;
};

__global__ __launch_bounds__(256) void gdn_gate_kernel(const GateParams p) {
    const int c0 = (blockIdx.y * 256 + threadIdx.x) * LANE_CH;
    const bool live = c0 < p.vd;
    const int cc = live ? c0 : 0;
    const long t0 = (long)blockIdx.x * p.tok_per_wg;
    const long t1 = t0 + p.tok_per_wg < p.T ? t0 + p.tok_per_wg : p.T;
    const bf16x8 nw = *(const bf16x8*)(p.norm_w + cc % p.dv);
    const float inv_dv = 1.0f / (float)p.dv;
    bf16x8 ro[PF], rz[PF];   // PF tokens at a time: their rows are requested together, their results stored while the next come in
    for (long tb = t0; tb < t1; tb += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const long t = tb + u < t1 ? tb + u : t0;
            ro[u] = *(const bf16x8*)(p.o + t * p.o_tok + cc);
            rz[u] = *(const bf16x8*)(p.z + t * p.z_tok + cc);
        }
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const long t = tb + u;
            if (t >= t1) break;
            const bf16x8 o = ro[u], z = rz[u];
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < LANE_CH; i++) ss += (float)o[i] * (float)o[i];
            ss = head_sum(ss, p.head_lanes);
            const float r = rsqrtf(ss * inv_dv + p.eps);
            bf16x8 res;
#pragma unroll
            for (int i = 0; i < LANE_CH; i++) {
                const __bf16 n1 = (__bf16)((float)o[i] * r);                 // the normalised value, in the layer's dtype
                const __bf16 n2 = (__bf16)((float)nw[i] * (float)n1);        // times norm_w, a bf16 product
                res[i] = (__bf16)((float)n2 * silu((float)z[i]));
            }
            if (live) *(bf16x8*)(p.out + t * p.vd + cc) = res;
        }
    }
}

int tokens_per_workgroup(long T, int channel_blocks) {
    // enough workgroups to fill the chip several times over, long enough walks to amortise the per-channel constants
    long per = MAX_TOK;
    while (per > 8 && (T + per - 1) / per * channel_blocks < 4096) per /= 2;
    return (int)per;
}

bool pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

}  // namespace

extern "C" int spinf_gdn_prologue(const spinf_gdn_pre_args* a, void* stream) {
    if (!a) return spinf_fail(SPINF_E_ARG, "gdn_prologue: null args");
    if (a->T <= 0) return SPINF_OK;
    if (!a->y || !a->conv || !a->conv_w || !a->a_log || !a->dt_bias || !a->q || !a->k || !a->v || !a->g || !a->beta)
        return spinf_fail(SPINF_E_ARG, "gdn_prologue: null pointer");
    if (a->h <= 0 || a->hv <= 0 || a->hv > 128) return spinf_fail(SPINF_E_ARG, "gdn_prologue: heads %d / %d out of range", a->h, a->hv);
    if (a->dk % LANE_CH || a->dv % LANE_CH || !pow2(a->dk / LANE_CH) || a->dk / LANE_CH > 64)
        return spinf_fail(SPINF_E_ARG, "gdn_prologue: head dims %d / %d (dk must be 8 x a power of two up to 512, dv a multiple of 8)", a->dk, a->dv);
    const long kd = (long)a->h * a->dk, vd = (long)a->hv * a->dv, conv_dim = 2 * kd + vd;
    if (conv_dim + vd + 2 * a->hv > a->y_tok) return spinf_fail(SPINF_E_ARG, "gdn_prologue: rows of %lld elements cannot hold q k v z b a", (long long)a->y_tok);
    if (a->y_tok % LANE_CH || (uintptr_t)a->y % 16 || (uintptr_t)a->q % 16 || (uintptr_t)a->k % 16 || (uintptr_t)a->v % 16 || (uintptr_t)a->conv_w % 16)
        return spinf_fail(SPINF_E_ARG, "gdn_prologue: tensors must be 16-byte aligned, the row stride a multiple of 8 elements");
    if (a->T >= (1L << 31)) return spinf_fail(SPINF_E_ARG, "gdn_prologue: too many rows");
    PreParams p;
    p.y = (const __bf16*)a->y; p.y_tok = a->y_tok; p.conv = a->conv; p.w = a->conv_w; p.a_log = a->a_log; p.dt_bias = a->dt_bias;
    p.q = (__bf16*)a->q; p.k = (__bf16*)a->k; p.v = (__bf16*)a->v; p.g = a->g; p.beta = (__bf16*)a->beta;
    p.T = a->T; p.hv = a->hv; p.kd = (int)kd; p.vd = (int)vd; p.conv_dim = (int)conv_dim;
    p.head_lanes = a->dk / LANE_CH; p.normalize = a->normalize != 0;
    const int cb = (int)((conv_dim + WG_CH - 1) / WG_CH);
    p.tok_per_wg = tokens_per_workgroup(a->T, cb);
    const dim3 grid((unsigned)((a->T + p.tok_per_wg - 1) / p.tok_per_wg), cb);
    hipLaunchKernelGGL(gdn_prologue_kernel, grid, dim3(256), 0, (hipStream_t)stream, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn_prologue: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}

extern "C" int spinf_gdn_gate(const spinf_gdn_gate_args* a, void* stream) {
    if (!a) return spinf_fail(SPINF_E_ARG, "gdn_gate: null args");
    if (a->T <= 0) return SPINF_OK;
    if (!a->o || !a->z || !a->norm_w || !a->out) return spinf_fail(SPINF_E_ARG, "gdn_gate: null pointer");
    if (a->hv <= 0 || a->dv % LANE_CH || !pow2(a->dv / LANE_CH) || a->dv / LANE_CH > 64)
        return spinf_fail(SPINF_E_ARG, "gdn_gate: %d heads of %d (dv must be 8 x a power of two up to 512)", a->hv, a->dv);
    const long vd = (long)a->hv * a->dv;
    if (a->o_tok < vd || a->z_tok < vd || a->o_tok % LANE_CH || a->z_tok % LANE_CH)
        return spinf_fail(SPINF_E_ARG, "gdn_gate: row strides must be multiples of 8 elements and hold %lld channels", (long long)vd);
    if ((uintptr_t)a->o % 16 || (uintptr_t)a->z % 16 || (uintptr_t)a->norm_w % 16 || (uintptr_t)a->out % 16)
        return spinf_fail(SPINF_E_ARG, "gdn_gate: tensors must be 16-byte aligned");
    if (!(a->eps > 0.f)) return spinf_fail(SPINF_E_ARG, "gdn_gate: eps must be positive");
    GateParams p;
    p.o = (const __bf16*)a->o; p.o_tok = a->o_tok; p.z = (const __bf16*)a->z; p.z_tok = a->z_tok;
    p.norm_w = (const __bf16*)a->norm_w; p.eps = a->eps; p.out = (__bf16*)a->out;
    p.T = a->T; p.vd = (int)vd; p.dv = a->dv; p.head_lanes = a->dv / LANE_CH;
    const int cb = (int)((vd + WG_CH - 1) / WG_CH);
    p.tok_per_wg = tokens_per_workgroup(a->T, cb);
    const dim3 grid((unsigned)((a->T + p.tok_per_wg - 1) / p.tok_per_wg), cb);
    hipLaunchKernelGGL(gdn_gate_kernel, grid, dim3(256), 0, (hipStream_t)stream, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "gdn_gate: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}
