// Extraction-decode attention ("x_decode") for gfx950 (MI355X): one decoding step of every slot x beam of every group.
//
// Replaces _x_attention of spinf_serve/decode.py:71-104.  A query (group g, slot x beam q, head) attends to three key
// ranges that live in three caches and are never copied per slot or per beam:
//   the group's prefix        kp, vp [G, h, Lp, D]   visible to every query of the group where pos_p >= 0,
//   the slots' templates      kt, vt [G, h, Tt, D]   key j visible to the queries of slot own_t[j] (q / beam == own_t[j]),
//   the beams' own tokens     gk, gv [G, h, Q, S, D] key (q', s) visible to query q' alone and only for s <= step,
// on sliding layers the first two also only where qpos[g, q] - pos < window.  The softmax runs over the three ranges
// together (decode.py:96).
//
// Layout of the work.  The three ranges are taken as ONE stream of keys per (group, kv head), cut into tiles of 32 keys:
// prefix | templates | generated (row-major over (q, s), which is how gk / gv lie in memory).  The rows of a (group, kv
// head) are its Q queries x r = H / h heads, row = q * r + head % r, so that the rows of one 32-row block are neighbouring
// queries and their generated keys one contiguous piece of the stream.  A workgroup of four waves owns up to 128 rows (wave
// w the rows 32 w ..) and a contiguous share of the key tiles (a split); it visits the prefix / template tiles of its share
// and those generated tiles that hold keys of its own queries.  K / V tiles go global -> LDS by DMA (global_load_lds), double
// buffered (a ring of NBUF buffers, NBUF - 1 tiles ahead of the arithmetic), one barrier per tile, and are shared by the four
// waves, so every key is read from memory once per 128 rows; two workgroups share a CU, so one's arithmetic runs under the
// other's DMA and softmax.  Padding behind a group's own prefix / template length is neither read nor scheduled.  The loop
// issues no memory operation but these DMAs (the words that say who sees a key ride along), so its wait can count them: all
// but the tiles issued after the one it is about to use.  Scores are S^T = K Q^T with v_mfma_f32_32x32x16_bf16 (a lane owns
// one query row), classic online softmax with a lazily raised reference, O^T = V^T P^T with V^T fragments read through
// ds_read_b64_tr_b16.  A list longer than one split (XdecParams::per tiles) leaves (O, reference, sum) per row and split in a
// workspace and xdec_combine_kernel merges them; a list that fits one split is written out by its one workgroup.
//
// Head dim 512: the output is computed 256 head dims at a time, in two launches (see launch_d).
//
// A row's result depends on its own keys only (fixed tile order, masked entries are exact zeros), so a group's outputs do
// not depend on which other groups share the call.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
#include "attn_tiles.h"

namespace {

constexpr int XTK = 32;            // keys per tile
constexpr int XROWS = 128;         // rows per workgroup
constexpr float XTAU = 8.f;        // the reference point is raised when a tile's maximum exceeds it by more than this (log2 units)
constexpr int NBUF = 2;            // tile buffers in LDS: the DMA runs NBUF - 1 tiles ahead of the arithmetic (two workgroups share a CU)
constexpr int RANGE_EMPTY = 1;     // lo = 1 > hi = 0: a key nobody sees
constexpr int POS_ALWAYS = 0x3fffffff;   // position of a key the window never hides

struct XdecParams {
    const __bf16* q; long q_g, q_h, q_q;
    const __bf16 *kp, *vp, *kt, *vt, *gk, *gv;
    const int *pos_p, *pos_t, *own_t, *len_p, *len_t;
    const long long* qpos;
    const long long* step;
    __bf16* out;
    float* part_o; float* part_ml;
    int G, H, h, r, Q, Lp, Tt, S, beam, window;
    int R, nchunk, nsplit, per;
    int vcol;   // first of the DV value / output head dims this launch computes (head dim 512: two launches of 256)
    float c, cap_in, cap_out;
};

// Key tiles (32 keys of the stream prefix | templates | generated) of a workgroup that owns the queries qlo .. qhi of a group
// whose prefix holds keys in its first len_p entries only and whose template range in its first len_t: the tiles of those
// prefix entries, of those template entries, and of the generated entries of its queries; a tile is listed once.
struct TileList {
    int e0, s1, e1, s2, nt;
    __host__ __device__ TileList(int Lp, int Tt, int S, int len_p, int len_t, int qlo, int qhi) {
        const long lk = (long)Lp + Tt;
        e0 = (len_p + XTK - 1) / XTK;
        s1 = len_t > 0 ? Lp / XTK : e0;
        s1 = s1 > e0 ? s1 : e0;
        e1 = len_t > 0 ? (int)(((long)Lp + len_t + XTK - 1) / XTK) : s1;
        e1 = e1 > s1 ? e1 : s1;
        s2 = (int)((lk + (long)qlo * S) / XTK);
        s2 = s2 > e1 ? s2 : e1;
        int e2 = (int)((lk + (long)(qhi + 1) * S + XTK - 1) / XTK);
        e2 = e2 > s2 ? e2 : s2;
        nt = e0 + (e1 - s1) + (e2 - s2);
    }
    __host__ __device__ int tile(int i) const { return i < e0 ? i : i < e0 + (e1 - s1) ? s1 + (i - e0) : s2 + (i - e0 - (e1 - s1)); }
};

// entries of a group's prefix / template range that can hold keys (the whole range when the caller gave no lengths)
__device__ __forceinline__ int group_len(const int* len, long g, int full) {
    if (!len) return full;
    const int n = len[g];
    return n < 0 ? 0 : n < full ? n : full;
}

// s_waitcnt immediate that waits for all but the n youngest vector memory operations (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
constexpr int vmcnt_imm(int n) { return 0x0f70 | (n & 15) | ((n >> 4) << 14); }

template <int D, int DV, bool WIN, bool CAP>
// (two waves per SIMD asked for: the compiler then stays inside 256 registers; allowed 512, it kept O^T in the accumulator half
// of the file and spent 400 copy instructions per tile moving values between the halves)
__global__ __launch_bounds__(256, D <= 256 ? 2 : 1) void xdec_kernel(const XdecParams p) {
    using GK = Geo<D, XTK>;    // K tile: 32 rows of D head dims
    using GV = Geo<DV, XTK>;   // V tile: 32 rows of DV of the D head dims (DV = D but for head dim 512)
    constexpr int KTILEB = GK::KTILEB, VTILEB = GV::VTILEB, METAB = 2 * 256 + 2 * XTK * 4;   // two words per key as they lie in memory (by DMA), then (range, position) per key
    constexpr int BUFB = KTILEB + VTILEB + METAB;
    constexpr int NS = D / 16, NDT = DV / 32;
    constexpr int IPWK = GK::NREG / 4, IPWV = GV::NREG / 4;
    static_assert(IPWK >= 1 && IPWK * 4 == GK::NREG && IPWV >= 1 && IPWV * 4 == GV::NREG, "the tile's regions must divide among the four waves");
    static_assert(NBUF * BUFB <= 160 * 1024, "LDS budget");
    __shared__ __attribute__((aligned(16))) char bufs[NBUF * BUFB];

    const int lane = threadIdx.x & 63, m = lane & 31, g2 = lane >> 5;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // blockIdx.x = chunk * (G h nsplit) + (g h + hh) * nsplit + split: the row chunks of one (group, kv head) are a multiple of
    // 8 workgroups apart when G h nsplit is, i.e. they share an XCD's L2
    const int per_chunk = p.G * p.h * p.nsplit;
    const int chunk = blockIdx.x / per_chunk;
    const int rest = blockIdx.x - chunk * per_chunk;
    const int split = rest % p.nsplit, gh = rest / p.nsplit;
    const int g = gh / p.h, hh = gh - g * p.h;

    const int row0 = chunk * XROWS + 32 * w;
    const int row = row0 + m;
    const bool valid = row < p.R;
    const int rowc = valid ? row : p.R - 1;
    const int qi = rowc / p.r, head = hh * p.r + (rowc - qi * p.r);
    const bool wave_on = row0 < p.R;
    const int qlo_w = row0 / p.r, qhi_w = ((row0 + 31 < p.R ? row0 + 31 : p.R - 1)) / p.r;
    const int last_row = chunk * XROWS + XROWS - 1 < p.R ? chunk * XROWS + XROWS - 1 : p.R - 1;
    const TileList tl(p.Lp, p.Tt, p.S, group_len(p.len_p, g, p.Lp), group_len(p.len_t, g, p.Tt), (chunk * XROWS) / p.r, last_row / p.r);
    // a split is p.per tiles of the list: a group with a short prefix has fewer splits than p.nsplit, the rest leave at once
    const int i0 = split * p.per, i1 = i0 + p.per < tl.nt ? i0 + p.per : tl.nt;
    if (i0 >= i1) return;

    const long ltot = (long)p.Lp + p.Tt + (long)p.Q * p.S;
    const int step = (int)*p.step;
    const int qpos_q = WIN ? (int)p.qpos[(long)g * p.Q + qi] : 0;

    bf16x8 qf[NS];
    {
        const __bf16* qp = p.q + (long)g * p.q_g + (long)head * p.q_h + (long)qi * p.q_q + 8 * g2;
#pragma unroll
        for (int s = 0; s < NS; s++) qf[s] = *(const bf16x8*)(qp + 16 * s);
    }
    f32x16 o[NDT];
#pragma unroll
    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[dt][i] = 0.f;
    float M = -INFINITY, l = 0.f;

    // fragment addresses inside a tile (see Geo): K row m, 16-byte chunk g2 of each 32-byte step; V^T through the transposing read
    const int tr_a = lane & 3, tr_j = (lane >> 2) & 3, tr_mb = (lane >> 4) & 1;
    const int k_lane = GK::k_off(m) + 16 * g2;
    const int v_lane = GV::v_off(4 * g2 + tr_j) + 32 * tr_mb + 8 * tr_a;

    // element offset of key `key` of the stream inside its cache, and which cache (0 prefix, 1 templates, 2 generated)
    auto locate = [&](long key, int& which) -> long {
        key = key < ltot ? key : ltot - 1;
        if (key < p.Lp) { which = 0; return ((long)gh * p.Lp + key) * D; }
        if (key < (long)p.Lp + p.Tt) { which = 1; return ((long)gh * p.Tt + (key - p.Lp)) * D; }
        which = 2;
        return ((long)gh * p.Q * p.S + (key - p.Lp - p.Tt)) * D;
    };
    // per-lane part of a DMA's source address when the tile's 32 keys are 32 consecutive rows of one cache
    const unsigned lane_src_k = (unsigned)((lane / GK::CPR) * GK::NREG * D * 2 + (lane % GK::CPR) * 16);
    const unsigned lane_src_v = (unsigned)((lane / GV::CPR) * GV::NREG * D * 2 + (lane % GV::CPR) * 16);
    constexpr int DMAS = IPWK + IPWV + 2;   // DMA instructions per wave and tile: its share of K and of V, two words per key
    // Starts the DMA of a tile: K and V rows, and for every key the two words that say who sees it (prefix: position; template:
    // owning slot, position), which every wave copies to the same place (so that all waves have the same number of DMAs in
    // flight and the loop's wait can count them).  No other memory operation is issued inside the loop.
    auto issue = [&](const unsigned buf, const int tile) {
        const long k0 = (long)tile * XTK, lk = (long)p.Lp + p.Tt;
        const int which = k0 + XTK <= p.Lp ? 0 : (k0 >= p.Lp && k0 + XTK <= lk) ? 1 : (k0 >= lk && k0 + XTK <= ltot) ? 2 : -1;
        if (which >= 0) {   // the usual case: a wave-uniform base, no vector arithmetic on addresses
            const long first = which == 0 ? (long)gh * p.Lp + k0 : which == 1 ? (long)gh * p.Tt + (k0 - p.Lp) : (long)gh * p.Q * p.S + (k0 - lk);
            const char* kb = (const char*)(which == 0 ? p.kp : which == 1 ? p.kt : p.gk) + first * (D * 2);
            const char* vb = (const char*)(which == 0 ? p.vp : which == 1 ? p.vt : p.gv) + first * (D * 2) + p.vcol * 2;
#pragma unroll
            for (int i = 0; i < IPWK; i++) {
                const int reg = w * IPWK + i;
                dma16_uniform(kb + reg * (D * 2), lane_src_k, buf + reg * GK::KRS);
            }
#pragma unroll
            for (int i = 0; i < IPWV; i++) {
                const int reg = w * IPWV + i;
                dma16_uniform(vb + reg * (D * 2), lane_src_v, buf + KTILEB + reg * GV::VRS);
            }
        } else {
            // (the cache pointers as opaque scalar values: picking one per lane is then a register select; left as fields of
            // the argument block, the compiler picks the FIELD per lane and loads the pointer from memory in front of every
            // DMA, with a wait that also waits for the DMAs before it)
            const char* const kp_s = uniform_ptr((const char*)p.kp); const char* const vp_s = uniform_ptr((const char*)p.vp);
            const char* const kt_s = uniform_ptr((const char*)p.kt); const char* const vt_s = uniform_ptr((const char*)p.vt);
            const char* const gk_s = uniform_ptr((const char*)p.gk); const char* const gv_s = uniform_ptr((const char*)p.gv);
#pragma unroll
            for (int i = 0; i < IPWK; i++) {   // a tile across two caches, or the stream's last
                const int reg = w * IPWK + i;
                int wh;
                const long off = locate(k0 + reg + GK::NREG * (lane / GK::CPR), wh) + (lane % GK::CPR) * 8;
                dma16_lane((wh == 0 ? kp_s : wh == 1 ? kt_s : gk_s) + off * 2, buf + reg * GK::KRS);
            }
#pragma unroll
            for (int i = 0; i < IPWV; i++) {
                const int reg = w * IPWV + i;
                int wh;
                const long off = locate(k0 + reg + GV::NREG * (lane / GV::CPR), wh) + (lane % GV::CPR) * 8 + p.vcol;
                dma16_lane((wh == 0 ? vp_s : wh == 1 ? vt_s : gv_s) + off * 2, buf + KTILEB + reg * GV::VRS);
            }
        }
        const long key = k0 + (lane & (XTK - 1));
        const bool pre = key < p.Lp, tem = !pre && key < lk;
        const int* const pos_p_s = (const int*)uniform_ptr((const char*)p.pos_p); const int* const pos_t_s = (const int*)uniform_ptr((const char*)p.pos_t);
        const int* const own_t_s = (const int*)uniform_ptr((const char*)p.own_t); const char* const step_s = uniform_ptr((const char*)p.step);
        const int* a0 = pre ? pos_p_s + (long)g * p.Lp + key : tem ? own_t_s + (long)g * p.Tt + (key - p.Lp) : (const int*)step_s;
        const int* a1 = tem ? pos_t_s + (long)g * p.Tt + (key - p.Lp) : (const int*)step_s;
        dma4_lane(a0, buf + KTILEB + VTILEB);
        dma4_lane(a1, buf + KTILEB + VTILEB + 256);
    };
    // (range, position) of key m of a tile from its two words: who may see it (queries lo .. hi, packed lo | hi << 16)
    auto derive = [&](const int tile, const int r0, const int r1, int& range, int& kpos) {
        const long key = (long)tile * XTK + m;
        range = RANGE_EMPTY;
        kpos = POS_ALWAYS;
        if (key < p.Lp) {
            kpos = r0;
            if (kpos >= 0) range = (p.Q - 1) << 16;
        } else if (key < (long)p.Lp + p.Tt) {
            kpos = r1;
            if (r0 >= 0 && r0 * p.beam < p.Q) {
                const int hi = r0 * p.beam + p.beam - 1;
                range = (r0 * p.beam) | ((hi < p.Q ? hi : p.Q - 1) << 16);
            }
        } else if (key < ltot) {
            const int idx = (int)(key - p.Lp - p.Tt), qq = idx / p.S;
            if (idx - qq * p.S <= step) range = qq | (qq << 16);
        }
    };

    // Everything loaded so far (queries, step, positions) is waited for HERE: left to the compiler, the waits would sit in front
    // of the first uses inside the loop, where they would wait for the tile DMAs in flight as well, every iteration.
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
#pragma unroll
    for (int s = 0; s < NS; s++) asm volatile("" : "+v"(qf[s]));
    const unsigned buf_base = lds_addr(bufs);
    for (int j = 0; j < NBUF - 1; j++)
        if (i0 + j < i1) issue(buf_base + j * BUFB, tl.tile(i0 + j));
    for (int i = i0; i < i1; i++) {
        // this wave's share of tile i has landed: all but the DMAs of the tiles issued after it
        const int ahead = i1 - 1 - i;
        if (ahead >= NBUF - 2) __builtin_amdgcn_s_waitcnt(vmcnt_imm((NBUF - 2) * DMAS));
        else if (ahead == 1) __builtin_amdgcn_s_waitcnt(vmcnt_imm(DMAS));
        else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();                      // ... and everybody's; all waves are done with tile i - 1
        const int b = (i - i0) % NBUF;
        if (i + NBUF - 1 < i1) issue(buf_base + ((i - i0 + NBUF - 1) % NBUF) * BUFB, tl.tile(i + NBUF - 1));
        const char* kb = bufs + b * BUFB;
        const char* vb = kb + KTILEB;
        int* meta = (int*)(bufs + b * BUFB + KTILEB + VTILEB);
        bool all_seen;
        {   // who sees key m of the tile; does any key belong to a query of this wave, do all queries see all keys?
            int range, kpos;
            derive(tl.tile(i), meta[m], meta[64 + m], range, kpos);
            const int lo = range & 0xffff, hi = (unsigned)range >> 16;
            const bool need = wave_on && lo <= hi && lo <= qhi_w && hi >= qlo_w;
            if (__builtin_amdgcn_ballot_w64(need) == 0) continue;
            all_seen = !WIN && __builtin_amdgcn_ballot_w64(range != ((p.Q - 1) << 16)) == 0;
            if (!all_seen) {   // every wave leaves the same values at the same place and reads back what it wrote itself
                meta[128 + m] = range;
                meta[128 + XTK + m] = kpos;
            }
        }
        meta += 128;
        const char* krow = kb + k_lane;
        const char* vrow = vb + v_lane;
        f32x16 s_acc;
#pragma unroll
        for (int i2 = 0; i2 < 16; i2++) s_acc[i2] = 0.f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const bf16x8 kf = *(const bf16x8*)(krow + 32 * s);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], s_acc, 0, 0, 0);
        }
        // register i of the S^T tile holds key 8 (i / 4) + 4 g2 + i % 4 of the tile
        float mx = -INFINITY;
        auto to_log2 = [&](float t) {
            if (CAP) {   // softcap * tanh(score * scale / softcap), in log2 units
                const float e = __builtin_amdgcn_exp2f(t * p.cap_in);   // exp(2 y), y = score * scale / softcap
                return p.cap_out * (1.0f - 2.0f * __builtin_amdgcn_rcpf(e + 1.0f));
            }
            return t * p.c;
        };
        if (all_seen) {   // every row sees every key of the tile: no mask
#pragma unroll
            for (int i2 = 0; i2 < 16; i2++) {
                s_acc[i2] = to_log2(s_acc[i2]);
                mx = fmaxf(mx, s_acc[i2]);
            }
        } else {
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                const int ko = 8 * i4 + 4 * g2;
                const int4 rg4 = *(const int4*)(meta + ko);
                const int4 kp4 = *(const int4*)(meta + XTK + ko);
                const int rgv[4] = {rg4.x, rg4.y, rg4.z, rg4.w};
                const int kpv[4] = {kp4.x, kp4.y, kp4.z, kp4.w};
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int lo = rgv[jj] & 0xffff, hi = (unsigned)rgv[jj] >> 16;
                    bool vis = (lo <= qi) & (qi <= hi);
                    if (WIN) vis = vis & ((qpos_q - kpv[jj]) < p.window);
                    const float t = vis ? to_log2(s_acc[4 * i4 + jj]) : -INFINITY;
                    s_acc[4 * i4 + jj] = t;
                    mx = fmaxf(mx, t);
                }
            }
        }
        mx = lane32_max(mx);
        const bool up = mx > M + XTAU;
        const float mn = up ? mx : M;
        const float alpha = up ? __builtin_amdgcn_exp2f(M - mn) : 1.0f;
        if (__builtin_amdgcn_ballot_w64(up && M != -INFINITY) != 0) {   // rows without a key so far hold zeros
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i2 = 0; i2 < 16; i2++) o[dt][i2] *= alpha;
        }
        l *= alpha;
        M = mn;
        const float ms = mn == -INFINITY ? 0.f : mn;
        bf16x8 pb[2];
        float sum = 0.f;
#pragma unroll
        for (int i2 = 0; i2 < 16; i2++) {
            const float pr = __builtin_amdgcn_exp2f(s_acc[i2] - ms);
            sum += pr;
            pb[i2 >> 3][i2 & 7] = (__bf16)pr;
        }
        l += sum;
#pragma unroll
        for (int f = 0; f < 2 * NDT; f++) {
            const char* vp = vrow + GV::v_off(16 * (f / NDT)) + 64 * (f % NDT);
            const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)vp);
            const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vp + GV::v_off(8)));
            const bf16x8 a = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
            o[f % NDT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[f / NDT], o[f % NDT], 0, 0, 0);
        }
    }

    // register i of O^T tile dt holds head dim 32 dt + 8 (i / 4) + 4 g2 + i % 4 of this lane's row
    const float lsum = lane32_sum(l);
    if (!valid) return;
    if (p.nsplit == 1 || tl.nt <= p.per) {   // the list's only split: the output itself (lists longer than p.per leave partial results)
        const float inv = 1.0f / lsum;
        __bf16* ob = p.out + (((long)g * p.Q + qi) * p.H + head) * D + p.vcol;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                bf16x4 r;
#pragma unroll
                for (int jj = 0; jj < 4; jj++) r[jj] = (__bf16)(o[dt][4 * i4 + jj] * inv);
                *(bf16x4*)(ob + 32 * dt + 8 * i4 + 4 * g2) = r;
            }
    } else {
        const long prow = (((long)g * p.H + head) * p.Q + qi) * p.nsplit + split;
        float* po = p.part_o + prow * DV;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++)
                *(float4*)(po + 32 * dt + 8 * i4 + 4 * g2) = make_float4(o[dt][4 * i4], o[dt][4 * i4 + 1], o[dt][4 * i4 + 2], o[dt][4 * i4 + 3]);
        if (g2 == 0) *(float2*)(p.part_ml + prow * 2) = make_float2(M, lsum);
    }
}

// out = sum_s 2^(M_s - M*) O_s / sum_s 2^(M_s - M*) l_s over the splits of a row, splits in ascending order; one thread per 4 head dims
template <int D, int DV>
__global__ __launch_bounds__(256) void xdec_combine_kernel(const XdecParams p, const long n_rows) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    const long rowid = idx / (DV / 4);
    const int d4 = (int)(idx - rowid * (DV / 4));
    if (rowid >= n_rows) return;
    const long gg = rowid / ((long)p.H * p.Q);
    const int head = (int)((rowid / p.Q) % p.H), qi = (int)(rowid % p.Q);
    // the splits that exist for this row: those of its row chunk's tile list
    const int chunk = (qi * p.r + head % p.r) / XROWS;
    const int last_row = chunk * XROWS + XROWS - 1 < p.R ? chunk * XROWS + XROWS - 1 : p.R - 1;
    const TileList tl(p.Lp, p.Tt, p.S, group_len(p.len_p, gg, p.Lp), group_len(p.len_t, gg, p.Tt), (chunk * XROWS) / p.r, last_row / p.r);
    const int ns = (tl.nt + p.per - 1) / p.per;
    if (ns == 1) return;   // written by the one workgroup itself
    const float* ml = p.part_ml + rowid * p.nsplit * 2;
    float mstar = -INFINITY;
    for (int s = 0; s < ns; s++) mstar = fmaxf(mstar, ml[2 * s]);
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float lsum = 0.f;
    for (int s = 0; s < ns; s++) {
        const float ms = ml[2 * s];
        if (ms == -INFINITY) continue;
        const float wgt = __builtin_amdgcn_exp2f(ms - mstar);
        const float4 x = *(const float4*)(p.part_o + (rowid * p.nsplit + s) * DV + 4 * d4);
        acc.x += wgt * x.x; acc.y += wgt * x.y; acc.z += wgt * x.z; acc.w += wgt * x.w;
        lsum += wgt * ml[2 * s + 1];
    }
    const float inv = 1.0f / lsum;
    bf16x4 r;
    r[0] = (__bf16)(acc.x * inv); r[1] = (__bf16)(acc.y * inv); r[2] = (__bf16)(acc.z * inv); r[3] = (__bf16)(acc.w * inv);
    *(bf16x4*)(p.out + ((gg * p.Q + qi) * p.H + head) * D + p.vcol + 4 * d4) = r;
}

int check_args(const spinf_xdec_args* a) {
    if (!a) return spinf_fail(SPINF_E_ARG, "xdecode_attn: null args");
    if (a->G < 0 || a->H <= 0 || a->h <= 0 || a->H % a->h || a->Q < 0 || a->S <= 0 || a->Lp < 0 || a->Tt < 0 || a->beam <= 0)
        return spinf_fail(SPINF_E_ARG, "xdecode_attn: bad sizes (G %d H %d h %d Q %d S %d Lp %d Tt %d beam %d)", a->G, a->H, a->h, a->Q, a->S, a->Lp, a->Tt, a->beam);
    if (a->d != 64 && a->d != 128 && a->d != 256 && a->d != 512) return spinf_fail(SPINF_E_ARG, "xdecode_attn: head dim %d not supported (64, 128, 256, 512)", a->d);
    if (a->Q > 32767 || (int64_t)a->Q * (a->H / a->h) > (1 << 20)) return spinf_fail(SPINF_E_ARG, "xdecode_attn: %d queries per group out of range", a->Q);
    if ((int64_t)a->Lp + a->Tt + (int64_t)a->Q * a->S > (1 << 30)) return spinf_fail(SPINF_E_ARG, "xdecode_attn: key stream too long");
    if ((int64_t)a->G * a->h > (1 << 24)) return spinf_fail(SPINF_E_ARG, "xdecode_attn: too many (group, kv head) pairs");
    if (a->window < 0) return spinf_fail(SPINF_E_ARG, "xdecode_attn: window %d", a->window);
    if (a->softcap < 0.f) return spinf_fail(SPINF_E_ARG, "xdecode_attn: softcap %g", (double)a->softcap);
    return SPINF_OK;
}

int n_chunks(const spinf_xdec_args* a) { return (int)(((int64_t)a->Q * (a->H / a->h) + XROWS - 1) / XROWS); }

// Head dim 512 (the Gemma-4 full-attention layers): O^T for 32 rows x 512 head dims would be 256 accumulator registers per lane
// next to 128 of queries, so the output is computed 256 head dims at a time, in two launches: each computes the scores over all
// 512 head dims and P V for one half of V's columns (DV = 256, XdecParams::vcol), in one workgroup per CU.
template <int D, int DV>
int launch_d(XdecParams p, bool cap, int blocks, hipStream_t s) {
    const bool win = p.window > 0;
    p.part_ml = p.part_o ? p.part_o + (long)p.G * p.H * p.Q * p.nsplit * DV : nullptr;
    for (p.vcol = 0; p.vcol < D; p.vcol += DV) {
        if (win && cap) hipLaunchKernelGGL((xdec_kernel<D, DV, true, true>), dim3(blocks), dim3(256), 0, s, p);
        else if (win) hipLaunchKernelGGL((xdec_kernel<D, DV, true, false>), dim3(blocks), dim3(256), 0, s, p);
        else if (cap) hipLaunchKernelGGL((xdec_kernel<D, DV, false, true>), dim3(blocks), dim3(256), 0, s, p);
        else hipLaunchKernelGGL((xdec_kernel<D, DV, false, false>), dim3(blocks), dim3(256), 0, s, p);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "xdecode_attn: launch: %s", hipGetErrorString(e));
        if (p.nsplit > 1) {
            const long n_rows = (long)p.G * p.H * p.Q;
            const long threads = n_rows * (DV / 4);
            hipLaunchKernelGGL((xdec_combine_kernel<D, DV>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s, p, n_rows);
            e = hipGetLastError();
            if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "xdecode_attn: launch (combine): %s", hipGetErrorString(e));
        }
    }
    return SPINF_OK;
}

// tiles of the longest list of the call: a group whose prefix and template ranges are full, the row chunk with the most tiles
// (not always the first: the tile where the template range ends and the generated entries begin counts with the former, and
// where a chunk's generated entries begin and end inside their tiles differs from chunk to chunk)
int max_tiles(const spinf_xdec_args* a) {
    const int r = a->H / a->h;
    const long R = (long)a->Q * r;
    int most = 0;
    for (long row0 = 0; row0 < R; row0 += XROWS) {
        const long last = row0 + XROWS - 1 < R ? row0 + XROWS - 1 : R - 1;
        const int nt = TileList(a->Lp, a->Tt, a->S, a->Lp, a->Tt, (int)(row0 / r), (int)(last / r)).nt;
        most = nt > most ? nt : most;
    }
    return most;
}

}  // namespace

extern "C" int spinf_xdecode_plan(const spinf_xdec_args* a, int32_t* nsplit, int64_t* workspace_bytes) {
    const int rc = check_args(a);
    if (rc) return rc;
    if (!nsplit || !workspace_bytes) return spinf_fail(SPINF_E_ARG, "xdecode_plan: null output");
    *nsplit = 1;
    *workspace_bytes = 0;
    if (a->G == 0 || a->Q == 0) return SPINF_OK;
    // Two workgroups per CU of 256 run at a time.  Take the split count with the fewest tile steps one after the other:
    // rounds of workgroups x (tiles per split + 2 for a workgroup's start and end + what a split's partial results cost in
    // memory traffic, written and read back, in tiles), a split keeping at least 8 tiles.
    const long base = (long)a->G * a->h * n_chunks(a);
    const int nt = max_tiles(a);
    long best = -1;
    for (int ns = 1; ns <= 16; ns++) {
        const int per = (nt + ns - 1) / ns;
        if (ns > 1 && per < 8) break;
        const long slots = 512;
        const long rounds = (base * ns + slots - 1) / slots;
        const int r = a->H / a->h;
        const long rows = (int64_t)a->Q * r < XROWS ? (int64_t)a->Q * r : XROWS;
        const long partial_tiles = ns > 1 ? (rows * (a->d + 2) * 8 + XTK * a->d * 4 - 1) / (XTK * a->d * 4) : 0;
        const long cost = rounds * (per + 2 + partial_tiles);
        if (best < 0 || cost < best) { best = cost; *nsplit = ns; }
    }
    if (*nsplit > 1) *workspace_bytes = (int64_t)a->G * a->H * a->Q * *nsplit * (a->d + 2) * 4;
    return SPINF_OK;
}

extern "C" int spinf_xdecode_tiles(const spinf_xdec_args* a, int32_t* tiles) {
    const int rc = check_args(a);
    if (rc) return rc;
    if (!tiles) return spinf_fail(SPINF_E_ARG, "xdecode_tiles: null output");
    *tiles = a->G == 0 || a->Q == 0 ? 0 : max_tiles(a);
    return SPINF_OK;
}

extern "C" int spinf_xdecode_attn_fwd(const spinf_xdec_args* a, void* stream) {
    const int rc = check_args(a);
    if (rc) return rc;
    if (a->G == 0 || a->Q == 0) return SPINF_OK;
    if (!a->q || !a->out || !a->gk || !a->gv || !a->step) return spinf_fail(SPINF_E_ARG, "xdecode_attn: null pointer (q, out, gk, gv, step)");
    if (a->Lp > 0 && (!a->kp || !a->vp || !a->pos_p)) return spinf_fail(SPINF_E_ARG, "xdecode_attn: prefix of %d keys without kp / vp / pos_p", a->Lp);
    if (a->Tt > 0 && (!a->kt || !a->vt || !a->pos_t || !a->own_t)) return spinf_fail(SPINF_E_ARG, "xdecode_attn: %d template keys without kt / vt / pos_t / own_t", a->Tt);
    if (a->window > 0 && !a->qpos) return spinf_fail(SPINF_E_ARG, "xdecode_attn: a sliding layer needs qpos");
    if (a->q_q % 8 || a->q_h % 8 || a->q_g % 8) return spinf_fail(SPINF_E_ARG, "xdecode_attn: query strides must be multiples of 8 elements");
    for (const void* ptr : {a->q, (const void*)a->out, a->kp, a->vp, a->kt, a->vt, a->gk, a->gv})
        if ((uintptr_t)ptr % 16) return spinf_fail(SPINF_E_ARG, "xdecode_attn: q, out and the caches must be 16-byte aligned");
    if (a->nsplit < 1 || a->nsplit > 64) return spinf_fail(SPINF_E_ARG, "xdecode_attn: nsplit %d (1 .. 64)", a->nsplit);
    if (a->tiles_per_split < 0 || (a->tiles_per_split > 0 && (int64_t)a->tiles_per_split * a->nsplit < max_tiles(a)))
        return spinf_fail(SPINF_E_ARG, "xdecode_attn: %d splits of %d tiles do not cover the longest list (%d tiles)", a->nsplit, a->tiles_per_split, max_tiles(a));
    const int64_t need = a->nsplit > 1 ? (int64_t)a->G * a->H * a->Q * a->nsplit * (a->d + 2) * 4 : 0;
    if (need > 0 && (!a->workspace || a->workspace_bytes < need || (uintptr_t)a->workspace % 16))
        return spinf_fail(SPINF_E_ARG, "xdecode_attn: %d splits need a 16-byte aligned workspace of %lld bytes", a->nsplit, (long long)need);
    XdecParams p;
    p.q = (const __bf16*)a->q; p.q_g = a->q_g; p.q_h = a->q_h; p.q_q = a->q_q;
    p.kp = (const __bf16*)a->kp; p.vp = (const __bf16*)a->vp; p.kt = (const __bf16*)a->kt; p.vt = (const __bf16*)a->vt;
    p.gk = (const __bf16*)a->gk; p.gv = (const __bf16*)a->gv;
    p.pos_p = a->pos_p; p.pos_t = a->pos_t; p.own_t = a->own_t; p.len_p = a->len_p; p.len_t = a->len_t;
    p.qpos = (const long long*)a->qpos; p.step = (const long long*)a->step;
    p.out = (__bf16*)a->out;
    p.part_o = (float*)a->workspace;
    p.part_ml = p.part_o ? p.part_o + (int64_t)a->G * a->H * a->Q * a->nsplit * a->d : nullptr;
    p.G = a->G; p.H = a->H; p.h = a->h; p.r = a->H / a->h; p.Q = a->Q; p.Lp = a->Lp; p.Tt = a->Tt; p.S = a->S; p.beam = a->beam;
    p.window = a->window;
    p.R = p.Q * p.r; p.nchunk = n_chunks(a); p.nsplit = a->nsplit;
    p.per = a->tiles_per_split > 0 ? a->tiles_per_split : (max_tiles(a) + p.nsplit - 1) / p.nsplit;
    const float log2e = 1.4426950408889634f;
    p.c = a->scale * log2e;
    p.cap_in = a->softcap > 0.f ? 2.0f * log2e * a->scale / a->softcap : 0.f;
    p.cap_out = a->softcap * log2e;
    const long blocks = (long)p.G * p.h * p.nsplit * p.nchunk;
    if (blocks > 0x7fffffffL) return spinf_fail(SPINF_E_ARG, "xdecode_attn: too many workgroups");
    const bool cap = a->softcap > 0.f;
    hipStream_t s = (hipStream_t)stream;
    switch (a->d) {
        case 64: return launch_d<64, 64>(p, cap, (int)blocks, s);
        case 128: return launch_d<128, 128>(p, cap, (int)blocks, s);
        case 256: return launch_d<256, 256>(p, cap, (int)blocks, s);
        default: return launch_d<512, 256>(p, cap, (int)blocks, s);
    }
}
