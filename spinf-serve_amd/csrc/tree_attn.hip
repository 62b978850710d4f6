// Tree-mask packed-prefill attention for gfx950 (MI355X): flash-style forward over a per-query-tile list of key tiles.
//
// Replaces the flex_attention call of spinf_serve/models/gemma4.py:107-118 and spinf_serve/models/qwen35/qwen.py:614,620;
// the per-element visibility test is the predicate of spinf_serve/scorer.py:173-177.
//
// Work decomposition.  One workgroup (4 waves) = one 128-token query tile x RT query heads of one GQA group; wave w owns
// tokens 32w..32w+31 of the tile for all RT heads, so a K or V fragment read from LDS feeds RT MFMAs and the mask of a
// 32x32 block is evaluated once for all RT heads.  Scores are computed transposed, S^T = K Q^T, with
// v_mfma_f32_32x32x16_bf16: a lane then owns ONE query row (column lane%32 of the 32x32 result) and 16 of the 32 keys,
// so the softmax row reductions are in-lane plus one exchange with lane^32.  O^T = V^T P^T reuses the score registers
// as the B operand without any shuffle; V^T fragments come from row-major V in LDS through ds_read_b64_tr_b16.
//
// K/V tiles (64 keys) are copied global -> LDS by the DMA path (global_load_lds_dwordx4), double-buffered, with an XOR
// swizzle of the 16-byte chunks that keeps both the b128 reads of K and the transposing reads of V free of bank
// conflicts.  The key tile's art/end/pos ride along so that masked blocks never touch global memory in the loop.
//
// Reduction order.  A row's keys are visited in ascending 32-key blocks that depend only on the row's own job (jobs start
// on 128-token boundaries), masked entries contribute exact zeros, and a skipped block equals a fully masked one bit for
// bit; the running maximum is updated per row from that row's scores only.  A job's output is therefore bit-identical
// whatever it is packed with.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

struct AttnParams {
    const __bf16* q; const __bf16* k; const __bf16* v; __bf16* o;
    long q_tok, q_head, k_tok, k_head, v_tok, v_head, o_tok, o_head;
    int n, group;
    float c;              // scale * log2(e)
    int window;
    const int* art; const int* end; const int* pos;
    const int* qt_ptr; const int* kv_idx; const unsigned* kv_bits; const int* order;
    int nqt, total, per_xcd;
};


__device__ __forceinline__ float lane32_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float lane32_sum(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int D>
struct Geo {
    // LDS image of one 64-row K or V tile.  One wave-wide 16-byte DMA instruction fills 1 KiB of contiguous LDS (a
    // "region"); a region holds rows r, r + NREG, r + 2 NREG ... so that consecutive rows lie in consecutive regions, and
    // regions are padded apart: by 16 bytes for K (the b128 fragment reads of 16 consecutive rows then cover all 64
    // banks) and by 64 bytes for V (the transposing reads touch 64 bytes of each of 4 consecutive rows).  Every address
    // is a per-lane base plus a compile-time offset.
    static constexpr int ROWB = D * 2;                 // bytes of one K / V row
    static constexpr int CPR = ROWB / 16;              // 16-byte chunks per row
    static constexpr int RPI = 1024 / ROWB;            // rows per region
    static constexpr int NREG = 64 / RPI;              // regions per tile
    static constexpr int IPW = NREG / 4;               // DMA instructions per wave and tile
    static constexpr int KRS = 1024 + 16, VRS = 1024 + 64;
    static constexpr int KTILEB = NREG * KRS, VTILEB = NREG * VRS;
    static constexpr int METAB = 3 * 64 * 4;
    static constexpr int BUFB = KTILEB + VTILEB + METAB;   // K tile | V tile | art,end,pos of the keys
    __host__ __device__ static constexpr int k_off(int row) { return (row % NREG) * KRS + (row / NREG) * ROWB; }
    __host__ __device__ static constexpr int v_off(int row) { return (row % NREG) * VRS + (row / NREG) * ROWB; }
};

// Starts the DMA of key tile kt (64 keys of kv head kvh) into an LDS buffer.  Wave w copies regions w*IPW .. w*IPW+IPW-1;
// lane -> (slot = which row of the region, 16-byte chunk of the row).  For a tile that lies fully inside the stream every
// address is a wave-uniform base plus a per-lane constant (lane_k / lane_v, bytes), so the loop spends no vector ALU on
// addressing; the last, partial tile clamps its rows per lane.
template <int D>
__device__ __forceinline__ void issue_tile(const AttnParams& p, char* buf, int kt, int kvh, int w, int lane, unsigned lane_k, unsigned lane_v) {
    using G = Geo<D>;
    const char* kbase = (const char*)(p.k + (long)kvh * p.k_head);
    const char* vbase = (const char*)(p.v + (long)kvh * p.v_head);
    if (kt * 64 + 64 <= p.n) {
#pragma unroll
        for (int i = 0; i < G::IPW; i++) {
            const int reg = w * G::IPW + i;
            const long row = (long)kt * 64 + reg;
            __builtin_amdgcn_global_load_lds((gbl_void*)(kbase + row * p.k_tok * 2 + lane_k), (lds_void*)(buf + reg * G::KRS), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gbl_void*)(vbase + row * p.v_tok * 2 + lane_v), (lds_void*)(buf + G::KTILEB + reg * G::VRS), 16, 0, 0);
        }
        if (w < 3) {   // wave 0: art, wave 1: end, wave 2: pos of the 64 keys
            const int* src = (w == 0 ? p.art : w == 1 ? p.end : p.pos) + (long)kt * 64;
            __builtin_amdgcn_global_load_lds((gbl_void*)(src + lane), (lds_void*)(buf + G::KTILEB + G::VTILEB + w * 256), 4, 0, 0);
        }
    } else {
        const int slot = lane / G::CPR, chunk = lane % G::CPR;
#pragma unroll
        for (int i = 0; i < G::IPW; i++) {
            const int reg = w * G::IPW + i;
            long grow = (long)kt * 64 + reg + G::NREG * slot;
            grow = grow < p.n ? grow : p.n - 1;
            __builtin_amdgcn_global_load_lds((gbl_void*)(kbase + grow * p.k_tok * 2 + chunk * 16), (lds_void*)(buf + reg * G::KRS), 16, 0, 0);
            __builtin_amdgcn_global_load_lds((gbl_void*)(vbase + grow * p.v_tok * 2 + chunk * 16), (lds_void*)(buf + G::KTILEB + reg * G::VRS), 16, 0, 0);
        }
        if (w < 3) {
            long gk = (long)kt * 64 + lane;
            gk = gk < p.n ? gk : p.n - 1;
            const int* src = (w == 0 ? p.art : w == 1 ? p.end : p.pos) + gk;
            __builtin_amdgcn_global_load_lds((gbl_void*)src, (lds_void*)(buf + G::KTILEB + G::VTILEB + w * 256), 4, 0, 0);
        }
    }
}

#ifndef SPINF_ABL
#define SPINF_ABL 0   // measurement builds only: 1 = no tile DMA after the first, 2 = no block compute
#endif
#ifdef SPINF_TRACE
__device__ long g_trace[16 * 16384];
extern "C" int spinf_debug_trace(long* out, int n) { return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_trace), sizeof(long) * n, 0, hipMemcpyDeviceToHost); }
#define TRACE(slot, val) do { if (threadIdx.x == 0 && blockIdx.x < 16384) g_trace[blockIdx.x * 16 + (slot)] = (val); } while (0)
#define PH_DECL long ph_t = 0, ph_acc[4] = {0, 0, 0, 0};
#define PH_START do { ph_t = clock64(); } while (0)
#define PH_MARK(k) do { const long ph_n = clock64(); ph_acc[k] += ph_n - ph_t; ph_t = ph_n; } while (0)
#else
#define TRACE(slot, val) do { } while (0)
#define PH_DECL
#define PH_START do { } while (0)
#define PH_MARK(k) do { } while (0)
#endif
constexpr int ENT_CAP = 256;   // plan entries of the current query tile kept in LDS at a time

// Softmax reference point.  The first pass over a query tile fixes each row's reference at the maximum of the first 32-key
// block in which the row sees a key and never rescales the accumulators: probabilities are exp2(t - ref) and stay below
// 2^TAU_FAST in fp32 / bf16 range.  If any row of the tile meets a score more than TAU_FAST above its reference, the
// whole tile is recomputed by the second, classic online-softmax pass (reference raised, accumulators rescaled, whenever a
// block maximum exceeds it by more than TAU_LAZY).  Which pass produced a row depends on the rows of its own 128-token tile
// only, so it does not depend on what the job is packed with.
constexpr float TAU_FAST = 60.f;
constexpr float TAU_LAZY = 8.f;

// One workgroup's whole job: load the query fragments, walk the tile's key list, normalise and store.  EXACT = false is the
// fast pass (returns true, without storing, when some row needs the exact pass); EXACT = true the classic online softmax.
template <int D, int RT, bool WIN, int KPF, int VPF, bool EXACT>
__device__ __forceinline__ bool attn_tile(const AttnParams& p, char* buf0, char* buf1, int2* ent) {
    using G = Geo<D>;
    constexpr int NS = D / 16;    // contraction steps of K Q^T
    constexpr int NDT = D / 32;   // 32-wide slices of the head dimension in O^T

    const int lane = threadIdx.x & 63, m = lane & 31, g = lane >> 5;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // consecutive workgroups go round-robin over the 8 XCDs; give every XCD a contiguous range of the
    // (head group major, job by job) work list so that the tiles sharing K/V meet in one L2
    const int L = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
    if (L >= p.total) return false;
    TRACE(0, (long)__builtin_amdgcn_s_memrealtime());
    TRACE(1, (long)clock64());
    const int hp = L / p.nqt;
    const int t = p.order[L - hp * p.nqt];
    const int h0 = hp * RT, kvh = h0 / p.group;
    const int tok = t * SPINF_QTILE + 32 * w + m;
    const int tok_c = tok < p.n ? tok : p.n - 1;

    // per-lane part of the DMA source addresses (bytes): row slot of the region and 16-byte chunk
    const unsigned lane_k = (unsigned)((lane / G::CPR) * G::NREG * p.k_tok * 2 + (lane % G::CPR) * 16);
    const unsigned lane_v = (unsigned)((lane / G::CPR) * G::NREG * p.v_tok * 2 + (lane % G::CPR) * 16);

    const int e0 = p.qt_ptr[t], e1 = p.qt_ptr[t + 1];
    const int ne = e1 - e0;

    bf16x8 qf[RT][NS];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const __bf16* qp = p.q + (long)tok_c * p.q_tok + (long)(h0 + rt) * p.q_head + 8 * g;
#pragma unroll
        for (int s = 0; s < NS; s++) qf[rt][s] = *(const bf16x8*)(qp + 16 * s);
    }
    const int art_q = tok < p.n ? p.art[tok_c] : -1;
    const int pos_q = WIN ? p.pos[tok_c] : 0;

    f32x16 o[RT][NDT];
    float M[RT], l[RT];
    bool viol = false;
    PH_DECL

    // lane parts of the LDS addresses.  K fragment: row m of the 32-key block, 16-byte chunk g of each 32-byte step.
    // V^T fragment (ds_read_b64_tr_b16): inside its 16-lane group a lane supplies the address of key row 4g + tr_j,
    // head dims 16 tr_mb + 4 tr_a .. +3 of the 32-wide slice, and receives head dim lane%32 of 4 consecutive keys.
    const int tr_a = lane & 3, tr_j = (lane >> 2) & 3, tr_mb = (lane >> 4) & 1;
    const int k_lane = G::k_off(m) + 16 * g;
    const int v_lane = G::v_off(4 * g + tr_j) + 32 * tr_mb + 8 * tr_a;

    // ---- one 32-key block of the current tile against this wave's 32 query rows (x RT heads)
    auto block = [&](const char* kb, const char* vb, const int* meta, const int kt, const int sub, const bool needmask)
                     __attribute__((always_inline)) {
        // rows 32 sub .. 32 sub + 31 of the tile sit in region slot(s) sub * 32 / NREG: a runtime byte offset
        const char* krow = kb + k_lane + sub * (32 / G::NREG) * G::ROWB;
        const char* vrow = vb + v_lane + sub * (32 / G::NREG) * G::ROWB;

        // S^T = K Q^T : rows = 32 keys, columns = this wave's 32 query rows; K fragments run PF reads ahead of the MFMAs
        f32x16 s_acc[RT];
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int i2 = 0; i2 < 16; i2++) s_acc[rt][i2] = 0.f;
        {
            constexpr int PF = KPF < NS ? KPF : NS;
            bf16x8 kf[PF];
#pragma unroll
            for (int s = 0; s < PF; s++) kf[s] = *(const bf16x8*)(krow + 32 * s);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int s = 0; s < NS; s++) {
#pragma unroll
                for (int rt = 0; rt < RT; rt++)
                    s_acc[rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s % PF], qf[rt][s], s_acc[rt], 0, 0, 0);
                if (s + PF < NS) kf[s % PF] = *(const bf16x8*)(krow + 32 * (s + PF));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        PH_MARK(1);
        // V^T fragments (fragment f = 16-key half f / NDT, head-dim slice f % NDT): the first VPF are in flight while the
        // softmax runs, the rest replace them as they are consumed
        constexpr int NVF = 2 * NDT;
        constexpr int VPF_ = VPF < NVF ? VPF : NVF;
        s16x4 vlo[VPF_], vhi[VPF_];
        auto vload = [&](const int f, const int slot) __attribute__((always_inline)) {
            const char* vp = vrow + G::v_off(16 * (f / NDT)) + 64 * (f % NDT);
            vlo[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)vp);
            vhi[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vp + G::v_off(8)));
        };
#pragma unroll
        for (int f = 0; f < VPF_; f++) vload(f, f);
        __builtin_amdgcn_sched_barrier(0);

        // mask (register i of the result holds key 8*(i/4) + 4g + i%4 of the block)
        if (needmask) {
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                const int ko = 32 * sub + 8 * i4 + 4 * g;
                const int4 ka = *(const int4*)(meta + ko);
                const int4 ke = *(const int4*)(meta + 64 + ko);
                int4 kp = make_int4(0, 0, 0, 0);
                if (WIN) kp = *(const int4*)(meta + 128 + ko);
                const int kg = kt * 64 + ko;
                const int kav[4] = {ka.x, ka.y, ka.z, ka.w};
                const int kev[4] = {ke.x, ke.y, ke.z, ke.w};
                const int kpv[4] = {kp.x, kp.y, kp.z, kp.w};
#pragma unroll
                for (int jj = 0; jj < 4; jj++) {
                    const int kk = kg + jj;
                    bool vis = (kk <= tok) & (art_q >= 0) & (kav[jj] == art_q) & (tok < kev[jj]);
                    vis = vis | (kk == tok);
                    if (WIN) vis = vis & ((pos_q - kpv[jj]) < p.window);
#pragma unroll
                    for (int rt = 0; rt < RT; rt++) s_acc[rt][4 * i4 + jj] = vis ? s_acc[rt][4 * i4 + jj] : -INFINITY;
                }
            }
        }

        // softmax numerators, one query row per lane pair (lane, lane^32)
        bf16x8 pb[RT][2];
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            float mx = s_acc[rt][0];
#pragma unroll
            for (int i2 = 1; i2 < 16; i2++) mx = fmaxf(mx, s_acc[rt][i2]);
            mx = lane32_max(mx);
            const float tm = mx * p.c;
            if (EXACT) {
                const bool up = tm > M[rt] + TAU_LAZY;
                const float mn = up ? tm : M[rt];
                const float alpha = up ? __builtin_amdgcn_exp2f(M[rt] - mn) : 1.0f;
                if (__builtin_amdgcn_ballot_w64(up && M[rt] != -INFINITY) != 0) {   // rows without a key so far hold zeros
#pragma unroll
                    for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                        for (int i2 = 0; i2 < 16; i2++) o[rt][dt][i2] *= alpha;
                }
                l[rt] *= alpha;
                M[rt] = mn;
            } else {
                const bool first = M[rt] == -INFINITY;
                viol = viol | (!first & (tm > M[rt] + TAU_FAST));
                M[rt] = first ? tm : M[rt];
            }
            const float ms = M[rt] == -INFINITY ? 0.f : M[rt];
            float sum = 0.f;
            float pv[16];
#pragma unroll
            for (int i2 = 0; i2 < 16; i2++) {
                pv[i2] = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[rt][i2], p.c, -ms));
                sum += pv[i2];
            }
            l[rt] += sum;
#pragma unroll
            for (int i2 = 0; i2 < 8; i2++) {
                pb[rt][0][i2] = (__bf16)pv[i2];
                pb[rt][1][i2] = (__bf16)pv[8 + i2];
            }
        }
        __builtin_amdgcn_sched_barrier(0);

        PH_MARK(2);
        // O^T += V^T P^T : rows = 32 head dims, columns = query rows, contraction = 16 keys per MFMA
#pragma unroll
        for (int f = 0; f < NVF; f++) {
            const s16x8 av = __builtin_shufflevector(vlo[f % VPF_], vhi[f % VPF_], 0, 1, 2, 3, 4, 5, 6, 7);
            const bf16x8 a = __builtin_bit_cast(bf16x8, av);
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
                o[rt][f % NDT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[rt][f / NDT], o[rt][f % NDT], 0, 0, 0);
            if (f + VPF_ < NVF) vload(f + VPF_, f % VPF_);
            __builtin_amdgcn_sched_barrier(0);
        }
        PH_MARK(3);
    };

    // ---- one pass over the tile's key list
    {
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            M[rt] = -INFINITY;
            l[rt] = 0.f;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i2 = 0; i2 < 16; i2++) o[rt][dt][i2] = 0.f;
        }
        int base = 0;
        __syncthreads();   // nobody still reads the entry window or the buffers of the fast pass
        if ((int)threadIdx.x < ne) ent[threadIdx.x] = make_int2(p.kv_idx[e0 + threadIdx.x], (int)p.kv_bits[e0 + threadIdx.x]);
        __syncthreads();
        if (ne > 0) issue_tile<D>(p, buf0, __builtin_amdgcn_readfirstlane(ent[0].x), kvh, w, lane, lane_k, lane_v);
        TRACE(2, (long)clock64());
        PH_START;
        auto step = [&](char* buf, char* nxt, const int i) __attribute__((always_inline)) {
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's DMA into buf has landed
            __syncthreads();                     // ... and everyone's; the other buffer is free again
            if (i + 1 - base >= ENT_CAP) {       // slide the window of plan entries (uniform; rare)
                base = i;
                if (i + (int)threadIdx.x < ne) ent[threadIdx.x] = make_int2(p.kv_idx[e0 + i + threadIdx.x], (int)p.kv_bits[e0 + i + threadIdx.x]);
                __syncthreads();
            }
#if SPINF_ABL != 1
            if (i + 1 < ne) issue_tile<D>(p, nxt, __builtin_amdgcn_readfirstlane(ent[i + 1 - base].x), kvh, w, lane, lane_k, lane_v);
#endif
            const int2 en = ent[i - base];
            const int kt = __builtin_amdgcn_readfirstlane(en.x);
            const unsigned bits = (unsigned)__builtin_amdgcn_readfirstlane(en.y) >> (2 * w);
            const char* kb = buf;
            const char* vb = buf + G::KTILEB;
            const int* meta = (const int*)(buf + G::KTILEB + G::VTILEB);
            PH_MARK(0);
#pragma unroll 1
            for (int sub = 0; sub < 2; sub++) {
                if (!((bits >> sub) & 1u)) continue;   // wave-uniform: no row of this wave sees these 32 keys
#if SPINF_ABL != 2
                block(kb, vb, meta, kt, sub, (bits >> (8 + sub)) & 1u);
#endif
            }
        };
        for (int i = 0; i < ne; i += 2) {
            step(buf0, buf1, i);
            if (i + 1 < ne) step(buf1, buf0, i + 1);
        }
    }
    TRACE(3, (long)clock64());
    TRACE(6, (long)ne);
    if (!EXACT && __syncthreads_or(viol)) return true;

    // ---- epilogue: normalise, transpose through LDS and store whole rows.  Register i of O^T[dt] is head dim
    // 32dt + 8(i/4) + 4g + i%4 of row `tok`; each wave stages its 32 rows in its own slice of the (now idle) tile buffers
    // and writes them out as 16-byte pieces, 32 lanes per row.
    __syncthreads();   // every wave is done with the tile buffers
    {
        constexpr int SROW = G::ROWB + 16;
        static_assert(2 * 32 * SROW <= G::BUFB, "output staging must fit the tile buffers");
        char* stage = ((w & 2) ? buf1 : buf0) + (w & 1) * 32 * SROW;
        const int tok0 = t * SPINF_QTILE + 32 * w;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            const float inv = 1.0f / lane32_sum(l[rt]);
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    bf16x4 r;
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) r[jj] = (__bf16)(o[rt][dt][4 * i4 + jj] * inv);
                    *(bf16x4*)(stage + m * SROW + (32 * dt + 8 * i4 + 4 * g) * 2) = r;
                }
            __bf16* ob = p.o + (long)(h0 + rt) * p.o_head;
#pragma unroll
            for (int j = 0; j < 32 * G::CPR / 64; j++) {
                const int c = j * 64 + lane, row = c / G::CPR, col = c % G::CPR;
                const bf16x8 val = *(const bf16x8*)(stage + row * SROW + col * 16);
                if (tok0 + row < p.n) *(bf16x8*)(ob + (long)(tok0 + row) * p.o_tok + col * 8) = val;
            }
        }
    }
    TRACE(4, (long)clock64());
    TRACE(5, (long)__builtin_amdgcn_s_memrealtime());
    {
        unsigned hwid;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hwid));
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        TRACE(7, (long)hwid | ((long)xcc << 32));
    }
#ifdef SPINF_TRACE
    if (threadIdx.x == 64 && blockIdx.x < 16384) {   // wave 1: time spent waiting (0), in K Q^T (1), softmax (2), P V (3)
        g_trace[blockIdx.x * 16 + 8] = ph_acc[0]; g_trace[blockIdx.x * 16 + 9] = ph_acc[1];
        g_trace[blockIdx.x * 16 + 10] = ph_acc[2]; g_trace[blockIdx.x * 16 + 11] = ph_acc[3];
    }
#endif
    return false;
}

// the exact pass lives in its own, never inlined function: its accumulator rescaling (vector ALU on all of O) would
// otherwise cost the fast pass its register allocation
template <int D, int RT, bool WIN, int KPF, int VPF>
__device__ __attribute__((noinline)) void attn_tile_exact(const AttnParams p, char* buf0, char* buf1, int2* ent) {   // by value: a reference would pin the kernel arguments in scratch
    (void)attn_tile<D, RT, WIN, KPF, VPF, true>(p, buf0, buf1, ent);
}

template <int D, int RT, bool WIN, int KPF, int VPF>
__global__ __launch_bounds__(256) void tree_attn_kernel(const AttnParams p) {
    using G = Geo<D>;
    // two tile buffers as DISTINCT LDS objects: the compiler then knows that the DMA writes into one of them cannot
    // alias the fragment reads of the other, and does not make those reads wait for the DMA
    __shared__ __attribute__((aligned(16))) char buf0[G::BUFB];
    __shared__ __attribute__((aligned(16))) char buf1[G::BUFB];
    __shared__ int2 ent[ENT_CAP];   // (key tile, bits) of plan entries base .. base + ENT_CAP - 1
    if (attn_tile<D, RT, WIN, KPF, VPF, false>(p, buf0, buf1, ent)) attn_tile_exact<D, RT, WIN, KPF, VPF>(p, buf0, buf1, ent);
}

template <int D, int RT, bool WIN>
static int launch(const AttnParams& p, hipStream_t stream) {
    using G = Geo<D>;
    static_assert(2 * G::BUFB + ENT_CAP * 8 <= 160 * 1024, "LDS budget");
    // fragment prefetch depths: at head dim 256 with two heads per wave the accumulators and query fragments take 416 of the
    // 512 registers, which leaves room for two fragments in flight; elsewhere eight
    constexpr int KPF = (D == 256 && RT == 2) ? 2 : 8;
    constexpr int VPF = (D == 256 && RT == 2) ? 2 : 8;
    hipLaunchKernelGGL((tree_attn_kernel<D, RT, WIN, KPF, VPF>), dim3(8 * p.per_xcd), dim3(256), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}

template <int D>
static int launch_d(const AttnParams& p, int rt, bool win, hipStream_t s) {
    if (rt == 2) return win ? launch<D, 2, true>(p, s) : launch<D, 2, false>(p, s);
    return win ? launch<D, 1, true>(p, s) : launch<D, 1, false>(p, s);
}

extern "C" int spinf_tree_attn_fwd(const spinf_attn_args* a, void* stream) {
    if (!a) return spinf_fail(SPINF_E_ARG, "tree_attn: null args");
    if (a->n <= 0 || a->n_qtiles <= 0) return SPINF_OK;
    if (!a->q || !a->k || !a->v || !a->out || !a->art || !a->end || !a->pos || !a->qt_ptr || !a->order)
        return spinf_fail(SPINF_E_ARG, "tree_attn: null pointer");
    if (a->d != 64 && a->d != 128 && a->d != 256) return spinf_fail(SPINF_E_ARG, "tree_attn: head dim %d not in {64,128,256}", a->d);
    if (a->hq <= 0 || a->hkv <= 0 || a->hq % a->hkv) return spinf_fail(SPINF_E_ARG, "tree_attn: hq %d not a multiple of hkv %d", a->hq, a->hkv);
    if (a->n > INT32_MAX / 2) return spinf_fail(SPINF_E_ARG, "tree_attn: stream too long");
    if (a->n_qtiles != (a->n + SPINF_QTILE - 1) / SPINF_QTILE) return spinf_fail(SPINF_E_ARG, "tree_attn: plan has %lld query tiles, stream needs %lld", (long long)a->n_qtiles, (long long)((a->n + SPINF_QTILE - 1) / SPINF_QTILE));
    if (!(a->scale > 0.f)) return spinf_fail(SPINF_E_ARG, "tree_attn: scale must be positive");
    const int64_t strides[8] = {a->q_tok, a->q_head, a->k_tok, a->k_head, a->v_tok, a->v_head, a->o_tok, a->o_head};
    for (int i = 0; i < 8; i++)
        if (strides[i] % 8) return spinf_fail(SPINF_E_ARG, "tree_attn: strides must be multiples of 8 elements");
    const uintptr_t ptrs[4] = {(uintptr_t)a->q, (uintptr_t)a->k, (uintptr_t)a->v, (uintptr_t)a->out};
    for (int i = 0; i < 4; i++)
        if (ptrs[i] % 16) return spinf_fail(SPINF_E_ARG, "tree_attn: tensors must be 16-byte aligned");
    const int group = a->hq / a->hkv;
    // two heads of a GQA group per wave halve the LDS traffic per MFMA; at head dim 256 their accumulators and query
    // fragments (384 registers) leave too little room, so that size runs one head per wave
    int rt = (group % 2 == 0 && a->d <= 128) ? 2 : 1;
    if (a->variant == 1) rt = 1;
    if (a->variant == 2 && group % 2 == 0) rt = 2;
    AttnParams p;
    p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v; p.o = (__bf16*)a->out;
    p.q_tok = a->q_tok; p.q_head = a->q_head; p.k_tok = a->k_tok; p.k_head = a->k_head;
    p.v_tok = a->v_tok; p.v_head = a->v_head; p.o_tok = a->o_tok; p.o_head = a->o_head;
    p.n = (int)a->n; p.group = group;
    p.c = a->scale * 1.4426950408889634f;
    p.window = a->window > 0 ? a->window : 0;
    p.art = a->art; p.end = a->end; p.pos = a->pos;
    p.qt_ptr = a->qt_ptr; p.kv_idx = a->kv_idx; p.kv_bits = a->kv_bits; p.order = a->order;
    p.nqt = (int)a->n_qtiles;
    const int64_t total = a->n_qtiles * (a->hq / rt);
    if (total > INT32_MAX / 2) return spinf_fail(SPINF_E_ARG, "tree_attn: too many work items");
    p.total = (int)total;
    p.per_xcd = (int)((total + 7) / 8);
    const bool win = p.window > 0;
    hipStream_t s = (hipStream_t)stream;
    switch (a->d) {
        case 64: return launch_d<64>(p, rt, win, s);
        case 128: return launch_d<128>(p, rt, win, s);
        default: return launch_d<256>(p, rt, win, s);
    }
}
