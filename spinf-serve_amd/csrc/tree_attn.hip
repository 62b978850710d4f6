// Tree-mask packed-prefill attention for gfx950 (MI355X): flash-style forward over a per-query-tile list of key tiles.
//
// Replaces the flex_attention call of spinf_serve/models/gemma4.py:107-118 and spinf_serve/models/qwen35/qwen.py:614,620;
// the per-element visibility test is the predicate of spinf_serve/scorer.py:173-177.
//
// Work decomposition.  A work item = one 128-token query tile x the heads of one GQA group that share it: RT heads per
// wave times NHW head sets across waves.  The default for an even group is RT = 1, NHW = 2: eight waves, wave w owns
// 32 tokens of head w/4 (row group w%4 for the first head, 3 - w%4 for the second), two waves per SIMD on the same K / V tiles, so that one wave's softmax runs under
// the other's MFMAs.  (NHW = 1 are the four-wave kernels: one head per wave for odd groups, or RT = 2 heads per wave at
// head dim <= 128, where a K or V fragment read from LDS feeds two MFMAs.)  Scores are computed transposed, S^T = K Q^T, with
// v_mfma_f32_32x32x16_bf16: a lane then owns ONE query row (column lane%32 of the 32x32 result) and 16 of the 32 keys,
// so the softmax row reductions are in-lane plus one exchange with lane^32.  O^T = V^T P^T reuses the score registers
// as the B operand without any shuffle; V^T fragments come from row-major V in LDS through ds_read_b64_tr_b16.
//
// Persistent workgroups.  One workgroup per CU pulls work items from eight lists (one per XCD, so that the tiles sharing
// K/V meet in one L2; a workgroup that exhausts its list continues with the next one).  While an item is computed the
// next item's descriptor, plan entries and query fragments are fetched, and the K/V tile pipeline runs straight across
// the item boundary, so the fixed cost of an item is its epilogue only.
//
// K/V tiles (64 keys) are copied global -> LDS by the DMA path (global_load_lds_dwordx4), double-buffered, in a padded
// layout that keeps both the b128 reads of K and the transposing reads of V free of bank conflicts.  The key tile's
// art/end/pos ride along so that masked blocks never touch global memory in the loop.
//
// Reduction order.  A row's keys are visited in ascending 32-key blocks that depend only on the row's own job (jobs start
// on 128-token boundaries), masked entries contribute exact zeros, and a skipped block equals a fully masked one bit for
// bit; the softmax reference point of a row is taken from that row's scores only.  A job's output is therefore
// bit-identical whatever it is packed with, and whichever workgroup happens to compute it.
#include <hip/hip_runtime.h>

#include <mutex>
#include <vector>

#include "spinf_tree.h"
#include "common.h"

#include "attn_tiles.h"
#include "attn_kernels.h"

// normalise O^T and store it as rows: each wave stages 32 rows x 64 head dims at a time in its own LDS slice (144-byte
// rows) and writes them out as 16-byte pieces, 8 lanes per 128-byte row segment
template <int D, int RT, bool ROWS = false, class LaneT>
__device__ __forceinline__ void store_rows(const AttnParams& p, const LaneT& L, char* stage, const f32x16 (&o)[RT][D / 32], const float (&l)[RT],
                                           int t, int h0) {
    constexpr int NDT = D / 32;
    constexpr int SROW = 128 + 16;
    const int tok0 = t * SPINF_QTILE + 32 * L.wr;
    const int lane = fresh_lane_id(), m = lane & 31, g = lane >> 5;
    int orow[4] = {0, 0, 0, 0};   // compact rows: row of the four tokens this lane stores pieces of, -1 for a pad position
    if (ROWS) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int tok = tok0 + ((j * 64 + lane) >> 3);
            orow[j] = tok < p.n ? p.row_of[tok] : -1;
        }
    }
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const float inv = 1.0f / lane32_sum(l[rt]);
        __bf16* ob = p.o + (long)(h0 + rt) * p.o_head;
#pragma unroll
        for (int qd = 0; qd < NDT / 2; qd++) {
#pragma unroll
            for (int dd = 0; dd < 2; dd++)
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    bf16x4 r;
#pragma unroll
                    for (int jj = 0; jj < 4; jj++) r[jj] = (__bf16)(o[rt][2 * qd + dd][4 * i4 + jj] * inv);
                    *(bf16x4*)(stage + m * SROW + (32 * dd + 8 * i4 + 4 * g) * 2) = r;
                }
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int c = j * 64 + lane, row = c >> 3, col = c & 7;
                const bf16x8 val = *(const bf16x8*)(stage + row * SROW + col * 16);
                if (ROWS) {
                    if (orow[j] >= 0) *(bf16x8*)(ob + (long)orow[j] * p.o_tok + 64 * qd + col * 8) = val;
                } else {
                    if (tok0 + row < p.n) *(bf16x8*)(ob + (long)(tok0 + row) * p.o_tok + 64 * qd + col * 8) = val;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------ exact pass
// Classic online softmax over one work item, one 32-key block at a time, nothing overlapped: the rare fallback, in a
// kernel of its own because its accumulator rescaling (vector ALU on all of O) would cost the fast pass its register
// allocation.
template <int D, int RT, bool WIN, bool ROWS, int GRP, int TK, int DV>
__device__ __forceinline__ void attn_item_exact(const AttnParams& p, const int4 item, const int h0, char* buf0, int2* ent, int* ent_row0, char* stage) {
    using G = TileGeo<D, TK, DV>;
    constexpr int NS = D / 16, NDT = DV / 32;
    const Lane<D, TK, DV> L(p);
    const int t = item.x, e0 = item.y, ne = item.z & 0xfffff;   // heads h0 .. h0 + RT - 1 of the item
    const int kvh = h0 / p.group;
    const int tok = t * SPINF_QTILE + 32 * L.w + L.m;
    const int tok_c = tok < p.n ? tok : p.n - 1;
    int q_row = tok_c;
    if (ROWS) {   // a pad position has no row: it computes on some row's queries and stores nothing
        q_row = p.row_of[tok_c];
        q_row = q_row < 0 ? 0 : q_row;
    }
    bf16x8 qf[RT][NS];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const __bf16* qp = p.q + (long)q_row * p.q_tok + (long)(h0 + rt) * p.q_head + 8 * L.g;
#pragma unroll
        for (int s = 0; s < NS; s++) qf[rt][s] = *(const bf16x8*)(qp + 16 * s);
    }
    const int art_q = tok < p.n ? p.art[tok_c] : -1;
    const int pos_q = WIN ? p.pos[tok_c] : 0;
    const int grp_q = GRP && tok < p.n ? p.grp[tok_c] : -1;
    f32x16 o[RT][NDT];
    float M[RT], l[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        M[rt] = -INFINITY;
        l[rt] = 0.f;
#pragma unroll
        for (int dt = 0; dt < NDT; dt++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[rt][dt][i] = 0.f;
    }
    int base = 0;
    __syncthreads();
    if ((int)threadIdx.x < ne) {
        ent[threadIdx.x] = make_int2(p.kv_idx[e0 + threadIdx.x], (int)p.kv_bits[e0 + threadIdx.x]);
        if (ROWS) ent_row0[threadIdx.x] = p.kv_row0[e0 + threadIdx.x];
    }
    __syncthreads();
    for (int i = 0; i < ne; i++) {
        if (i - base >= ENT_CAP) {
            __syncthreads();
            base = i;
            if (i + (int)threadIdx.x < ne) {
                ent[threadIdx.x] = make_int2(p.kv_idx[e0 + i + threadIdx.x], (int)p.kv_bits[e0 + i + threadIdx.x]);
                if (ROWS) ent_row0[threadIdx.x] = p.kv_row0[e0 + i + threadIdx.x];
            }
            __syncthreads();
        }
        const int2 en = ent[i - base];
        const int kt = __builtin_amdgcn_readfirstlane(en.x);
        const unsigned bits = (unsigned)__builtin_amdgcn_readfirstlane(en.y) >> (2 * L.w);
        const int row0 = ROWS ? __builtin_amdgcn_readfirstlane(ent_row0[i - base]) : 0;
        __syncthreads();   // everyone is done with the buffer
        issue_tile<D, 4, ROWS, GRP, TK, DV>(p, lds_addr(buf0), kt, row0, kvh, L.w, L.lane, L.lane_k, L.lane_v);
        __builtin_amdgcn_s_waitcnt(0x0f70);
        __syncthreads();
        const char* kb = buf0;
        const char* vb = buf0 + G::KTILEB;
        const int* meta = (const int*)(buf0 + G::KTILEB + G::VTILEB);
#pragma unroll 1
        for (int sub = 0; sub < TK / 32; sub++) {
            if (!((bits >> sub) & 1u)) continue;
            const char* krow = kb + L.k_lane + sub * G::KSUB;
            const char* vrow = vb + L.v_lane + sub * G::VSUB;
            f32x16 s_acc[RT];
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
#pragma unroll
                for (int i2 = 0; i2 < 16; i2++) s_acc[rt][i2] = 0.f;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const bf16x8 kf = *(const bf16x8*)(krow + 32 * s);
#pragma unroll
                for (int rt = 0; rt < RT; rt++) s_acc[rt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[rt][s], s_acc[rt], 0, 0, 0);
            }
            if ((bits >> (8 + sub)) & 1u) apply_mask<RT, WIN, GRP, TK>(s_acc, meta, kt, sub, L.g, tok, art_q, pos_q, p.window, grp_q);
            bf16x8 pb[RT][2];
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                float mx = s_acc[rt][0];
#pragma unroll
                for (int i2 = 1; i2 < 16; i2++) mx = fmaxf(mx, s_acc[rt][i2]);
                mx = lane32_max(mx);
                const float tm = mx * p.c;
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
                const float ms = mn == -INFINITY ? 0.f : mn;
                float sum = 0.f;
#pragma unroll
                for (int i2 = 0; i2 < 16; i2++) {
                    const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[rt][i2], p.c, -ms));
                    sum += pr;
                    pb[rt][i2 >> 3][i2 & 7] = (__bf16)pr;
                }
                l[rt] += sum;
            }
            // (no 16-byte read of K or of the keys' metadata in flight when the transposing reads of V begin: the two kinds do not
            // complete in the order they were issued, which the compiler's counting of outstanding LDS operations assumes)
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int f = 0; f < 2 * NDT; f++) {
                const char* vp = vrow + G::V::v_off(16 * (f / NDT)) + 64 * (f % NDT);
                const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)vp);
                const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vp + G::V::v_off(8)));
                const bf16x8 a = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
                for (int rt = 0; rt < RT; rt++) o[rt][f % NDT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[rt][f / NDT], o[rt][f % NDT], 0, 0, 0);
            }
        }
    }
    store_rows<DV, RT, ROWS>(p, L, stage, o, l, t, h0);
}

// An item of HPI heads is recomputed RT heads at a time.
template <int D, int RT, bool WIN, int HPI, bool ROWS, int GRP, int TK = 64, int DV = D>
__global__ __launch_bounds__(256) void tree_attn_exact_kernel(const AttnParams p) {
    using G = TileGeo<D, TK, DV>;
    __shared__ __attribute__((aligned(16))) char buf0[G::BUFB];
    __shared__ int2 ent[ENT_CAP];
    __shared__ int ent_row0[ROWS ? ENT_CAP : 1];
    __shared__ __attribute__((aligned(16))) char stage_all[4 * 32 * 144];
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_redo = p.counters[NLIST + 1];
    // the fast pass is over (stream order): its list cursors and its count of finished workgroups go back to zero for the block's next call
    if (blockIdx.x == 0 && threadIdx.x <= NLIST) p.counters[threadIdx.x] = 0;
    if (n_redo == 0) return;   // the normal case: the fast pass handed nothing on (every workgroup reads the same count)
    for (int j = blockIdx.x; j < n_redo; j += gridDim.x) {
        const int4 it = p.items[p.redo[j]];
        const int4 item = make_int4(__builtin_amdgcn_readfirstlane(it.x), __builtin_amdgcn_readfirstlane(it.y),
                                    __builtin_amdgcn_readfirstlane(it.z), __builtin_amdgcn_readfirstlane(it.w));
        const int hp = (int)((unsigned)item.z >> 20);
        for (int sub = 0; sub < HPI; sub += RT) attn_item_exact<D, RT, WIN, ROWS, GRP, TK, DV>(p, item, hp * HPI + sub, buf0, ent, ent_row0, stage_all + w * 32 * 144);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    if (threadIdx.x == 0) {
        __threadfence();
        if (atomicAdd(&p.counters[NLIST + 2], 1) == (int)gridDim.x - 1) {
            atomicAdd(&p.counters[NLIST + 3], n_redo);   // running total, for spinf_attn_exact_items
            p.counters[NLIST + 1] = 0;
            p.counters[NLIST + 2] = 0;
            __threadfence();
        }
    }
}

// ------------------------------------------------------------------------------------------------ fast pass, persistent
// NHW = 1: four waves, each with RT heads of the item.  NHW = 2: eight waves, waves 4..7 take the item's second set of RT heads
// on the same K / V tiles (two waves per SIMD: one wave's softmax runs under the other's MFMAs).
// ROWS: q, k, v, o hold the real tokens only (compact rows); the stream positions of the plan are mapped through row_of.
// GRP: image groups (1: their tokens see each other whatever the window, 2: within the window).
template <int D, int RT, bool WIN, int NHW, bool ROWS, int GRP, int TK = 64, int DV = D>
__global__ __launch_bounds__(256 * NHW) void tree_attn_kernel(const AttnParams p) {
    using G = TileGeo<D, TK, DV>;
    constexpr int HPI = RT * NHW;  // heads per work item
    constexpr int NS = D / 16;     // contraction steps of K Q^T
    constexpr int NDT = DV / 32;   // 32-wide slices of the (value) head dimension in O^T
    constexpr int NVF = 2 * NDT;   // V^T fragments of one 32-key block
    // fragment read-ahead depth: the register file is the tight one at head dim 256 (4 with one wave per SIMD, 3 with two:
    // measured 0.374 / 0.351 / 0.343 / 0.368 ms on the 24-content pass for depths 4 / 2 / 3 / 1); no effect at 128
    constexpr int PFD = D >= 256 ? (NHW == 2 ? 3 : 4) : 8;
    constexpr int PF = NS < PFD ? NS : PFD;     // K fragments read ahead of the MFMAs
    constexpr int VPF = NVF < PFD ? NVF : PFD;  // V^T fragments read ahead
    __shared__ __attribute__((aligned(16))) char bufs[2 * G::BUFB];   // the two tile buffers
    __shared__ int2 ent_a[ENT_CAP];   // (key tile, bits) of the current item's plan entries base .. base + ENT_CAP - 1
    __shared__ int2 ent_b[ENT_CAP];   // first entries of the next item
    __shared__ int entr_a[ROWS ? ENT_CAP : 1];   // compact rows: first row of each entry's key tile, alongside ent_a / ent_b
    __shared__ int entr_b[ROWS ? ENT_CAP : 1];
    // output staging, one slice per wave; with eight waves at head dim 256 there is no room left for it and the slices lie in
    // the tile buffer the item's last tile was computed from (free from the barrier after the tile loop until the next
    // item's first tile step requests a tile into it, which comes after that step's barrier)
    constexpr bool STAGE_IN_TILE = NHW == 2 && D == 256;
    static_assert(!STAGE_IN_TILE || 4 * NHW * 32 * 144 <= G::BUFB, "the staging slices must fit a tile buffer");
    __shared__ __attribute__((aligned(16))) char stage_all[STAGE_IN_TILE ? 16 : 4 * NHW * 32 * 144];
    __shared__ int s_next[2];         // item grabbed by thread 0 for the whole workgroup, double buffered

    const Lane<D, TK, DV> L(p);
    char* const stage_own = stage_all + (STAGE_IN_TILE ? 0 : L.w * 32 * 144);

    // ---- work lists: start with the list of this workgroup's XCD, continue with the following ones
    unsigned xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    int my_list = (int)(xcc & 7u), lists_done = 0;    // thread 0 only
    int own_next = p.static_lists ? p.list_ptr[blockIdx.x] : 0;   // static schedule: this workgroup's own list, in order, nobody else's
    auto grab = [&](const int slot) __attribute__((always_inline)) {   // thread 0: next item index into s_next[slot], -1 when all lists are empty
        if (threadIdx.x == 0) {
            int idx = -1;
            if (p.static_lists) {
                if (own_next < p.list_ptr[blockIdx.x + 1]) idx = own_next++;
                lists_done = NLIST;
            }
            while (lists_done < NLIST) {
                const int lo = p.list_ptr[my_list], hi = p.list_ptr[my_list + 1];
                const int j = lo + atomicAdd(&p.counters[my_list], 1);
                if (j < hi) { idx = j; break; }
                my_list = (my_list + 1) & (NLIST - 1);
                lists_done++;
            }
            s_next[slot] = idx;
        }
    };

    // ---- per-item state
    int4 cur = make_int4(0, 0, 0, 0), nxt = make_int4(0, 0, 0, 0);
    int cur_idx = -1, nxt_idx = -1;
    bool cur_ok = false, nxt_ok = false;
    bf16x8 qf[RT][NS];
    int art_q = -1, pos_q = 0, grp_q = -1;
    f32x16 o[RT][NDT];
    float M[RT], l[RT];
    bool viol = false;
    int2* ent_cur = ent_a;
    int2* ent_nxt = ent_b;
    int* entr_cur = entr_a;
    int* entr_nxt = entr_b;
    int nxt_row0 = 0;   // compact rows: first row of the next item's first key tile

    auto uniform4 = [](const int4 v) __attribute__((always_inline)) {   // the same value in every lane: keep it in scalar registers
        return make_int4(__builtin_amdgcn_readfirstlane(v.x), __builtin_amdgcn_readfirstlane(v.y), __builtin_amdgcn_readfirstlane(v.z),
                         __builtin_amdgcn_readfirstlane(v.w));
    };
    auto item_t = [](const int4& it) { return it.x; };
    auto item_ne = [](const int4& it) { return it.z & 0xfffff; };
    auto item_hp = [](const int4& it) { return (int)((unsigned)it.z >> 20); };

    auto load_q = [&](const int4& it, bf16x8 (&dst)[RT][NS], int& a_q, int& p_q, int& g_q) __attribute__((always_inline)) {
        const int lane = fresh_lane_id();
        const int tok = item_t(it) * SPINF_QTILE + 32 * L.wr + (lane & 31);
        const int tok_c = tok < p.n ? tok : p.n - 1;
        const int h0 = item_hp(it) * HPI + L.wh * RT;
        int q_row = tok_c;
        if (ROWS) {   // a pad position has no row: it computes on some row's queries and stores nothing
            q_row = p.row_of[tok_c];
            q_row = q_row < 0 ? 0 : q_row;
        }
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            const __bf16* qp = p.q + (long)q_row * p.q_tok + (long)(h0 + rt) * p.q_head + 8 * (lane >> 5);
#pragma unroll
            for (int s = 0; s < NS; s++) dst[rt][s] = *(const bf16x8*)(qp + 16 * s);
        }
        a_q = tok < p.n ? p.art[tok_c] : -1;
        p_q = WIN ? p.pos[tok_c] : 0;
        g_q = GRP && tok < p.n ? p.grp[tok_c] : -1;
    };
    auto load_ent = [&](const int4& it, int2* dst, int* dst_row0, const int from) __attribute__((always_inline)) {
        const int ne = item_ne(it);
        if ((int)threadIdx.x < ENT_CAP && from + (int)threadIdx.x < ne) {
            dst[threadIdx.x] = make_int2(p.kv_idx[it.y + from + threadIdx.x], (int)p.kv_bits[it.y + from + threadIdx.x]);
            if (ROWS) dst_row0[threadIdx.x] = p.kv_row0[it.y + from + threadIdx.x];
        }
    };
    auto reset_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            M[rt] = -INFINITY;
            l[rt] = 0.f;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[rt][dt][i] = 0.f;
        }
        viol = false;
    };

    // ---- compute pieces
    auto sm_head = [&](const int rt, const f32x16& sv) __attribute__((always_inline)) -> float {
        // the block's maximum is needed only where a row meets its first keys (it becomes the row's reference): in the steady state
        // no row of the wave does, and the 16 maxima and the lane exchange are skipped.  Whether a score lies too far above the
        // reference shows in the probabilities (the caller checks their sum against 2^TAU_FAST).
        const bool first = M[rt] == -INFINITY;
        if (__builtin_amdgcn_ballot_w64(first) != 0) {
            float mx = sv[0];
#pragma unroll
            for (int i2 = 1; i2 < 16; i2++) mx = fmaxf(mx, sv[i2]);
            mx = lane32_max(mx);
            M[rt] = first ? mx * p.c : M[rt];
        }
        return M[rt] == -INFINITY ? 0.f : M[rt];
    };
    auto sm_elem = [&](const f32x16& sv, const int i2, const float ms, float& sum, bf16x8 (&pb)[2]) __attribute__((always_inline)) {
        const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(sv[i2], p.c, -ms));
        sum += pr;
        pb[i2 >> 3][i2 & 7] = (__bf16)pr;
    };
    // S^T = K Q^T for one 32-key block
    auto qk_phase = [&](const char* krow, f32x16 (&s_acc)[RT]) __attribute__((always_inline)) {
#pragma unroll
        for (int rt = 0; rt < RT; rt++)
#pragma unroll
            for (int i2 = 0; i2 < 16; i2++) s_acc[rt][i2] = 0.f;
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
    };
    // O^T += V^T P^T for one 32-key block
    auto pv_phase = [&](const char* vrow, const bf16x8 (&pb)[RT][2]) __attribute__((always_inline)) {
        s16x4 vlo[VPF], vhi[VPF];
        auto vload = [&](const int f, const int slot) __attribute__((always_inline)) {
            const char* vp = vrow + G::V::v_off(16 * (f / NDT)) + 64 * (f % NDT);
            vlo[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)vp);
            vhi[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vp + G::V::v_off(8)));
        };
#pragma unroll
        for (int f = 0; f < VPF; f++) vload(f, f);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int f = 0; f < NVF; f++) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, __builtin_shufflevector(vlo[f % VPF], vhi[f % VPF], 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
            for (int rt = 0; rt < RT; rt++)
                o[rt][f % NDT] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[rt][f / NDT], o[rt][f % NDT], 0, 0, 0);
            if (f + VPF < NVF) vload(f + VPF, f % VPF);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto compute_tile = [&](const char* buf, const int kt, const unsigned bits) __attribute__((always_inline)) {
        const bool a0 = bits & 1u, a1 = bits & 2u;
        if (!a0 && !a1) return;   // wave-uniform: no row of this wave sees a key of the tile
        const char* kb = buf + L.k_lane;
        const char* vb = buf + G::KTILEB + L.v_lane;
        const int* meta = (const int*)(buf + G::KTILEB + G::VTILEB);
        const int tok = item_t(cur) * SPINF_QTILE + 32 * L.wr + L.m;
        // one 32-key block on its own: K Q^T, softmax, P V in sequence
        auto one_block = [&](const int sub) __attribute__((always_inline)) {
            f32x16 sa[RT];
            bf16x8 pa[RT][2];
            qk_phase(kb + sub * G::KSUB, sa);
            if ((bits >> (8 + sub)) & 1u) apply_mask<RT, WIN, GRP, TK>(sa, meta, kt, sub, L.g, tok, art_q, pos_q, p.window, grp_q);
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                const float ms = sm_head(rt, sa[rt]);
                float sum = 0.f;
#pragma unroll
                for (int i2 = 0; i2 < 16; i2++) sm_elem(sa[rt], i2, ms, sum, pa[rt]);
                l[rt] += sum;
                viol = viol | !(sum <= VIOL_SUM);   // (a NaN counts as too far as well)
            }
            pv_phase(vb + sub * G::VSUB, pa);
        };
        // (hiding each block's softmax behind the other block's MFMAs inside one wave was measured slower than plain
        // sequence: the second wave on the SIMD does that job)
        if (a0) one_block(0);
        if (TK > 32 && a1) one_block(1);
    };

    // ---- prologue: first item, its queries, entries and first tile; the second item is grabbed right away
    grab(0);
    __syncthreads();
    {
        cur_idx = __builtin_amdgcn_readfirstlane(s_next[0]);
        cur_ok = cur_idx >= 0;
        if (cur_ok) cur = uniform4(p.items[cur_idx]);
    }
    if (cur_ok) {
        load_q(cur, qf, art_q, pos_q, grp_q);
        load_ent(cur, ent_cur, entr_cur, 0);
        const int row0 = ROWS ? __builtin_amdgcn_readfirstlane(p.kv_row0[cur.y]) : 0;
        if (L.wh == 0) issue_tile<D, 4, ROWS, GRP, TK, DV>(p, lds_addr(bufs), cur.w, row0, item_hp(cur) * HPI / p.group, L.w, L.lane, L.lane_k, L.lane_v);
    }
    // The item after the current one is fetched from the lists as late as the prefetch pipeline allows (three tile steps
    // before the current item ends; at once for items shorter than that): an item fetched long before it starts keeps the
    // workgroup busy long after the lists have run dry, and the pass ends with the last workgroup.
    auto grab_step = [](const int ne) { return ne >= 4 ? ne - 3 : -1; };
    int gslot = 1;      // slot of s_next that holds the item after `cur`
    if (cur_ok && grab_step(item_ne(cur)) < 0) grab(1);
    int i = 0;          // tile step inside the current item
    int base = 0;       // first plan entry held in ent_cur
    int pstage = 0;     // next-item prefetch: 0 nothing, 1 descriptor known, 2 entries requested, 3 first tile requested

    // The tile DMA is issued by waves 0..3 alone: with eight waves they are the older wave of each SIMD, win the issue
    // arbitration and finish a tile step first, so the younger waves, which set the pace, are spared that work.
    // Item loop around a tile loop (two real loop levels on purpose: the accumulators are touched by the vector ALU only
    // outside the tile loop, so inside it they stay in the MFMA accumulator registers).
    // One tile step = one key tile of the current item from buffer `par`, the next tile (of this item or of the next one)
    // requested into the other buffer.
    int par = 0;
    while (cur_ok) {
        const int ne = item_ne(cur);
        const int kvh = item_hp(cur) * HPI / p.group;
        const int grab_at = grab_step(ne);
        reset_acc();
        base = 0;
        pstage = 0;
        nxt_ok = false;
        for (i = 0; i < ne; i++, par ^= 1) {
            const char* buf = bufs + par * G::BUFB;
            const unsigned oth = lds_addr(bufs + (par ^ 1) * G::BUFB);
            __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's DMA into buf (and its other loads) have landed
            __syncthreads();                     // ... and everyone's; the other buffer is free; s_next[gslot] is visible
            // next-item prefetch, one stage per step
            if (i < grab_at) {
            } else if (i == grab_at) {
                grab(gslot);
            } else if (pstage == 0) {
                nxt_idx = __builtin_amdgcn_readfirstlane(s_next[gslot]);
                nxt_ok = nxt_idx >= 0;
                if (nxt_ok) nxt = uniform4(p.items[nxt_idx]);
                if (ROWS && nxt_ok) nxt_row0 = __builtin_amdgcn_readfirstlane(p.kv_row0[nxt.y]);
                pstage = 1;
            } else if (pstage == 1) {
                if (nxt_ok) load_ent(nxt, ent_nxt, entr_nxt, 0);
                pstage = 2;
            }
            if (i + 1 - base >= ENT_CAP) {       // slide the window of plan entries (uniform; long key lists only)
                base = i;
                load_ent(cur, ent_cur, entr_cur, i);
                __syncthreads();
            }
            if (i + 1 < ne) {
                const int row0 = ROWS ? __builtin_amdgcn_readfirstlane(entr_cur[i + 1 - base]) : 0;
                if (L.wh == 0)
                    issue_tile<D, 4, ROWS, GRP, TK, DV>(p, oth, __builtin_amdgcn_readfirstlane(ent_cur[i + 1 - base].x), row0, kvh, L.w, L.lane, L.lane_k, L.lane_v);
            } else if (nxt_ok) {
                if (L.wh == 0) issue_tile<D, 4, ROWS, GRP, TK, DV>(p, oth, nxt.w, nxt_row0, item_hp(nxt) * HPI / p.group, L.w, L.lane, L.lane_k, L.lane_v);
                pstage = pstage == 2 ? 3 : -1;   // -1: tile requested before the entries (one-tile items)
            }
            const int2 en = ent_cur[i - base];
            compute_tile(buf, __builtin_amdgcn_readfirstlane(en.x), (unsigned)__builtin_amdgcn_readfirstlane(en.y) >> (2 * L.wr));
        }
        // ---- item finished: output (or hand the item to the exact pass), switch to the next item
        const int any_viol = __builtin_amdgcn_readfirstlane(__syncthreads_or(viol));
        if (any_viol) {
            if (threadIdx.x == 0) p.redo[atomicAdd(&p.counters[NLIST + 1], 1)] = cur_idx;
        } else {
            // (the loop has already flipped par: the last tile came from buffer par ^ 1)
            char* const stage = STAGE_IN_TILE ? bufs + (par ^ 1) * G::BUFB + L.w * 32 * 144 : stage_own;
            store_rows<DV, RT, ROWS>(p, L, stage, o, l, item_t(cur), item_hp(cur) * HPI + L.wh * RT);
        }
        cur_ok = nxt_ok;
        if (!cur_ok) break;
        // finish whatever of the next item's prefetch has not happened yet (one-tile items), then switch
        if (pstage == -1) load_ent(nxt, ent_nxt, entr_nxt, 0);
        cur = nxt;
        cur_idx = nxt_idx;
        load_q(cur, qf, art_q, pos_q, grp_q);
        { int2* tmp = ent_cur; ent_cur = ent_nxt; ent_nxt = tmp; }
        { int* tmp = entr_cur; entr_cur = entr_nxt; entr_nxt = tmp; }
        gslot ^= 1;
        if (grab_step(item_ne(cur)) < 0) grab(gslot);   // short item: fetch its successor now; read at the next tile step's barrier
    }
}

// ------------------------------------------------------------------------------------------------ host side
// Scratch memory of the entry point that allocates nothing (spinf_tree_attn_fwd_noalloc): list cursors, counts and the redo
// list.  In host code this name is a stand-in, not a device address: hipGetSymbolAddress gives the address, per device.
constexpr long NOALLOC_MAX_ITEMS = 1 << 16;                            // work items (query tiles x head groups) of one call
// 64 cursors and counts | the redo list: 256.25 KiB per GPU, held until the process ends
static __device__ __align__(256) int scratch[64 + NOALLOC_MAX_ITEMS];

namespace {

// Cursor blocks of the allocating entry point (64 ints of list cursors and counts, then the redo list).  A block belongs to the
// stream it was first used on: calls on one stream follow each other in stream order and share it, calls on different streams
// (or from host threads that use different streams) never share cursors, and no event or query is needed to tell when a block is
// free.  Blocks are never freed before the process ends: a bigger schedule gets a new block for its stream, and a launch
// recorded into a graph keeps the block it was recorded with for good (replays may run at any time): the calls that ONE capture
// records on a stream share that block (the graph runs them in the order they were recorded), no other call gets it again.
struct CursorBlock {
    int* ptr = nullptr;
    long cap = 0;               // redo entries
    hipStream_t owner = nullptr;
    bool taken = false;         // between acquire and release on some host thread
    bool pinned = false;        // recorded into a graph ...
    unsigned long long capture = 0;   // ... by the capture with this id
    bool dirty = false;         // a call on it failed to get all its kernels onto the stream: clear it before the next use
};
struct DeviceState {
    std::vector<CursorBlock> blocks;
    int cus = 0;
};
constexpr size_t MAX_CURSOR_BLOCKS = 1024;
std::mutex g_mu;
DeviceState g_dev[64];

int device_cus(int* cus) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) return spinf_fail(SPINF_E_HIP, "tree_attn: hipGetDevice: %s", hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_mu);
    DeviceState& s = g_dev[dev];
    if (!s.cus) {
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: hipGetDeviceProperties: %s", hipGetErrorString(e));
        s.cus = prop.multiProcessorCount;
    }
    *cus = s.cus;
    return SPINF_OK;
}

// -> the stream's block with room for n_items redo entries; *slot names it for release_block
int acquire_block(long n_items, bool capturing, unsigned long long capture, hipStream_t stream, int** ptr, int* slot, bool* dirty, long* cap) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) return spinf_fail(SPINF_E_HIP, "tree_attn: hipGetDevice: %s", hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_mu);
    DeviceState& s = g_dev[dev];
    for (int pass = 0; pass < 2; pass++)   // a capture's later calls take the block its first call pinned, before a fresh one
    for (size_t i = 0; i < s.blocks.size(); i++) {
        CursorBlock& b = s.blocks[i];
        if (b.taken || b.owner != stream || b.cap < n_items) continue;
        if (pass == 0 ? !(capturing && b.pinned && b.capture == capture) : b.pinned) continue;
        b.taken = true;
        b.pinned = capturing;
        b.capture = capturing ? capture : 0;
        *ptr = b.ptr;
        *slot = (int)i;
        *dirty = b.dirty;
        *cap = b.cap;
        return SPINF_OK;
    }
    if (capturing)
        return spinf_fail(SPINF_E_ARG, "tree_attn: this stream has no free cursor block of this size (a block recorded into an earlier graph stays with that "
                                       "graph) and none can be allocated during capture: run one call of this size on the stream before the capture, or "
                                       "record spinf_tree_attn_fwd_noalloc");
    if (s.blocks.size() >= MAX_CURSOR_BLOCKS) return spinf_fail(SPINF_E_NOMEM, "tree_attn: %zu cursor blocks on one device (one per stream in use)", s.blocks.size());
    CursorBlock b;
    b.cap = n_items < (1 << 16) ? (1 << 16) : 2 * n_items;
    b.owner = stream;
    e = hipMalloc((void**)&b.ptr, (64 + b.cap) * sizeof(int));
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: hipMalloc: %s", hipGetErrorString(e));
    e = hipMemset(b.ptr, 0, 64 * sizeof(int));   // cursors, counts and the running totals at [NLIST + 3], [NLIST + 4] start at zero
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: cursor block: %s", hipGetErrorString(e));
    b.taken = true;
    s.blocks.push_back(b);
    *ptr = b.ptr;
    *slot = (int)s.blocks.size() - 1;
    *dirty = false;
    *cap = b.cap;
    return SPINF_OK;
}

// after the call's kernels are on the stream (or failed to get there)
void release_block(int slot, bool failed) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return;
    std::lock_guard<std::mutex> lock(g_mu);
    CursorBlock& b = g_dev[dev].blocks[slot];
    b.dirty = failed;
    b.taken = false;
}

// ---- the entry point that allocates nothing

struct ScratchState {
    int* ptr = nullptr;   // device address of `scratch` on this device (every GPU holds its own copy of the array)
    int cus = 0;
};
ScratchState g_scratch[64];

int scratch_state(ScratchState** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) return spinf_fail(SPINF_E_HIP, "tree_attn (no allocation): hipGetDevice: %s", hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_mu);
    ScratchState& s = g_scratch[dev];
    if (!s.ptr) {   // first call on this device (it is the current one)
        hipDeviceProp_t prop;
        e = hipGetDeviceProperties(&prop, dev);
        if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn (no allocation): hipGetDeviceProperties: %s", hipGetErrorString(e));
        int* ptr = nullptr;
        e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) return spinf_fail(SPINF_E_HIP, "tree_attn (no allocation): hipGetSymbolAddress: %s", hipGetErrorString(e));
        s.cus = prop.multiProcessorCount;
        s.ptr = ptr;
    }
    *out = &s;
    return SPINF_OK;
}

// cursors and counts of a call start at zero whatever the previous call on this GPU left behind (a fill kernel, not a memset
// node: the call may be recorded into a graph); the running total of exact-pass items at [NLIST + 3] is kept
__global__ void attn_clear_counters_kernel(int* counters) {
    if (threadIdx.x < NLIST + 3) counters[threadIdx.x] = 0;
}

template <int D, int RT, bool WIN, int NHW, bool ROWS, int GRP = 0, int TK = 64, int DV = D>
int launch(const AttnParams& p, int blocks, hipStream_t stream) {
    using G = TileGeo<D, TK, DV>;
    static_assert(2 * G::BUFB + 2 * ENT_CAP * 12 + ((NHW == 2 && D == 256) ? 16 : 4 * NHW * 32 * 144) + 64 <= 160 * 1024, "LDS budget");
    if (p.clear_first) {
        hipLaunchKernelGGL(attn_clear_counters_kernel, dim3(1), dim3(64), 0, stream, p.counters);
        hipError_t e0 = hipGetLastError();
        if (e0 != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: launch (clear): %s", hipGetErrorString(e0));
    }
    hipLaunchKernelGGL((tree_attn_kernel<D, RT, WIN, NHW, ROWS, GRP, TK, DV>), dim3(blocks), dim3(256 * NHW), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: launch: %s", hipGetErrorString(e));
    // the exact pass over whatever the fast pass handed on (normally nothing: its workgroups read a zero count and leave)
    hipLaunchKernelGGL((tree_attn_exact_kernel<D, RT, WIN, RT * NHW, ROWS, GRP, TK, DV>), dim3(blocks < 64 ? blocks : 64), dim3(256), 0, stream, p);
    e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: launch (exact pass): %s", hipGetErrorString(e));
    return SPINF_OK;
}

// heads per wave (rt) and head sets across waves (nhw) for a head geometry; an item holds rt * nhw heads of one GQA group.
//   variant 0: eight waves (nhw = 2) wherever a group has an even number of heads, else one head per item
//   variant 1: one head per item, four waves
//   variant 2: four waves with two heads each where their registers fit (head dim <= 128), else as 1
void pick_kernel(int hq, int hkv, int d, int variant, int* rt, int* nhw) {
    const bool pairs = (hq / hkv) % 2 == 0;
    *rt = 1;
    *nhw = 1;
    if (d > 256) return;   // head dim 512: one head per item, the single-pass kernel
    if ((variant == 0 || variant == 3) && pairs) *nhw = 2;
    if (variant == 2 && pairs && d <= 128) *rt = 2;
}

template <int D>
int launch_d(const AttnParams& p, int rt, int nhw, bool win, int grp_mode, int blocks, hipStream_t s) {
    if (p.grp) {   // image groups: the one-head-per-wave kernels, stream layout
        if (nhw == 2) {
            if (!win) return launch<D, 1, false, 2, false, 1>(p, blocks, s);
            return grp_mode == 1 ? launch<D, 1, true, 2, false, 1>(p, blocks, s) : launch<D, 1, true, 2, false, 2>(p, blocks, s);
        }
        if (!win) return launch<D, 1, false, 1, false, 1>(p, blocks, s);
        return grp_mode == 1 ? launch<D, 1, true, 1, false, 1>(p, blocks, s) : launch<D, 1, true, 1, false, 2>(p, blocks, s);
    }
    if (p.row_of) {   // compact rows: the one-head-per-wave kernels only
        if (nhw == 2) return win ? launch<D, 1, true, 2, true>(p, blocks, s) : launch<D, 1, false, 2, true>(p, blocks, s);
        return win ? launch<D, 1, true, 1, true>(p, blocks, s) : launch<D, 1, false, 1, true>(p, blocks, s);
    }
    if (nhw == 2) return win ? launch<D, 1, true, 2, false>(p, blocks, s) : launch<D, 1, false, 2, false>(p, blocks, s);
    if constexpr (D <= 128) {
        if (rt == 2) return win ? launch<D, 2, true, 1, false>(p, blocks, s) : launch<D, 2, false, 1, false>(p, blocks, s);
    }
    return win ? launch<D, 1, true, 1, false>(p, blocks, s) : launch<D, 1, false, 1, false>(p, blocks, s);
}

// Head dim 512 (the full-attention layers of the Gemma-4 checkpoints, one key / value head) for compact rows and image groups
// (the stream layout without groups goes to the ring kernel, which keeps the accumulators in registers of its own choosing).
// O^T for 32 rows x 512 dims is 256
// accumulator registers per lane, which with the score tile and the 128 query registers leaves the register allocator no way
// out but scratch memory.  So the output is computed 256 dims at a time, in two launches over the same plan: each computes the
// scores over all 512 dims (that part is done twice) and P V for one half of V's columns.  Tiles are 32 keys (the plan is
// built with 32-key entries): a K tile of 32 KB and a half-width V tile of 16 KB, twice, fit the LDS with room to spare.
template <bool WIN, bool ROWS, int GRP>
int launch_512(const AttnParams& p, int blocks, hipStream_t s) {
    for (int half = 0; half < 2; half++) {
        AttnParams ph = p;
        ph.v = p.v + 256 * half;
        ph.o = p.o + 256 * half;
        if (int rc = launch<512, 1, WIN, 1, ROWS, GRP, 32, 256>(ph, blocks, s)) return rc;
    }
    return SPINF_OK;
}

// The ring kernel (tree_attn_ring.hip) over a static schedule: one launch.  It takes no item from a shared list and recomputes
// the items that need the exact arithmetic itself, so the call uses none of the block's cursors and no second kernel.
int launch_ring(const AttnParams& p, int d, bool win, int n_wg, hipStream_t stream) {
    if (p.clear_first) {
        hipLaunchKernelGGL(attn_clear_counters_kernel, dim3(1), dim3(64), 0, stream, p.counters);
        hipError_t e0 = hipGetLastError();
        if (e0 != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: launch (clear): %s", hipGetErrorString(e0));
    }
    return spinf_launch_ring(p, d, win, n_wg, stream);
}

int launch_d512(const AttnParams& p, bool win, int grp_mode, int blocks, hipStream_t s) {
    if (p.grp) {
        if (!win) return launch_512<false, false, 1>(p, blocks, s);
        return grp_mode == 1 ? launch_512<true, false, 1>(p, blocks, s) : launch_512<true, false, 2>(p, blocks, s);
    }
    if (p.row_of) return win ? launch_512<true, true, 0>(p, blocks, s) : launch_512<false, true, 0>(p, blocks, s);
    return win ? launch_512<true, false, 0>(p, blocks, s) : launch_512<false, false, 0>(p, blocks, s);
}

}  // namespace

extern "C" int spinf_attn_exact_items(int64_t* total) {
    if (!total) return spinf_fail(SPINF_E_ARG, "attn_exact_items: null pointer");
    *total = 0;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) return spinf_fail(SPINF_E_HIP, "attn_exact_items: hipGetDevice: %s", hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_mu);
    std::vector<const int*> blocks{(const int*)g_scratch[dev].ptr};
    for (const CursorBlock& b : g_dev[dev].blocks) blocks.push_back(b.ptr);
    for (const int* c : blocks) {
        if (!c) continue;   // no attention launch of that kind on this device yet
        int v = 0;
        e = hipMemcpy(&v, c + NLIST + 3, sizeof(int), hipMemcpyDeviceToHost);
        if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "attn_exact_items: hipMemcpy: %s", hipGetErrorString(e));
        *total += v;
    }
    return SPINF_OK;
}

extern "C" int spinf_attn_ring_aborts(int64_t* total) {
    if (!total) return spinf_fail(SPINF_E_ARG, "attn_ring_aborts: null pointer");
    *total = 0;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= 64) return spinf_fail(SPINF_E_HIP, "attn_ring_aborts: hipGetDevice: %s", hipGetErrorString(e));
    std::lock_guard<std::mutex> lock(g_mu);
    std::vector<const int*> blocks{(const int*)g_scratch[dev].ptr};
    for (const CursorBlock& b : g_dev[dev].blocks) blocks.push_back(b.ptr);
    for (const int* c : blocks) {
        if (!c) continue;
        int v = 0;
        e = hipMemcpy(&v, c + NLIST + 4, sizeof(int), hipMemcpyDeviceToHost);
        if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "attn_ring_aborts: hipMemcpy: %s", hipGetErrorString(e));
        *total += v;
    }
    return SPINF_OK;
}

extern "C" int spinf_attn_heads_per_item(int32_t hq, int32_t hkv, int32_t d, int32_t variant) {
    if (hq <= 0 || hkv <= 0 || hq % hkv) return 0;
    int rt, nhw;
    pick_kernel(hq, hkv, d, variant, &rt, &nhw);
    return rt * nhw;
}

static int attn_fwd(const spinf_attn_args* a, void* stream, bool no_alloc) {
    if (!a) return spinf_fail(SPINF_E_ARG, "tree_attn: null args");
    if (a->n <= 0 || a->n_items <= 0) return SPINF_OK;
    if (!a->q || !a->k || !a->v || !a->out || !a->art || !a->end || !a->pos || !a->kv_idx || !a->kv_bits || !a->items || !a->list_ptr)
        return spinf_fail(SPINF_E_ARG, "tree_attn: null pointer");
    if (no_alloc && a->n_items > NOALLOC_MAX_ITEMS)
        return spinf_fail(SPINF_E_ARG, "tree_attn (no allocation): %lld work items, at most %ld (query tiles x head groups)", (long long)a->n_items, NOALLOC_MAX_ITEMS);
    if (a->d != 64 && a->d != 128 && a->d != 256 && a->d != 512) return spinf_fail(SPINF_E_ARG, "tree_attn: head dim %d not in {64,128,256,512}", a->d);
    if (a->hq <= 0 || a->hkv <= 0 || a->hq % a->hkv) return spinf_fail(SPINF_E_ARG, "tree_attn: hq %d not a multiple of hkv %d", a->hq, a->hkv);
    if (a->n > INT32_MAX / 2) return spinf_fail(SPINF_E_ARG, "tree_attn: stream too long");
    if (!(a->scale > 0.f)) return spinf_fail(SPINF_E_ARG, "tree_attn: scale must be positive");
    int rt, nhw;
    pick_kernel(a->hq, a->hkv, a->d, a->variant, &rt, &nhw);
    if ((a->row_of != nullptr) != (a->kv_row0 != nullptr)) return spinf_fail(SPINF_E_ARG, "tree_attn: row_of and kv_row0 come together");
    if (a->row_of && rt != 1) return spinf_fail(SPINF_E_ARG, "tree_attn: variant %d does not take compact rows", a->variant);
    if (a->n_lists < 0 || a->n_lists > LAND_CAP) return spinf_fail(SPINF_E_ARG, "tree_attn: %d item lists, at most %d", a->n_lists, LAND_CAP);
    // the ring kernel: a static schedule over 32-key entries (head dim 256 and 512), or variant 3 at head dim 128 (64-key entries)
    const bool ring128 = a->variant == 3;
    const bool ring = a->n_lists > 0 && (a->ktile == 32 || ring128);
    if (ring128 && !(a->d == 128 && a->n_lists > 0 && (a->ktile == 0 || a->ktile == 64) && nhw == 2 && rt == 1 && !a->row_of && !a->grp))
        return spinf_fail(SPINF_E_ARG, "tree_attn: variant 3 (the kernel with decoupled waves at head dim 128) takes head dim 128, an even number of query heads per "
                                       "key / value head, a static schedule over 64-key entries, the stream layout and no image groups");
    if (ring && !ring128) {
        if (!((a->d == 256 && nhw == 2 && rt == 1) || a->d == 512) || a->row_of || a->grp)
            return spinf_fail(SPINF_E_ARG, "tree_attn: a static schedule over 32-key entries goes with head dim 512, or head dim 256 with an even number of query heads "
                                           "per key / value head and variant 0; with the stream layout and no image groups");
    } else if ((a->d == 512) != (a->ktile == 32) || (a->ktile != 0 && a->ktile != 32 && a->ktile != 64))
        return spinf_fail(SPINF_E_ARG, "tree_attn: plan entries of %d keys with head dim %d (32 goes with 512, 64 with the others)", a->ktile ? a->ktile : 64, a->d);
    if (a->grp && (a->grp_mode != 1 && a->grp_mode != 2)) return spinf_fail(SPINF_E_ARG, "tree_attn: group mode %d not in {1, 2}", a->grp_mode);
    if (a->grp && a->grp_mode == 2 && a->window <= 0)
        return spinf_fail(SPINF_E_ARG, "tree_attn: group mode 2 widens the mask inside the window only; a global layer takes no groups (pass grp = NULL)");
    if (a->grp && (rt != 1 || a->row_of)) return spinf_fail(SPINF_E_ARG, "tree_attn: image groups go with variant 0 / 1 and the stream layout only");
    const int hpi = rt * nhw;
    const int64_t nqt = (a->n + SPINF_QTILE - 1) / SPINF_QTILE;
    if (a->n_items != nqt * (a->hq / hpi))
        return spinf_fail(SPINF_E_ARG, "tree_attn: schedule has %lld items, %lld query tiles x %d head groups need %lld", (long long)a->n_items,
                          (long long)nqt, a->hq / hpi, (long long)(nqt * (a->hq / hpi)));
    const int64_t strides[8] = {a->q_tok, a->q_head, a->k_tok, a->k_head, a->v_tok, a->v_head, a->o_tok, a->o_head};
    for (int i = 0; i < 8; i++)
        if (strides[i] % 8) return spinf_fail(SPINF_E_ARG, "tree_attn: strides must be multiples of 8 elements");
    const uintptr_t ptrs[4] = {(uintptr_t)a->q, (uintptr_t)a->k, (uintptr_t)a->v, (uintptr_t)a->out};
    for (int i = 0; i < 4; i++)
        if (ptrs[i] % 16) return spinf_fail(SPINF_E_ARG, "tree_attn: tensors must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    int* counters = nullptr;
    int cus = 0, slot = -1;
    long redo_cap = NOALLOC_MAX_ITEMS;
    bool capturing = false, dirty = false;
    if (no_alloc) {
        ScratchState* st = nullptr;
        if (int rc = scratch_state(&st)) return rc;
        counters = st->ptr;
        cus = st->cus;
    } else {
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        unsigned long long capture = 0;
        if (hipStreamGetCaptureInfo(s, &cs, &capture) != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: hipStreamGetCaptureInfo failed");
        capturing = cs != hipStreamCaptureStatusNone;
        if (int rc = device_cus(&cus)) return rc;
        if (int rc = acquire_block((long)a->n_items, capturing, capture, s, &counters, &slot, &dirty, &redo_cap)) return rc;
    }
    AttnParams p;
    // A block's cursors are zero: it was cleared when allocated, and every call's exact-pass kernel, which runs after the fast pass,
    // puts them back.  Only a block whose last call failed to get its kernels onto the stream is cleared first; so is the scratch
    // array of the entry point that allocates nothing, which every caller on the GPU shares.
    // (the ring kernel uses no cursors: only a block left dirty is cleared in front of it, for the calls that follow)
    p.clear_first = ring ? dirty : no_alloc || dirty;
    p.static_lists = a->n_lists > 0;
    p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v; p.o = (__bf16*)a->out;
    p.q_tok = a->q_tok; p.q_head = a->q_head; p.k_tok = a->k_tok; p.k_head = a->k_head;
    p.v_tok = a->v_tok; p.v_head = a->v_head; p.o_tok = a->o_tok; p.o_head = a->o_head;
    p.n = (int)a->n; p.group = a->hq / a->hkv;
    p.c = a->scale * 1.4426950408889634f;
    p.window = a->window > 0 ? a->window : 0;
    p.art = a->art; p.end = a->end; p.pos = a->pos;
    p.kv_idx = a->kv_idx; p.kv_bits = a->kv_bits;
    p.items = (const int4*)a->items; p.list_ptr = a->list_ptr;
    p.row_of = a->row_of; p.kv_row0 = a->kv_row0;
    p.grp = a->grp;
    p.counters = counters;
    p.spin_limit = a->debug_expire > 0 ? a->debug_expire : (1 << 18);
    p.redo = counters + 64;
    const int blocks = a->n_lists > 0 ? a->n_lists : (int)(a->n_items < cus ? a->n_items : cus);
    const bool win = p.window > 0;
    int rc;
    if (ring) rc = launch_ring(p, a->d, win, a->n_lists, s);
    else switch (a->d) {
        case 64: rc = launch_d<64>(p, rt, nhw, win, a->grp_mode, blocks, s); break;
        case 128: rc = launch_d<128>(p, rt, nhw, win, a->grp_mode, blocks, s); break;
        case 256: rc = launch_d<256>(p, rt, nhw, win, a->grp_mode, blocks, s); break;
        default: rc = launch_d512(p, win, a->grp_mode, blocks, s);
    }
    if (slot >= 0) release_block(slot, rc != SPINF_OK);
    return rc;
}

extern "C" int spinf_tree_attn_fwd(const spinf_attn_args* a, void* stream) { return attn_fwd(a, stream, false); }

extern "C" int spinf_tree_attn_fwd_noalloc(const spinf_attn_args* a, void* stream) { return attn_fwd(a, stream, true); }
