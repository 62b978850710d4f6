// Tree-mask packed-prefill attention for gfx950, the ring kernel: the same arithmetic as tree_attn.hip's fast pass (same 32-key
// blocks in the same order, same softmax reference, same bits), with the waves of a workgroup decoupled.
//
// Replaces the flex_attention call of spinf_serve/models/gemma4.py:107-118 and spinf_serve/models/qwen35/qwen.py:614,620 for
// head dim 256 with an even number of query heads per key / value head (eight waves: four row groups x the two heads of an
// item) and for head dim 512 (four waves, one head per item, one wave per SIMD: the 32 x 512 outputs of a wave are all 256
// accumulation registers, which no kernel that leaves its accumulators to the compiler gets allocated; a ring of two slots).
//
// Why.  With a workgroup barrier at every key tile the eight waves move in lockstep: a wave whose 32 rows see nothing of a tile
// (the diagonal of a branch region) idles, all waves start their MFMA phases and their softmax phases together, and nothing
// overlaps the end of a work item (output rows, the next item's queries).  A free-running wave pair keeps a SIMD's matrix pipe
// busy by itself (measured: K Q^T, softmax and P V of a 32 x 32 block from LDS at the rate of the bare MFMAs), so here no wave
// ever waits for another one except through the tile ring:
//
//   * K / V tiles of 32 keys live in a ring of NSLOT slots.  Every wave walks the workgroup's tile sequence (all the tiles of
//     its work items, item after item) and skips the tiles its rows see nothing of.  When a wave is through with a tile it
//     counts itself in (`done`); once all have, whichever wave comes by first recycles the slot: it requests, by itself, the
//     DMA of the tile NSLOT places further on (`issued`); the last request of the batch writes the slot's flag, so the DMA engine itself
//     reports the tile as landed.  A wave needs the flag before it reads a tile and `issued` before it skips one, so the
//     waves stay within NSLOT - 1 tiles of each other.
//   * Work items are assigned to workgroups on the host (spinf_tileplan_schedule_static: a simulation of "the workgroup that
//     is free first takes the next item"), so the tile sequence of a workgroup is known to all its waves without any exchange
//     between workgroups; wave 0 expands it into a ring of tile descriptors in LDS, well ahead of everyone.
//   * A wave finishes an item on its own: its 32 output rows leave through a private LDS slice while the other waves compute,
//     and it requests its next queries right away.
//
// Every wait is a bounded spin on an LDS word; a wave that runs out of spins sets the workgroup's abort flag (and a counter the
// host can read), which makes every wave of the workgroup leave the ring at its next wait; the workgroup then computes its list
// again, one tile at a time between barriers (ring_paced_pass): the same bits, later.
#include <hip/hip_runtime.h>

#include <type_traits>

#include "attn_kernels.h"
#include "attn_ring_io.h"

namespace {

constexpr int MAX_SLOT = 4;         // tile ring depth (32-key tiles): 4, at head dim 512 (69 KB a tile) 2
constexpr int NDESC = 128;          // tile descriptors kept in LDS
constexpr int GEN_AHEAD = 48;       // wave 0 keeps the descriptors this far ahead of its own tile
constexpr int SPIN_LIMIT = 1 << 18; // polls of one wait before the workgroup gives up (a healthy wait takes a handful)
constexpr int SROW = 64 + 16;       // output staging: 32 rows x 32 head dims, 80-byte rows
constexpr unsigned DESC_FIRST = 1u << 16, DESC_LAST = 1u << 17;

__device__ __forceinline__ int lds_load(const int* p) { return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP); }
// plain (non-atomic) reads of words other waves write, as LDS instructions: a volatile access through a generic pointer becomes a
// flat load, which counts against the tile requests in flight
typedef __attribute__((ext_vector_type(4))) int i32x4;
__device__ __forceinline__ int lds_peek(const int* p) { return *(const volatile __attribute__((address_space(3))) int*)(const __attribute__((address_space(3))) void*)p; }
__device__ __forceinline__ i32x4 lds_peek4(const int* p) {
    return *(const volatile __attribute__((address_space(3))) i32x4*)(const __attribute__((address_space(3))) void*)p;
}
__device__ __forceinline__ void lds_store(int* p, int v) { __hip_atomic_store(p, v, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP); }


// ---- O^T accumulators in fixed accumulation registers.
// The 32 rows x D output accumulators of a wave live in a[0 : D/2 - 1] and are touched by inline assembly only: tile d (32
// head dims) is a[16 d : 16 d + 15].  The compiler never sees them as values: as values they go through the merge points of
// the tile loop (a wave either computes a tile or skips it), and the register allocator then keeps copies of them and spills
// the queries.  The file is compiled with -amdgpu-spill-vgpr-to-agpr=0 and contains no MFMA builtin, so nothing else ever
// uses an accumulation register.  The hazards the compiler would take care of are handled here: a full s_nop before the
// accumulators are read back (MFMA result -> v_accvgpr_read) and after they are zeroed (v_accvgpr_write -> MFMA srcC).
#define ACC_CLOB(b) "a" #b
#define ACC16_CLOBBERS(b0, b1, b2, b3, b4, b5, b6, b7, b8, b9, b10, b11, b12, b13, b14, b15) \
    ACC_CLOB(b0), ACC_CLOB(b1), ACC_CLOB(b2), ACC_CLOB(b3), ACC_CLOB(b4), ACC_CLOB(b5), ACC_CLOB(b6), ACC_CLOB(b7), ACC_CLOB(b8), ACC_CLOB(b9), \
        ACC_CLOB(b10), ACC_CLOB(b11), ACC_CLOB(b12), ACC_CLOB(b13), ACC_CLOB(b14), ACC_CLOB(b15)

#define ACC_TILE_OPS(DT, LO, HI, C0, C1, C2, C3, C4, C5, C6, C7, C8, C9, C10, C11, C12, C13, C14, C15)                                                 \
    if constexpr (TILE == DT) {                                                                                                                        \
        if constexpr (OP == 0)                                                                                                                         \
            asm volatile("v_mfma_f32_32x32x16_bf16 a[" #LO ":" #HI "], %0, %1, a[" #LO ":" #HI "]" ::"v"(a), "v"(b)                                    \
                         : ACC16_CLOBBERS(C0, C1, C2, C3, C4, C5, C6, C7, C8, C9, C10, C11, C12, C13, C14, C15));                                     \
        else if constexpr (OP == 1)                                                                                                                    \
            asm volatile("v_accvgpr_write_b32 a" #C0 ", 0\n\tv_accvgpr_write_b32 a" #C1 ", 0\n\tv_accvgpr_write_b32 a" #C2 ", 0\n\tv_accvgpr_write_b32 a" #C3 ", 0\n\t"   \
                         "v_accvgpr_write_b32 a" #C4 ", 0\n\tv_accvgpr_write_b32 a" #C5 ", 0\n\tv_accvgpr_write_b32 a" #C6 ", 0\n\tv_accvgpr_write_b32 a" #C7 ", 0\n\t"   \
                         "v_accvgpr_write_b32 a" #C8 ", 0\n\tv_accvgpr_write_b32 a" #C9 ", 0\n\tv_accvgpr_write_b32 a" #C10 ", 0\n\tv_accvgpr_write_b32 a" #C11 ", 0\n\t" \
                         "v_accvgpr_write_b32 a" #C12 ", 0\n\tv_accvgpr_write_b32 a" #C13 ", 0\n\tv_accvgpr_write_b32 a" #C14 ", 0\n\tv_accvgpr_write_b32 a" #C15 ", 0" :: \
                             : ACC16_CLOBBERS(C0, C1, C2, C3, C4, C5, C6, C7, C8, C9, C10, C11, C12, C13, C14, C15));                                 \
        else if constexpr (OP == 3)                                                                                                                    \
            asm volatile("v_accvgpr_write_b32 a" #C0 ", %0\n\tv_accvgpr_write_b32 a" #C1 ", %1\n\tv_accvgpr_write_b32 a" #C2 ", %2\n\tv_accvgpr_write_b32 a" #C3 ", %3\n\t"     \
                         "v_accvgpr_write_b32 a" #C4 ", %4\n\tv_accvgpr_write_b32 a" #C5 ", %5\n\tv_accvgpr_write_b32 a" #C6 ", %6\n\tv_accvgpr_write_b32 a" #C7 ", %7\n\t"     \
                         "v_accvgpr_write_b32 a" #C8 ", %8\n\tv_accvgpr_write_b32 a" #C9 ", %9\n\tv_accvgpr_write_b32 a" #C10 ", %10\n\tv_accvgpr_write_b32 a" #C11 ", %11\n\t" \
                         "v_accvgpr_write_b32 a" #C12 ", %12\n\tv_accvgpr_write_b32 a" #C13 ", %13\n\tv_accvgpr_write_b32 a" #C14 ", %14\n\tv_accvgpr_write_b32 a" #C15 ", %15" :: \
                             "v"(r[0]), "v"(r[1]), "v"(r[2]), "v"(r[3]), "v"(r[4]), "v"(r[5]), "v"(r[6]), "v"(r[7]), "v"(r[8]), "v"(r[9]), "v"(r[10]),            \
                         "v"(r[11]), "v"(r[12]), "v"(r[13]), "v"(r[14]), "v"(r[15])                                                                      \
                         : ACC16_CLOBBERS(C0, C1, C2, C3, C4, C5, C6, C7, C8, C9, C10, C11, C12, C13, C14, C15));                                     \
        else                                                                                                                                           \
            asm volatile("v_accvgpr_read_b32 %0, a" #C0 "\n\tv_accvgpr_read_b32 %1, a" #C1 "\n\tv_accvgpr_read_b32 %2, a" #C2 "\n\tv_accvgpr_read_b32 %3, a" #C3 "\n\t"     \
                         "v_accvgpr_read_b32 %4, a" #C4 "\n\tv_accvgpr_read_b32 %5, a" #C5 "\n\tv_accvgpr_read_b32 %6, a" #C6 "\n\tv_accvgpr_read_b32 %7, a" #C7 "\n\t"     \
                         "v_accvgpr_read_b32 %8, a" #C8 "\n\tv_accvgpr_read_b32 %9, a" #C9 "\n\tv_accvgpr_read_b32 %10, a" #C10 "\n\tv_accvgpr_read_b32 %11, a" #C11 "\n\t" \
                         "v_accvgpr_read_b32 %12, a" #C12 "\n\tv_accvgpr_read_b32 %13, a" #C13 "\n\tv_accvgpr_read_b32 %14, a" #C14 "\n\tv_accvgpr_read_b32 %15, a" #C15     \
                         : "=v"(r[0]), "=v"(r[1]), "=v"(r[2]), "=v"(r[3]), "=v"(r[4]), "=v"(r[5]), "=v"(r[6]), "=v"(r[7]), "=v"(r[8]), "=v"(r[9]), "=v"(r[10]),      \
                           "=v"(r[11]), "=v"(r[12]), "=v"(r[13]), "=v"(r[14]), "=v"(r[15]));                                                        \
    }

// OP 0: acc[TILE] += a * b (MFMA 32x32x16 bf16); OP 1: acc[TILE] = 0; OP 2: r[0..15] = acc[TILE]; OP 3: acc[TILE] = r[0..15]
template <int TILE, int OP>
__device__ __forceinline__ void acc_op(const bf16x8 a, const bf16x8 b, float (&r)[16]) {
    ACC_TILE_OPS(0, 0, 15, 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15)
    ACC_TILE_OPS(1, 16, 31, 16, 17, 18, 19, 20, 21, 22, 23, 24, 25, 26, 27, 28, 29, 30, 31)
    ACC_TILE_OPS(2, 32, 47, 32, 33, 34, 35, 36, 37, 38, 39, 40, 41, 42, 43, 44, 45, 46, 47)
    ACC_TILE_OPS(3, 48, 63, 48, 49, 50, 51, 52, 53, 54, 55, 56, 57, 58, 59, 60, 61, 62, 63)
    ACC_TILE_OPS(4, 64, 79, 64, 65, 66, 67, 68, 69, 70, 71, 72, 73, 74, 75, 76, 77, 78, 79)
    ACC_TILE_OPS(5, 80, 95, 80, 81, 82, 83, 84, 85, 86, 87, 88, 89, 90, 91, 92, 93, 94, 95)
    ACC_TILE_OPS(6, 96, 111, 96, 97, 98, 99, 100, 101, 102, 103, 104, 105, 106, 107, 108, 109, 110, 111)
    ACC_TILE_OPS(7, 112, 127, 112, 113, 114, 115, 116, 117, 118, 119, 120, 121, 122, 123, 124, 125, 126, 127)
    ACC_TILE_OPS(8, 128, 143, 128, 129, 130, 131, 132, 133, 134, 135, 136, 137, 138, 139, 140, 141, 142, 143)
    ACC_TILE_OPS(9, 144, 159, 144, 145, 146, 147, 148, 149, 150, 151, 152, 153, 154, 155, 156, 157, 158, 159)
    ACC_TILE_OPS(10, 160, 175, 160, 161, 162, 163, 164, 165, 166, 167, 168, 169, 170, 171, 172, 173, 174, 175)
    ACC_TILE_OPS(11, 176, 191, 176, 177, 178, 179, 180, 181, 182, 183, 184, 185, 186, 187, 188, 189, 190, 191)
    ACC_TILE_OPS(12, 192, 207, 192, 193, 194, 195, 196, 197, 198, 199, 200, 201, 202, 203, 204, 205, 206, 207)
    ACC_TILE_OPS(13, 208, 223, 208, 209, 210, 211, 212, 213, 214, 215, 216, 217, 218, 219, 220, 221, 222, 223)
    ACC_TILE_OPS(14, 224, 239, 224, 225, 226, 227, 228, 229, 230, 231, 232, 233, 234, 235, 236, 237, 238, 239)
    ACC_TILE_OPS(15, 240, 255, 240, 241, 242, 243, 244, 245, 246, 247, 248, 249, 250, 251, 252, 253, 254, 255)
}
template <int TILE>
__device__ __forceinline__ void acc_mfma(const bf16x8 a, const bf16x8 b) {
    float unused[16];
    acc_op<TILE, 0>(a, b, unused);
}
template <int N, int TILE = 0>
__device__ __forceinline__ void acc_zero() {
    if constexpr (TILE < N) {
        float unused[16];
        acc_op<TILE, 1>(bf16x8{}, bf16x8{}, unused);
        acc_zero<N, TILE + 1>();
    } else {
        asm volatile("s_nop 3" ::: "memory");   // v_accvgpr_write -> MFMA srcC
    }
}
template <int TILE>
__device__ __forceinline__ void acc_read(float (&r)[16]) {
    acc_op<TILE, 2>(bf16x8{}, bf16x8{}, r);
}
// acc[0 .. N-1] *= alpha (the exact recomputation's rescaling; the caller brackets it with the wait states that acc_read and
// acc_zero need)
template <int N, int TILE = 0>
__device__ __forceinline__ void acc_scale(const float alpha) {
    if constexpr (TILE < N) {
        float r[16];
        acc_op<TILE, 2>(bf16x8{}, bf16x8{}, r);
#pragma unroll
        for (int i = 0; i < 16; i++) r[i] *= alpha;
        acc_op<TILE, 3>(bf16x8{}, bf16x8{}, r);
        acc_scale<N, TILE + 1>(alpha);
    }
}
// S^T chain on ordinary registers, as assembly as well (a kernel that mixes MFMA builtins with the fixed accumulation registers
// above would let the compiler pick accumulation registers of its own for them)
__device__ __forceinline__ void qk_first(f32x16& sa, const bf16x8 k, const bf16x8 q) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(sa) : "v"(k), "v"(q));
}
__device__ __forceinline__ void qk_next(f32x16& sa, const bf16x8 k, const bf16x8 q) {
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(sa) : "v"(k), "v"(q));
}
__device__ __forceinline__ void qk_last(f32x16& sa, const bf16x8 k, const bf16x8 q) {   // + the wait states before the vector ALU reads the result
    asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\ts_nop 15" : "+v"(sa) : "v"(k), "v"(q));
}

template <int N, int F = 0, class Fn>
__device__ __forceinline__ void pv_steps(Fn& fn) {
    if constexpr (F < N) {
        fn(std::integral_constant<int, F>{});
        pv_steps<N, F + 1>(fn);
    }
}

// A wave's place in the workgroup: four row groups x HPI heads of the item.
template <int D>
struct RingShape {
    static constexpr int TK = D == 128 ? 64 : 32;    // keys per tile: at head dim 128 a 32-key tile is too little work per ring slot
    static constexpr int NSUB = TK / 32;             // 32-key blocks per tile
    static constexpr int NW = D == 512 ? 4 : 8;      // waves: four row groups x HPI heads of the item
    static constexpr int HPI = NW / 4;
    static constexpr int NSLOT = D == 512 ? 2 : MAX_SLOT;
    static constexpr int NS = D / 16;     // contraction steps of K Q^T
    static constexpr int NDT = D / 32;    // 32-wide slices of the head dimension in O^T
    static constexpr int NVF = 2 * NDT;   // V^T fragments of one 32-key block
};

// the queries of rows 32 wr .. of query tile tz & 0xfffff, head (tz >> 20) * HPI + wh, as B operands of K Q^T; art / pos of the wave's rows
template <int D, bool WIN>
__device__ __forceinline__ void ring_load_q(const AttnParams& p, const int wr, const int wh, const int tz, bf16x8 (&qf)[D / 16], int& art_q, int& pos_q) {
    const int lane = fresh_lane_id();
    const int tok = (tz & 0xfffff) * SPINF_QTILE + 32 * wr + (lane & 31);
    const int tok_c = tok < p.n ? tok : p.n - 1;
    const int h = (int)((unsigned)tz >> 20) * RingShape<D>::HPI + wh;
    const __bf16* qp = p.q + (long)tok_c * p.q_tok + (long)h * p.q_head + 8 * (lane >> 5);
#pragma unroll
    for (int s = 0; s < D / 16; s++) qf[s] = *(const bf16x8*)(qp + 16 * s);
    art_q = tok < p.n ? p.art[tok_c] : -1;
    pos_q = WIN ? p.pos[tok_c] : 0;
}

// normalise O^T and store it as rows: 32 rows x 32 head dims at a time through the wave's own LDS slice `stage`, 16-byte pieces out
// (pieces of 8 bytes straight from the registers were measured slower: twice the requests for the same bytes)
template <int D>
__device__ __forceinline__ void ring_store_rows(const AttnParams& p, const int wr, const int wh, char* const stage, const int tz, const float l) {
    constexpr int NDT = D / 32;
    const int lane = fresh_lane_id(), m = lane & 31, g = lane >> 5;
    const int tok0 = (tz & 0xfffff) * SPINF_QTILE + 32 * wr;
    const int h = (int)((unsigned)tz >> 20) * RingShape<D>::HPI + wh;
    const float inv = 1.0f / lane32_sum(l);
    __bf16* ob = p.o + (long)h * p.o_head;
    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");   // the last MFMAs' results -> v_accvgpr_read
    // tile dt is read back from the slice while tile dt + 1 is converted and written to it (the LDS takes a wave's requests
    // in order, so the write behind the read is safe), and stored after that: no wait between a write and its read-back
    auto put = [&](auto dt_c) __attribute__((always_inline)) {
        constexpr int dt = decltype(dt_c)::value;
        float r16[16];
        acc_read<dt>(r16);
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
            bf16x4 r;
#pragma unroll
            for (int jj = 0; jj < 4; jj++) r[jj] = (__bf16)(r16[4 * i4 + jj] * inv);
            *(bf16x4*)(stage + m * SROW + (8 * i4 + 4 * g) * 2) = r;
        }
    };
    auto round = [&](auto dt_c) __attribute__((always_inline)) {
        constexpr int dt = decltype(dt_c)::value;
        bf16x8 val[2];
#pragma unroll
        for (int jj = 0; jj < 2; jj++) {
            const int c = jj * 64 + lane;
            val[jj] = *(const bf16x8*)(stage + (c >> 2) * SROW + (c & 3) * 16);
        }
        if constexpr (dt + 1 < NDT) put(std::integral_constant<int, dt + 1>{});
#pragma unroll
        for (int jj = 0; jj < 2; jj++) {
            const int c = jj * 64 + lane, row = c >> 2, col = c & 3;
            if (tok0 + row < p.n) *(bf16x8*)(ob + (long)(tok0 + row) * p.o_tok + 32 * dt + col * 8) = val[jj];
        }
    };
    put(std::integral_constant<int, 0>{});
    pv_steps<NDT>(round);
}

// ---- after the list: the barrier-paced pass over single items.  One tile at a time into slot 0 of the ring, a workgroup barrier on
// either side of its request, nothing overlapped, no spin anywhere.  Every workgroup of the ring kernel ends in it (normally with
// nothing to do).  Two uses:
//   * the exact recomputation.  Items in which some row met scores too far above its reference (normally none) are done again by the
//     workgroup that owns them: classic online softmax over the same 32-key blocks in the same order (the reference is raised, and
//     the accumulators rescaled, whenever a block maximum exceeds it by more than TAU_LAZY), the arithmetic of tree_attn_exact_kernel
//     (tree_attn.hip) step for step, so the two give the same bits.  Whether an item comes here depends on its own rows only, so a
//     job's output does not depend on what it is packed with.
//   * the landing after an abort.  If a wave gave up a wait, every wave has left the ring; the items li .. hi - 1 of the list (from
//     the first one that some wave had not completed) are then computed here with the ring pass's own arithmetic (fixed reference, no
//     rescaling: the same bits), handing items to the exact recomputation by the same rule.  An abort costs time, never rows.
// Every wave of the workgroup calls it together: li < hi only after an abort; *sy_nredo = entries of the workgroup's redo list
// p.redo[lo ..]; *sy_vote = 0.
template <int D, bool WIN>
__device__ __forceinline__ void ring_paced_pass(const AttnParams& p, char* const ring, char* const stage_all, int* const sy_nredo, int* const sy_vote,
                                                const int lo, const int hi, int li) {
    using S = RingShape<D>;
    constexpr int TK = S::TK, HPI = S::HPI, NS = S::NS, NDT = S::NDT, NVF = S::NVF;
    using G = TileGeo<D, TK, D>;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wh = w >> 2, wr = wh ? 3 - (w & 3) : (w & 3);   // as Lane (attn_kernels.h)
    char* const stage = stage_all + w * 32 * SROW;
    bf16x8 qf[NS];
    int art_q = -1, pos_q = 0;
    int ri = 0;   // next entry of the redo list
#pragma unroll 1
    while (true) {
        const bool exact = li >= hi;   // first the landing's items, if any, then the recomputations
        int idx = li;
        if (exact) {
            if (ri >= __builtin_amdgcn_readfirstlane(lds_load(sy_nredo))) break;
            idx = __builtin_amdgcn_readfirstlane(__hip_atomic_load(&p.redo[lo + ri], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        }
        const int4 itv = p.items[idx];
        const int it_t = __builtin_amdgcn_readfirstlane(itv.x), it_e0 = __builtin_amdgcn_readfirstlane(itv.y), it_z = __builtin_amdgcn_readfirstlane(itv.z);
        const int ne = it_z & 0xfffff;
        const int tz = it_t | (int)((unsigned)it_z >> 20 << 20);
        const int kvh = (int)((unsigned)it_z >> 20) * HPI / p.group;
        ring_load_q<D, WIN>(p, wr, wh, tz, qf, art_q, pos_q);
        float M = -INFINITY, l = 0.f;
        bool viol = false;
        acc_zero<NDT>();
#pragma unroll 1
        for (int e = 0; e < ne; e++) {
            const int kt = __builtin_amdgcn_readfirstlane(p.kv_idx[it_e0 + e]);
            const unsigned bits = (unsigned)__builtin_amdgcn_readfirstlane((int)p.kv_bits[it_e0 + e]);
            __syncthreads();   // everyone is through with the slot
            if (w == 0) {
                using GK = Geo<D, TK>;
                const int lane = fresh_lane_id();
                const unsigned lane_k = (unsigned)((lane / GK::CPR) * GK::NREG * p.k_tok * 2 + (lane % GK::CPR) * 16);
                const unsigned lane_v = (unsigned)((lane / GK::CPR) * GK::NREG * p.v_tok * 2 + (lane % GK::CPR) * 16);
                issue_tile_wave<D, WIN, TK>(p, lds_addr(ring), kt, kvh, 0, lane, lane_k, lane_v);
            }
            __builtin_amdgcn_s_waitcnt(0x0f70);   // the tile has landed (and this wave's queries)
            __syncthreads();
#pragma unroll 1
            for (int sub = 0; sub < S::NSUB; sub++) {   // the tile's 32-key blocks
            if (!((bits >> (2 * wr + sub)) & 1u)) continue;   // (wave-uniform; the barriers above are passed by every wave)
            const int ln = fresh_lane_id();
            const char* krow = ring + G::K::k_off(ln & 31) + 16 * (ln >> 5) + sub * G::KSUB;
            const char* vrow = ring + G::KTILEB + G::V::v_off(4 * (ln >> 5) + ((ln >> 2) & 3)) + 32 * ((ln >> 4) & 1) + 8 * (ln & 3) + sub * G::VSUB;
            // (the scheduling barriers keep the phases apart.  The MFMAs are assembly, which the compiler's hazard recogniser does
            // not look into: left to interleave the softmax of the block's second half with the P V products of the first, it
            // put the conversion that writes a P fragment directly in front of the MFMA that reads it, and an MFMA that issues in
            // the cycle after a vector write of its A / B registers reads the old values (spinf_diag_mfma_hazard measures it).
            // With the phases apart, V fragment reads lie between the conversions and the first MFMA; the build scans the
            // generated assembly for the pattern.)
            f32x16 sa;
            __builtin_amdgcn_sched_barrier(0);
            auto score = [&](auto x_c) __attribute__((always_inline)) {
                constexpr int x = decltype(x_c)::value;
                const bf16x8 kf = *(const bf16x8*)(krow + 32 * x);
                if (x == 0) qk_first(sa, kf, qf[x]);
                else if (x == NS - 1) qk_last(sa, kf, qf[x]);
                else qk_next(sa, kf, qf[x]);
            };
            pv_steps<NS>(score);
            __builtin_amdgcn_sched_barrier(0);
            if ((bits >> (8 + 2 * wr + sub)) & 1u) {
                f32x16 sm[1] = {sa};
                const int tok = (tz & 0xfffff) * SPINF_QTILE + 32 * wr + (ln & 31);
                apply_mask<1, WIN, 0, TK>(sm, (const int*)(ring + G::KTILEB + G::VTILEB), kt, sub, ln >> 5, tok, art_q, pos_q, p.window);
                sa = sm[0];
            }
            __builtin_amdgcn_sched_barrier(0);
            bf16x8 pb[2];
            // (each branch is written out in full, statement for statement as in tree_attn_exact_kernel and in the ring loop: the
            // compiler contracts `l *= alpha; l += sum` into one fused multiply-add where it sees them together, and the bits follow)
            if (exact) {
                float mx = sa[0];
#pragma unroll
                for (int i2 = 1; i2 < 16; i2++) mx = fmaxf(mx, sa[i2]);
                mx = lane32_max(mx);
                const float tm = mx * p.c;
                const bool up = tm > M + TAU_LAZY;
                const float mn = up ? tm : M;
                const float alpha = up ? __builtin_amdgcn_exp2f(M - mn) : 1.0f;
                if (__builtin_amdgcn_ballot_w64(up && M != -INFINITY) != 0) {   // rows without a key so far hold zeros
                    asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");   // the last MFMAs' results -> v_accvgpr_read
                    acc_scale<NDT>(alpha);
                    asm volatile("s_nop 3" ::: "memory");                // v_accvgpr_write -> MFMA srcC
                }
                l *= alpha;
                M = mn;
                const float ms = mn == -INFINITY ? 0.f : mn;
                float sum = 0.f;
#pragma unroll
                for (int i2 = 0; i2 < 16; i2++) {
                    const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(sa[i2], p.c, -ms));
                    sum += pr;
                    pb[i2 >> 3][i2 & 7] = (__bf16)pr;
                }
                l += sum;
            } else {   // the ring pass's arithmetic: the row's reference is the maximum of the first block it sees a key in
                const bool first = M == -INFINITY;
                if (__builtin_amdgcn_ballot_w64(first) != 0) {
                    float mx = sa[0];
#pragma unroll
                    for (int i2 = 1; i2 < 16; i2++) mx = fmaxf(mx, sa[i2]);
                    mx = lane32_max(mx);
                    M = first ? mx * p.c : M;
                }
                const float ms = M == -INFINITY ? 0.f : M;
                float sum = 0.f;
#pragma unroll
                for (int i2 = 0; i2 < 16; i2++) {
                    const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(sa[i2], p.c, -ms));
                    sum += pr;
                    pb[i2 >> 3][i2 & 7] = (__bf16)pr;
                }
                l += sum;
                viol = viol | !(sum <= VIOL_SUM);
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0): the softmax phase ends here, the waits below are for V fragments only
            __builtin_amdgcn_sched_barrier(0);
            auto step = [&](auto f_c) __attribute__((always_inline)) {
                constexpr int f = decltype(f_c)::value;
                const char* vp = vrow + G::V::v_off(16 * (f / NDT)) + 64 * (f % NDT);
                const s16x4 lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)vp);
                const s16x4 hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vp + G::V::v_off(8)));
                const bf16x8 a = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7));
                acc_mfma<f % NDT>(a, pb[f / NDT]);
                __builtin_amdgcn_sched_barrier(0);
            };
            pv_steps<NVF>(step);
            }
        }
        if (!exact && __builtin_amdgcn_ballot_w64(viol) != 0) {   // scores ranged too widely somewhere in these 32 rows: the item is done again, exactly
            if (fresh_lane_id() == 0) __hip_atomic_store(sy_vote, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
            ring_store_rows<D>(p, wr, wh, stage, tz, l);
        }
        if (exact) {
            ri++;
            continue;
        }
        __syncthreads();
        if (threadIdx.x == 0 && lds_load(sy_vote) != 0) {   // (a wave may have handed the item over before the abort already)
            const int k = lds_load(sy_nredo);
            bool listed = false;
            for (int r = 0; r < k; r++) listed = listed || __hip_atomic_load(&p.redo[lo + r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == idx;
            if (!listed) {
                __hip_atomic_store(&p.redo[lo + k], idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                lds_store(sy_nredo, k + 1);
            }
            lds_store(sy_vote, 0);
        }
        __syncthreads();
        li++;
    }
    if (ri > 0 && threadIdx.x == 0) atomicAdd(&p.counters[NLIST + 3], ri);   // running total, for spinf_attn_exact_items
    __builtin_amdgcn_s_waitcnt(0x0f70);
}

template <int D, bool WIN>
__global__ __launch_bounds__(D == 512 ? 256 : 512) void tree_attn_ring_kernel(const AttnParams p) {
    constexpr int TK = RingShape<D>::TK, NSUB = RingShape<D>::NSUB;
    constexpr int NW = D == 512 ? 4 : 8;      // waves: four row groups x HPI heads of the item
    constexpr int HPI = NW / 4;
    constexpr int NSLOT = D == 512 ? 2 : MAX_SLOT;
    using G = TileGeo<D, TK, D>;
    constexpr int NS = D / 16;     // contraction steps of K Q^T
    constexpr int NDT = D / 32;    // 32-wide slices of the head dimension in O^T
    constexpr int NVF = 2 * NDT;   // V^T fragments of one 32-key block
    constexpr int PFD = D >= 256 ? 2 : 8;   // fragment read-ahead: at head dim 256 one more spills a query fragment inside the tile loop
    constexpr int PF = D >= 256 ? 4 : (NS < PFD ? NS : PFD);   // K fragments are live in the score phase only, where registers are free
    constexpr int VPF = NVF < PFD ? NVF : PFD;
    constexpr int DONE_AT = NVF - 1 - VPF > 0 ? NVF - 1 - VPF : 0;   // the P V step behind which a block's last V fragment read is on its way
    static_assert(NSLOT * G::BUFB + NW * 32 * SROW + NDESC * 16 + 256 <= 160 * 1024, "LDS budget");
    __shared__ __attribute__((aligned(16))) char ring[NSLOT * G::BUFB];
    __shared__ __attribute__((aligned(16))) char stage_all[NW * 32 * SROW];   // output staging, one slice per wave
    __shared__ int4 desc[NDESC];       // {key tile, bits | DESC_FIRST | DESC_LAST, query tile | head group << 20, item index}
    __shared__ __attribute__((aligned(16))) int sy_done[MAX_SLOT];   // waves through with the tile in the slot; NW = the slot waits for somebody to recycle it (words past NSLOT stay 0)
    __shared__ int sy_issued[MAX_SLOT];   // tile the slot was last recycled for (its DMA requested)
    __shared__ int sy_gen;             // descriptors written so far
    __shared__ int sy_abort;
    __shared__ int sy_gave_up;         // waves that gave up a wait
    __shared__ int sy_ntiles;
    __shared__ int sy_redo[16];        // item sequence number + 1 of the last hand-over to the exact recomputation, per sequence number mod 16
    __shared__ int sy_nredo;           // items of this workgroup handed over so far (their indices: p.redo[lo ..])

    const Lane<D, TK, D> L(p);
    const int lo = p.list_ptr[blockIdx.x], hi = p.list_ptr[blockIdx.x + 1];

    // ---- waits: bounded spins on an LDS word
    bool dead = false;   // wave-uniform
    // The spin itself is one block of assembly: a loop in the source here, inside the tile loop, makes the register allocator
    // spill the queries around it.  Leaves with 0 when the word has the wanted value (>= it with at_least), with 1 (if `watch`)
    // when all eight waves are through with some slot's tile and somebody has to recycle it, with 2 when the workgroup's abort flag is up or after SPIN_LIMIT polls.
    auto spin = [&](const int* word, const int want, const bool at_least, const bool watch) __attribute__((always_inline)) {
        const unsigned a_word = lds_addr(word), a_abort = lds_addr(&sy_abort), a_next = lds_addr(sy_done);
        int t0, t1, n0, n1, n2, n3, v, ab, code, cnt = p.spin_limit;
#define SPIN_ASM(CMP, WATCH)                                                                                                                         \
    asm volatile("1:\n\tds_read_b32 %0, %10\n\tds_read_b32 %1, %11\n\tds_read_b32 %2, %12\n\tds_read_b32 %3, %12 offset:4\n\t"                     \
                 "ds_read_b32 %4, %12 offset:8\n\tds_read_b32 %5, %12 offset:12\n\ts_waitcnt lgkmcnt(0)\n\t"                                        \
                 "v_readfirstlane_b32 %6, %0\n\tv_readfirstlane_b32 %7, %1\n\ts_mov_b32 %8, 0\n\t" CMP " %6, %13\n\ts_cbranch_scc1 2f\n\t"      \
                 "s_mov_b32 %8, 2\n\ts_cmp_lg_u32 %7, 0\n\ts_cbranch_scc1 2f\n\ts_sub_u32 %9, %9, 1\n\ts_cmp_eq_u32 %9, 0\n\ts_cbranch_scc1 2f\n\t" \
                 WATCH "s_sleep 1\n\ts_branch 1b\n2:"                                                                                               \
                 : "=&v"(t0), "=&v"(t1), "=&v"(n0), "=&v"(n1), "=&v"(n2), "=&v"(n3), "=&s"(v), "=&s"(ab), "=&s"(code), "+s"(cnt)                     \
                 : "v"(a_word), "v"(a_abort), "v"(a_next), "s"(want), "n"(NW)                                                                       \
                 : "memory", "scc", "vcc")
#define SPIN_WATCH "s_mov_b32 %8, 1\n\tv_cmp_eq_u32_e32 vcc, %c14, %2\n\ts_cbranch_vccnz 2f\n\tv_cmp_eq_u32_e32 vcc, %c14, %3\n\ts_cbranch_vccnz 2f\n\tv_cmp_eq_u32_e32 vcc, %c14, %4\n\ts_cbranch_vccnz 2f\n\tv_cmp_eq_u32_e32 vcc, %c14, %5\n\ts_cbranch_vccnz 2f\n\t"
        if (at_least) {
            if (watch) SPIN_ASM("s_cmp_ge_i32", SPIN_WATCH); else SPIN_ASM("s_cmp_ge_i32", "");
        } else {
            if (watch) SPIN_ASM("s_cmp_eq_u32", SPIN_WATCH); else SPIN_ASM("s_cmp_eq_u32", "");
        }
#undef SPIN_ASM
#undef SPIN_WATCH
        if (code == 2) {
            lds_store(&sy_abort, 1);
            dead = true;
        }
        return make_int2(code, v);
    };
    // wait for the descriptors (wave 0 writes them far ahead: a wait here is the exception)
    auto wait_gen = [&](const int want) __attribute__((always_inline)) {
        const int v = __builtin_amdgcn_readfirstlane(lds_load(&sy_gen));
        if (v >= want) return v;
        return spin(&sy_gen, want, true, false).y;
    };

    // ---- prologue: sync words, the workgroup's tile count, the first descriptors
    if (threadIdx.x < MAX_SLOT) {
        sy_done[threadIdx.x] = 0;
        sy_issued[threadIdx.x] = (int)threadIdx.x;
        if (threadIdx.x < NSLOT) *(int*)(ring + threadIdx.x * G::BUFB + G::KTILEB + G::VTILEB + 768) = -1;   // the slot's flag: no generation yet
    }
    if (threadIdx.x < 16) sy_redo[threadIdx.x] = 0;
    if (threadIdx.x == 0) { sy_gen = 0; sy_abort = 0; sy_gave_up = 0; sy_ntiles = 0; sy_nredo = 0; }
    __syncthreads();

    // descriptor generator (wave 0): items lo .. hi - 1, each item's plan entries in chunks of at most 64
    int gi = lo, ge = 0, gen = 0;   // next chunk: item, first entry inside it; descriptors written
    int pn = 0, p_first = 0, p_last = 0, p_tz = 0, p_item = 0;   // the requested chunk
    int pidx = 0, pbits = 0;
    auto gen_request = [&]() __attribute__((always_inline)) {   // loads of the next chunk's entries
        if (pn == 0 && gi < hi) {
            const int4 it = p.items[gi];
            const int t = __builtin_amdgcn_readfirstlane(it.x), e0 = __builtin_amdgcn_readfirstlane(it.y), z = __builtin_amdgcn_readfirstlane(it.z);
            const int ne = z & 0xfffff;
            const int n = ne - ge < 64 ? ne - ge : 64;
            const int gl = fresh_lane_id();
            if (gl < n) {
                pidx = p.kv_idx[e0 + ge + gl];
                pbits = (int)p.kv_bits[e0 + ge + gl];
            }
            pn = n;
            p_first = ge == 0;
            p_last = ge + n == ne;
            p_tz = t | (int)((unsigned)z >> 20 << 20);
            p_item = gi;
            ge += n;
            if (ge >= ne) { gi++; ge = 0; }
        }
    };
    auto gen_write = [&]() __attribute__((always_inline)) {   // descriptors of the requested chunk
        if (pn > 0) {
            const int gl = fresh_lane_id();
            if (gl < pn) {
                unsigned b = (unsigned)pbits & 0xffffu;
                if (p_first && gl == 0) b |= DESC_FIRST;
                if (p_last && gl == pn - 1) b |= DESC_LAST;
                desc[(gen + gl) & (NDESC - 1)] = make_int4(pidx, (int)b, p_tz, p_item);
            }
            gen += pn;
            pn = 0;
            lds_store(&sy_gen, gen);
        }
    };
    if (L.w == 0) {
        int nt = 0;
        for (int i = lo + L.lane; i < hi; i += 64) nt += p.items[i].z & 0xfffff;
        for (int off = 32; off > 0; off >>= 1) nt += __shfl_xor(nt, off);
        nt = __builtin_amdgcn_readfirstlane(nt);
        if (L.lane == 0) sy_ntiles = nt;
        while (gen < GEN_AHEAD && (gi < hi || pn > 0)) {
            gen_request();
            gen_write();
        }
        gen_request();
    }
    __syncthreads();
    const int ntiles = __builtin_amdgcn_readfirstlane(sy_ntiles);
    if (ntiles == 0) return;
    int gen_seen = __builtin_amdgcn_readfirstlane(lds_load(&sy_gen));

    auto read_desc = [&](const int j) __attribute__((always_inline)) {   // j < gen_seen
        const int4 d = desc[j & (NDESC - 1)];
        return make_int4(__builtin_amdgcn_readfirstlane(d.x), __builtin_amdgcn_readfirstlane(d.y), __builtin_amdgcn_readfirstlane(d.z),
                         __builtin_amdgcn_readfirstlane(d.w));
    };
    auto need_desc = [&](const int j) __attribute__((always_inline)) {
        if (j >= gen_seen) gen_seen = wait_gen(j + 1);
    };
    auto issue = [&](const int j, const int4& d) __attribute__((always_inline)) {
        const int kvh = (int)((unsigned)d.z >> 20) * HPI / p.group;
        // the per-lane parts of the source addresses are recomputed here: kept in registers they are spilled across the tile loop
        using GK = Geo<D, TK>;
        const int lane = fresh_lane_id();
        const unsigned lane_k = (unsigned)((lane / GK::CPR) * GK::NREG * p.k_tok * 2 + (lane % GK::CPR) * 16);
        const unsigned lane_v = (unsigned)((lane / GK::CPR) * GK::NREG * p.v_tok * 2 + (lane % GK::CPR) * 16);
        issue_tile_wave<D, WIN, TK>(p, lds_addr(ring + (j & (NSLOT - 1)) * G::BUFB), d.x, kvh, j / NSLOT + 1, lane, lane_k, lane_v);
    };

    // When all eight waves are through with a slot's tile (its count stands at 8), whichever wave comes by first recycles the slot:
    // it takes the count back to 0 (compare-and-swap: one winner) and requests the tile NSLOT places further on.  Not the last
    // wave through by design: that one is the wave the others are waiting for.  n0..n3 = sy_done as read a moment ago.
    auto claim = [&](const int n0, const int n1, const int n2, const int n3) __attribute__((always_inline)) {
        if (n0 == NW || n1 == NW || n2 == NW || n3 == NW) {
            const int sl = n0 == NW ? 0 : n1 == NW ? 1 : n2 == NW ? 2 : 3;
            int got = 0;
            if (fresh_lane_id() == 0) {
                int expect = NW;
                got = __hip_atomic_compare_exchange_strong(&sy_done[sl], &expect, 0, __ATOMIC_ACQ_REL, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            if (__builtin_amdgcn_readfirstlane(got)) {
                const int jn = __builtin_amdgcn_readfirstlane(lds_peek(&sy_issued[sl])) + NSLOT;   // only a winner writes this word
                if (jn < ntiles) {
                    need_desc(jn);
                    if (!dead) {
                        lds_store(&sy_issued[sl], jn);
                        issue(jn, read_desc(jn));
                    }
                }
            }
        }
    };
    auto try_issue = [&]() __attribute__((always_inline)) {
        const i32x4 nx = lds_peek4(sy_done);
        claim(__builtin_amdgcn_readfirstlane(nx[0]), __builtin_amdgcn_readfirstlane(nx[1]), __builtin_amdgcn_readfirstlane(nx[2]), __builtin_amdgcn_readfirstlane(nx[3]));
    };
    // wait for a slot's flag or recycling, lending a hand meanwhile: a round of the spin ends when the word is there, or with a
    // tile to request (then request it and go back to waiting)
    auto wait_watch = [&](const int* word, const int want) __attribute__((always_inline)) {
        if (__builtin_amdgcn_readfirstlane(lds_load(word)) == want) return;
#pragma unroll
        for (int round = 0; round < NSLOT + 2; round++) {
            const int code = spin(word, want, false, round < NSLOT + 1).x;
            if (code != 1) break;
            try_issue();
        }
    };

    // the first NSLOT tiles: one wave each
    if (L.w < NSLOT && L.w < ntiles) issue(L.w, read_desc(L.w));

    // ---- per-item state of this wave
    bf16x8 qf[NS];
    int art_q = -1, pos_q = 0;
    float M = -INFINITY, l = 0.f;
    bool viol = false;
    int iseq = 0;   // items begun

    auto load_q = [&](const int tz) __attribute__((always_inline)) {
        const int lane = fresh_lane_id();
        const int tok = (tz & 0xfffff) * SPINF_QTILE + 32 * L.wr + (lane & 31);
        const int tok_c = tok < p.n ? tok : p.n - 1;
        const int h = (int)((unsigned)tz >> 20) * HPI + L.wh;
        const __bf16* qp = p.q + (long)tok_c * p.q_tok + (long)h * p.q_head + 8 * (lane >> 5);
#pragma unroll
        for (int s = 0; s < NS; s++) qf[s] = *(const bf16x8*)(qp + 16 * s);
        art_q = tok < p.n ? p.art[tok_c] : -1;
        pos_q = WIN ? p.pos[tok_c] : 0;
    };
    auto reset_acc = [&]() __attribute__((always_inline)) {
        M = -INFINITY;
        l = 0.f;
        acc_zero<NDT>();
        viol = false;
    };
    // normalise O^T and store it as rows: 32 rows x 32 head dims at a time through the wave's own LDS slice, 16-byte pieces out
    // (pieces of 8 bytes straight from the registers were measured slower: twice the requests for the same bytes)
    auto store_rows = [&](const int tz) __attribute__((always_inline)) {
        const int lane = fresh_lane_id(), m = lane & 31, g = lane >> 5;
        const int tok0 = (tz & 0xfffff) * SPINF_QTILE + 32 * L.wr;
        const int h = (int)((unsigned)tz >> 20) * HPI + L.wh;
        const float inv = 1.0f / lane32_sum(l);
        __bf16* ob = p.o + (long)h * p.o_head;
        char* const stage = stage_all + L.w * 32 * SROW;
        asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");   // the last MFMAs' results -> v_accvgpr_read
        // tile dt is read back from the slice while tile dt + 1 is converted and written to it (the LDS takes a wave's requests
        // in order, so the write behind the read is safe), and stored after that: no wait between a write and its read-back
        auto put = [&](auto dt_c) __attribute__((always_inline)) {
            constexpr int dt = decltype(dt_c)::value;
            float r16[16];
            acc_read<dt>(r16);
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                bf16x4 r;
#pragma unroll
                for (int jj = 0; jj < 4; jj++) r[jj] = (__bf16)(r16[4 * i4 + jj] * inv);
                *(bf16x4*)(stage + m * SROW + (8 * i4 + 4 * g) * 2) = r;
            }
        };
        auto round = [&](auto dt_c) __attribute__((always_inline)) {
            constexpr int dt = decltype(dt_c)::value;
            bf16x8 val[2];
#pragma unroll
            for (int jj = 0; jj < 2; jj++) {
                const int c = jj * 64 + lane;
                val[jj] = *(const bf16x8*)(stage + (c >> 2) * SROW + (c & 3) * 16);
            }
            if constexpr (dt + 1 < NDT) put(std::integral_constant<int, dt + 1>{});
#pragma unroll
            for (int jj = 0; jj < 2; jj++) {
                const int c = jj * 64 + lane, row = c >> 2, col = c & 3;
                if (tok0 + row < p.n) *(bf16x8*)(ob + (long)(tok0 + row) * p.o_tok + 32 * dt + col * 8) = val[jj];
            }
        };
        put(std::integral_constant<int, 0>{});
        pv_steps<NDT>(round);
    };

    {   // the first item's queries
        need_desc(0);
        if (!dead) load_q(read_desc(0).z);
    }

    // ---- the tile sequence: item after item.
    // What a wave needs to know at the top of a tile (the tile's descriptor, the slots waiting for requests, the tile's flag) is
    // read from LDS while the previous tile's last MFMAs run (`pf_*`), and the wave counts itself through with a tile as soon as
    // its last fragment read of the tile is on its way: in the steady state no LDS round trip is waited for.
    int j = 0;
    bool have_pf = false;
    int4 pf_d = make_int4(0, 0, 0, 0);
    int pf_n0 = 0, pf_n1 = 0, pf_n2 = 0, pf_n3 = 0, pf_flag = -1;
    auto flag_word = [&](const int jj) __attribute__((always_inline)) { return (const int*)(ring + (jj & (NSLOT - 1)) * G::BUFB + G::KTILEB + G::VTILEB + 768); };
    while (j < ntiles && !dead) {
        reset_acc();
        iseq++;
        int4 d = make_int4(0, 0, 0, 0);
        bool last = false;
        do {
            const int s = j & (NSLOT - 1);
            int n0, n1, n2, n3, flag;
            if (have_pf) {
                d = pf_d; n0 = pf_n0; n1 = pf_n1; n2 = pf_n2; n3 = pf_n3; flag = pf_flag;
            } else {
                need_desc(j);
                if (dead) break;
                const int4 dv = desc[j & (NDESC - 1)];
                const i32x4 nx = lds_peek4(sy_done);
                const int fv = lds_peek(flag_word(j));
                d = make_int4(__builtin_amdgcn_readfirstlane(dv.x), __builtin_amdgcn_readfirstlane(dv.y), __builtin_amdgcn_readfirstlane(dv.z), __builtin_amdgcn_readfirstlane(dv.w));
                n0 = __builtin_amdgcn_readfirstlane(nx[0]); n1 = __builtin_amdgcn_readfirstlane(nx[1]);
                n2 = __builtin_amdgcn_readfirstlane(nx[2]); n3 = __builtin_amdgcn_readfirstlane(nx[3]);
                flag = __builtin_amdgcn_readfirstlane(fv);
            }
            have_pf = false;
            // The waves of the second head set run behind those of the first (a SIMD's arbiter favours its older wave), and the
            // kernel ends when they do: they leave the recycling to the first set, which is ahead and mostly waiting for
            // flags anyway, and lend a hand only from inside a wait.
            if (L.w < 4) claim(n0, n1, n2, n3);
            if (dead) break;
            const unsigned bits = (unsigned)d.y;
            last = (bits & DESC_LAST) != 0;
            // the tile's 32-key blocks that this wave's rows see something of (one bit per block)
            const unsigned ab = (bits >> (2 * L.wr)) & (NSUB == 2 ? 3u : 1u);
            const bool act = ab != 0;
            if (act) {
                if (flag != ((j / NSLOT + 1) & 63)) wait_watch(flag_word(j), (j / NSLOT + 1) & 63);
                if (dead) break;
                // fragment addresses from a fresh lane index (kept in registers across the tile loop they are spilled, and a reload
                // waits for every tile request in flight): K row lane % 32 of the block, 16-byte chunk lane / 32 of each 32-byte step;
                // V^T as ds_read_b64_tr_b16 wants it (see Lane in attn_kernels.h)
                const int ln = fresh_lane_id();
                const char* buf = ring + s * G::BUFB;
                // what the next tile's top needs, fetched under the last block's P V products
                int4 dv = make_int4(0, 0, 0, 0);
                i32x4 nx = {0, 0, 0, 0};
                int fv = -1;
                const bool pf_ok = j + 1 < ntiles && j + 1 < gen_seen;
                // one 32-key block: K Q^T, mask, softmax, P V.  TAIL: the last block of the tile that this wave computes
                auto block = [&](const int sub, auto tail_c) __attribute__((always_inline)) {
                    constexpr bool TAIL = decltype(tail_c)::value;
                    const char* krow = buf + G::K::k_off(ln & 31) + 16 * (ln >> 5) + sub * G::KSUB;
                    const char* vrow = buf + G::KTILEB + G::V::v_off(4 * (ln >> 5) + ((ln >> 2) & 3)) + 32 * ((ln >> 4) & 1) + 8 * (ln & 3) + sub * G::VSUB;
                    // S^T = K Q^T
                    f32x16 sa;
                    {
                        bf16x8 kf[PF];
#pragma unroll
                        for (int x = 0; x < PF; x++) kf[x] = *(const bf16x8*)(krow + 32 * x);
                        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                        for (int x = 0; x < NS; x++) {
                            if (x == 0) qk_first(sa, kf[x % PF], qf[x]);
                            else if (x == NS - 1) qk_last(sa, kf[x % PF], qf[x]);
                            else qk_next(sa, kf[x % PF], qf[x]);
                            if (x + PF < NS) kf[x % PF] = *(const bf16x8*)(krow + 32 * (x + PF));
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                    if ((bits >> (8 + 2 * L.wr + sub)) & 1u) {
                        f32x16 sm[1] = {sa};
                        const int tok = (d.z & 0xfffff) * SPINF_QTILE + 32 * L.wr + (ln & 31);
                        apply_mask<1, WIN, 0, TK>(sm, (const int*)(buf + G::KTILEB + G::VTILEB), d.x, sub, ln >> 5, tok, art_q, pos_q, p.window);
                        sa = sm[0];
                    }
                    // softmax against the row's fixed reference (the maximum of the first block it sees a key in)
                    bf16x8 pb[2];
                    {
                        const bool first = M == -INFINITY;
                        if (__builtin_amdgcn_ballot_w64(first) != 0) {   // only where a row meets its first keys (see the lockstep kernel)
                            float mx = sa[0];
#pragma unroll
                            for (int i2 = 1; i2 < 16; i2++) mx = fmaxf(mx, sa[i2]);
                            mx = lane32_max(mx);
                            M = first ? mx * p.c : M;
                        }
                        const float ms = M == -INFINITY ? 0.f : M;
                        float sum = 0.f;
#pragma unroll
                        for (int i2 = 0; i2 < 16; i2++) {
                            const float pr = __builtin_amdgcn_exp2f(__builtin_fmaf(sa[i2], p.c, -ms));
                            sum += pr;
                            pb[i2 >> 3][i2 & 7] = (__bf16)pr;
                        }
                        l += sum;
                        viol = viol | !(sum <= VIOL_SUM);
                    }
                    // O^T += V^T P^T, with what the next tile's top needs fetched meanwhile; once the last fragment read is on its way,
                    // count this wave through with the tile
                    // (requested before the first transposing read of V, so that every wait inside the MFMA sequence is for V
                    // fragments alone and stalls: a wait that is already satisfied takes no time, and then a vector write of an
                    // operand could end up in the issue cycle before the assembly MFMA that reads it; LDS reads of different kinds
                    // do return in issue order, spinf_diag_lds_order checks it)
                    if (TAIL && pf_ok) {
                        dv = desc[(j + 1) & (NDESC - 1)];
                        nx = lds_peek4(sy_done);
                        fv = lds_peek(flag_word(j + 1));
                    }
                    {
                        s16x4 vlo[VPF], vhi[VPF];
                        auto vload = [&](const int f, const int slot) __attribute__((always_inline)) {
                            const char* vp = vrow + G::V::v_off(16 * (f / NDT)) + 64 * (f % NDT);
                            vlo[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)vp);
                            vhi[slot] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vp + G::V::v_off(8)));
                        };
#pragma unroll
                        for (int f = 0; f < VPF; f++) vload(f, f);
                        __builtin_amdgcn_sched_barrier(0);
                        // (head dim 128 reads all of a block's V fragments ahead, and the compiler then sinks the conversions that write
                        // the P fragments below those reads, right in front of the first MFMA, which would multiply the registers' old
                        // contents: one instruction in between)
                        if constexpr (VPF >= NVF) asm volatile("s_nop 0" ::: "memory");
                        auto step = [&](auto f_c) __attribute__((always_inline)) {
                            constexpr int f = decltype(f_c)::value;
                            const bf16x8 a = __builtin_bit_cast(bf16x8, __builtin_shufflevector(vlo[f % VPF], vhi[f % VPF], 0, 1, 2, 3, 4, 5, 6, 7));
                            acc_mfma<f % NDT>(a, pb[f / NDT]);
                            if (f + VPF < NVF) vload(f + VPF, f % VPF);
                            if (TAIL && f == DONE_AT) {   // that was the tile's last fragment read
                                if (fresh_lane_id() == 0) __hip_atomic_fetch_add(&sy_done[s], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        };
                        pv_steps<NVF>(step);
                    }
                };
                if constexpr (NSUB == 1) {
                    block(0, std::true_type{});
                } else {
                    if (ab == 3u) {
                        block(0, std::false_type{});
                        block(1, std::true_type{});
                    } else {
                        block((int)(ab >> 1), std::true_type{});
                    }
                }
                if (pf_ok) {
                    pf_d = make_int4(__builtin_amdgcn_readfirstlane(dv.x), __builtin_amdgcn_readfirstlane(dv.y), __builtin_amdgcn_readfirstlane(dv.z), __builtin_amdgcn_readfirstlane(dv.w));
                    pf_n0 = __builtin_amdgcn_readfirstlane(nx[0]); pf_n1 = __builtin_amdgcn_readfirstlane(nx[1]);
                    pf_n2 = __builtin_amdgcn_readfirstlane(nx[2]); pf_n3 = __builtin_amdgcn_readfirstlane(nx[3]);
                    pf_flag = __builtin_amdgcn_readfirstlane(fv);
                    have_pf = true;
                }
            } else {
                // nothing of this tile for these rows: the slot must have been recycled for it before this wave counts itself through
                wait_watch(&sy_issued[s], j);
                if (dead) break;
                if (fresh_lane_id() == 0) __hip_atomic_fetch_add(&sy_done[s], 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            // wave 0 keeps the descriptors ahead
            if (L.w == 0 && gen - j < GEN_AHEAD) {
                gen_write();
                gen_request();
            }
            j++;
        } while (!last);
        if (dead) break;
        // this wave's rows of the item are complete: the next item's queries are requested (their registers are free), then the rows
        // go out (or the item goes to the exact pass)
        const bool hand_over = __builtin_amdgcn_ballot_w64(viol) != 0;   // scores ranged too widely somewhere in these 32 rows
        const int tz_done = d.z, item_done = d.w;
        if (j < ntiles) {
            need_desc(j);
            if (dead) break;
            load_q(read_desc(j).z);
        }
        if (hand_over) {
            if (fresh_lane_id() == 0) {
                const int was = __hip_atomic_fetch_max(&sy_redo[iseq & 15], iseq, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                if (was < iseq) {   // first wave of the item to say so: the workgroup recomputes the item after its list (below)
                    const int k = __hip_atomic_fetch_add(&sy_nredo, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_store(&p.redo[lo + k], item_done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        } else {
            store_rows(tz_done);
        }
    }
    if (dead && fresh_lane_id() == 0) __hip_atomic_fetch_add(&sy_gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);   // (the list is done again below)
    __builtin_amdgcn_s_waitcnt(0x0f70);

    // ---- after the list: normally nothing.  Items in which some row met scores too far above its reference are done again, exactly,
    // by ring_paced_pass; and if some wave gave up a wait (every wave has then left the ring), so is the whole list, with the ring
    // pass's own arithmetic: an abort costs time, never rows.
    __syncthreads();   // every wave is through with its list: the ring is free, the hand-overs are all in
    const bool gave_up = __builtin_amdgcn_readfirstlane(lds_load(&sy_abort)) != 0;
    if (!gave_up && __builtin_amdgcn_readfirstlane(lds_load(&sy_nredo)) == 0) return;
    __shared__ int sy_vote;
    if (gave_up) {   // some wave gave up a wait: the whole list again, one tile at a time between barriers (same bits)
        if (threadIdx.x == 0) {
            sy_nredo = 0;   // (whatever the list needs recomputed exactly is found again on the way)
            atomicAdd(&p.counters[NLIST + 4], lds_load(&sy_gave_up));   // running total, for spinf_attn_ring_aborts
        }
    }
    if (threadIdx.x == 0) sy_vote = 0;
    __syncthreads();
    ring_paced_pass<D, WIN>(p, ring, stage_all, &sy_nredo, &sy_vote, lo, gave_up ? hi : lo, lo);
}

template <int D, bool WIN>
int launch_ring_t(const AttnParams& p, int n_wg, hipStream_t stream) {
    hipLaunchKernelGGL((tree_attn_ring_kernel<D, WIN>), dim3(n_wg), dim3(D == 512 ? 256 : 512), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "tree_attn: launch (ring kernel): %s", hipGetErrorString(e));
    return SPINF_OK;
}

}  // namespace

int spinf_launch_ring(const AttnParams& p, int d, bool win, int n_wg, hipStream_t stream) {
    if (d == 128) return win ? launch_ring_t<128, true>(p, n_wg, stream) : launch_ring_t<128, false>(p, n_wg, stream);
    if (d == 256) return win ? launch_ring_t<256, true>(p, n_wg, stream) : launch_ring_t<256, false>(p, n_wg, stream);
    if (d == 512) return win ? launch_ring_t<512, true>(p, n_wg, stream) : launch_ring_t<512, false>(p, n_wg, stream);
    return spinf_fail(SPINF_E_ARG, "tree_attn: the ring kernel takes head dim 128, 256 or 512, not %d", d);
}
