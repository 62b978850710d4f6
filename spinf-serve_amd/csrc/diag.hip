// Yardstick kernels of the library's benchmark, for gfx950 (MI355X): what the matrix cores sustain on this part when nothing else
// is in the way.  No counterpart in the reference.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"
#include "attn_kernels.h"
#include "attn_ring_io.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

namespace {

constexpr int MFMA_PER_ITER = 8;   // independent accumulators: the pipe never waits for a result

// Eight waves per workgroup, two per SIMD, as the attention kernels run; every wave issues iters x 8 v_mfma_f32_32x32x16_bf16 on
// eight independent accumulators with operands that stay in registers.
__global__ __launch_bounds__(512) void mfma_rate_kernel(const long iters, float* out) {
    bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = (__bf16)(0.001f * (float)((threadIdx.x + i) & 15));
        b[i] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + i) & 7));
    }
    f32x16 acc[MFMA_PER_ITER];
#pragma unroll
    for (int k = 0; k < MFMA_PER_ITER; k++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[k][i] = 0.f;
    for (long it = 0; it < iters; it++) {
#pragma unroll
        for (int k = 0; k < MFMA_PER_ITER; k++) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[k], 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < MFMA_PER_ITER; k++)
#pragma unroll
        for (int i = 0; i < 16; i++) s += acc[k][i];
    out[(long)blockIdx.x * blockDim.x + threadIdx.x] = s;   // keeps the loop alive
}

// ---- do a wave's vector instructions run in the shadow of its own MFMAs?
// Every wave runs iters x { one v_mfma_f32_32x32x16_bf16 (32 clocks of the matrix pipe) on a single accumulator, then NV vector
// instructions that depend on nothing the MFMA touches: v_fma_f32 (KIND 0) or v_exp_f32 (KIND 1) }, with one, two or four waves per
// SIMD (KIND 2: rounds shaped like a 32 x 32 attention block at head dim 128: 8 chained MFMAs, 3 NV v_fma_f32 + NV v_exp_f32, 8 MFMAs
// on four accumulators).  Every wave of workgroup 0 records the clock before and after its loop (s_memtime ticks, which count core clocks here: the bare
// MFMA chain reads 32.3 per MFMA).  If the vector instructions ran under the MFMA a wave would need max(36, 4 + 4 NV) clocks per round;
// measured on MI355X it needs 36 + 4 NV (8 NV for v_exp_f32): they do not, the two add up, and only ANOTHER wave of the SIMD can use
// the vector ALU while an MFMA runs.  This is what bounds the attention kernels at head dim 128, where a 32 x 32 block is 16 MFMAs
// (512 clocks) and about as many clocks of softmax per wave.
template <int NV, int KIND>
__global__ __launch_bounds__(1024) void mfma_valu_kernel(const int iters, long long* out) {
    bf16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = (__bf16)(0.001f * (float)((threadIdx.x + i) & 15));
        b[i] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + i) & 7));
    }
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; i++) v[i] = 0.5f + 0.01f * (float)i + 0.0001f * (float)(threadIdx.x & 63);
    const float c = 0.999f, d = 0.0001f;
    __syncthreads();
    const long long t0 = __builtin_readcyclecounter();
    f32x16 o[4];   // (KIND 2)
#pragma unroll
    for (int n = 0; n < 4; n++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[n][i] = 0.f;
    for (int it = 0; it < iters; it++) {
        if (KIND == 2) {   // an attention block's phases: 8 chained MFMAs, the softmax's vector instructions, 8 MFMAs on four accumulators
#pragma unroll
            for (int x = 0; x < 8; x++) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
#pragma unroll
            for (int j = 0; j < 3 * NV; j++) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[j % 16]) : "v"(c), "v"(d));
#pragma unroll
            for (int j = 0; j < NV; j++) asm volatile("v_exp_f32 %0, %0" : "+v"(v[j % 16]));
#pragma unroll
            for (int x = 0; x < 8; x++) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(o[x & 3]) : "v"(a), "v"(b));
            continue;
        }
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
#pragma unroll
        for (int j = 0; j < NV; j++) {
            if (KIND == 0) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[j % 16]) : "v"(c), "v"(d));
            else asm volatile("v_exp_f32 %0, %0" : "+v"(v[j % 16]));
        }
    }
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last MFMA's result -> vector ALU reads (assembly: the compiler adds no wait states)
    const long long t1 = __builtin_readcyclecounter();
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) sum += acc[i] + v[i] + o[0][i] + o[1][i] + o[2][i] + o[3][i];
    if (sum == 12345.678f) out[0] = 0;   // keeps the loop alive (never true)
    if (blockIdx.x == 0 && (threadIdx.x & 63) == 0) {
        out[2 * (threadIdx.x >> 6)] = t0;
        out[2 * (threadIdx.x >> 6) + 1] = t1;
    }
}

// ---- do LDS reads of different kinds return in the order they were issued?
// The attention and scan kernels mix three kinds of LDS reads in one wave: transposing 8-byte reads (ds_read_b64_tr_b16: V^T
// fragments), 16-byte reads (K fragments, key metadata, descriptors) and 4-byte reads, and wait for them with partial counts
// (s_waitcnt lgkmcnt(n): "all but the n youngest have returned"), which is only right if a wave's LDS reads return in issue order
// whatever their kind.  This kernel checks exactly that, under load: every wave issues eight reads of mixed kinds back to back,
// waits with the partial count an in-order LDS allows before it touches each result (registers poisoned beforehand, so a read that
// has not returned shows), and compares with the same reads done one at a time with a full wait.  Assembly throughout, so that the
// waits are the ones written here and nothing else.
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;
constexpr int LDS_ORDER_WORDS = 8192;    // 32 KB of pattern
constexpr int LDS_ORDER_PATTERNS = 6;

__device__ __forceinline__ void lds_rd_tr(u32x2& d, const unsigned addr) { asm volatile("ds_read_b64_tr_b16 %0, %1" : "+v"(d) : "v"(addr) : "memory"); }
__device__ __forceinline__ void lds_rd_16(u32x4& d, const unsigned addr) { asm volatile("ds_read_b128 %0, %1" : "+v"(d) : "v"(addr) : "memory"); }
template <int N>
__device__ __forceinline__ void lds_wait(u32x2& d) { asm volatile("s_waitcnt lgkmcnt(%c1)" : "+v"(d) : "n"(N) : "memory"); }
template <int N>
__device__ __forceinline__ void lds_wait(u32x4& d) { asm volatile("s_waitcnt lgkmcnt(%c1)" : "+v"(d) : "n"(N) : "memory"); }
__device__ __forceinline__ unsigned fold(const u32x2 d) { return d[0] * 3u + d[1]; }
__device__ __forceinline__ unsigned fold(const u32x4 d) { return ((d[0] * 3u + d[1]) * 3u + d[2]) * 3u + d[3]; }

// KINDS: bit k set = read k is a 16-byte read, clear = a transposing 8-byte read
template <unsigned KINDS, int K = 0>
__device__ __forceinline__ void lds_order_issue(u32x2 (&t)[8], u32x4 (&b)[8], const unsigned (&at)[8], const unsigned (&ab)[8]) {
    if constexpr (K < 8) {
        if constexpr ((KINDS >> K) & 1u) lds_rd_16(b[K], ab[K]);
        else lds_rd_tr(t[K], at[K]);
        lds_order_issue<KINDS, K + 1>(t, b, at, ab);
    }
}
template <unsigned KINDS, int K = 0>
__device__ __forceinline__ void lds_order_take(u32x2 (&t)[8], u32x4 (&b)[8], unsigned (&got)[8]) {
    if constexpr (K < 8) {
        if constexpr ((KINDS >> K) & 1u) {
            lds_wait<7 - K>(b[K]);
            got[K] = fold(b[K]);
        } else {
            lds_wait<7 - K>(t[K]);
            got[K] = fold(t[K]);
        }
        lds_order_take<KINDS, K + 1>(t, b, got);
    }
}
template <unsigned KINDS, int K = 0>
__device__ __forceinline__ void lds_order_serial(const unsigned (&at)[8], const unsigned (&ab)[8], unsigned (&want)[8]) {
    if constexpr (K < 8) {
        if constexpr ((KINDS >> K) & 1u) {
            u32x4 d = {0xdeadbeefu, 0xdeadbeefu, 0xdeadbeefu, 0xdeadbeefu};
            lds_rd_16(d, ab[K]);
            lds_wait<0>(d);
            want[K] = fold(d);
        } else {
            u32x2 d = {0xdeadbeefu, 0xdeadbeefu};
            lds_rd_tr(d, at[K]);
            lds_wait<0>(d);
            want[K] = fold(d);
        }
        lds_order_serial<KINDS, K + 1>(at, ab, want);
    }
}

template <unsigned KINDS>
__device__ __forceinline__ int lds_order_round(const unsigned base, const int it) {
    const unsigned lane = threadIdx.x & 63u;
    unsigned at[8], ab[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {   // strides that change with the round: conflict-free and conflicting patterns both come by
        at[k] = base + ((lane * 8u * (1u + (unsigned)((it + k) % 9)) + 64u * (unsigned)k * (unsigned)(it % 7 + 1)) & (LDS_ORDER_WORDS * 4u - 8u));
        ab[k] = base + ((lane * 16u * (1u + (unsigned)((it + 3 * k) % 5)) + 256u * (unsigned)k + 16u * (unsigned)(it % 11)) & (LDS_ORDER_WORDS * 4u - 16u));
    }
    u32x2 t[8];
    u32x4 b[8];
#pragma unroll
    for (int k = 0; k < 8; k++) {
        t[k] = u32x2{0xdeadbeefu, 0xdeadbeefu};
        b[k] = u32x4{0xdeadbeefu, 0xdeadbeefu, 0xdeadbeefu, 0xdeadbeefu};
    }
    unsigned got[8], want[8];
    lds_order_issue<KINDS>(t, b, at, ab);
    lds_order_take<KINDS>(t, b, got);
    lds_order_serial<KINDS>(at, ab, want);
    int bad = 0;
#pragma unroll
    for (int k = 0; k < 8; k++) bad += got[k] != want[k];
    return bad;
}

__global__ __launch_bounds__(256) void lds_order_kernel(const int iters, int* out) {
    __shared__ __attribute__((aligned(16))) unsigned pat[LDS_ORDER_WORDS];
    for (int i = threadIdx.x; i < LDS_ORDER_WORDS; i += blockDim.x) pat[i] = (unsigned)i * 2654435761u ^ ((unsigned)i >> 3) ^ (blockIdx.x * 40503u);
    __syncthreads();
    const unsigned base = (unsigned)(size_t)(const __attribute__((address_space(3))) unsigned*)pat;
    int bad[LDS_ORDER_PATTERNS] = {0, 0, 0, 0, 0, 0};
    for (int it = 0; it < iters; it++) {
        bad[0] += lds_order_round<0xaau>(base, it);   // T B T B T B T B
        bad[1] += lds_order_round<0x55u>(base, it);   // B T B T B T B T
        bad[2] += lds_order_round<0xf0u>(base, it);   // T T T T B B B B
        bad[3] += lds_order_round<0x0fu>(base, it);   // B B B B T T T T
        bad[4] += lds_order_round<0xccu>(base, it);   // T T B B T T B B
        bad[5] += lds_order_round<0x24u>(base, it);   // T T B T T B T T: a 16-byte read among transposing ones
    }
#pragma unroll
    for (int v = 0; v < LDS_ORDER_PATTERNS; v++)
        if (bad[v]) atomicAdd(&out[v], bad[v]);
    if (threadIdx.x == 0) atomicAdd(&out[LDS_ORDER_PATTERNS], 1);   // workgroups that ran
}

// ---- what must lie between a VALU write of an MFMA's A / B registers and the MFMA, and between the MFMA and the next VALU write of
// them?  The attention kernels issue their MFMAs from inline assembly (the accumulators live in registers the compiler must not see),
// so the compiler's hazard recogniser does not know that those blocks read their operands as an MFMA does: whatever wait states
// the hardware wants around them must come from the source.  Each case runs four MFMAs to have the matrix pipe busy, then the
// sequence under test with GAP independent instructions (s_nop) in between, and counts lanes whose 16 results are not the expected
// value.  KIND 0: v_mov writes B, then the MFMA reads it.  KIND 1: the MFMA reads B, then v_mov overwrites it.  KIND 2: as 0, but B
// comes out of v_exp_f32 -> v_cvt_pk_bf16_f32, the chain the softmax feeds the P V product with.  KIND 3: as 2, with other things
// in the gap: one satisfied s_waitcnt lgkmcnt(0), two of them, a satisfied s_waitcnt vmcnt(0), v_nop, s_waitcnt + s_nop 0.
typedef __attribute__((ext_vector_type(16))) float diag_f32x16;
constexpr int MFMA_HAZARD_GAPS = 5;     // 0, 1, 2, 4, 8 instructions
constexpr int MFMA_HAZARD_KINDS = 4;

#define SPINF_DIAG_FILL                                                                                                              \
    "v_mov_b32 v20, %1\n\tv_mov_b32 v21, %1\n\tv_mov_b32 v22, %1\n\tv_mov_b32 v23, %1\n\t"                                           \
    "v_mov_b32 v24, %1\n\tv_mov_b32 v25, %1\n\tv_mov_b32 v26, %1\n\tv_mov_b32 v27, %1\n\tv_mov_b32 v29, 1.0\n\ts_nop 7\n\t"          \
    "v_mfma_f32_32x32x16_bf16 v[32:47], v[20:23], v[24:27], 0\n\tv_mfma_f32_32x32x16_bf16 v[48:63], v[20:23], v[24:27], 0\n\t"      \
    "v_mfma_f32_32x32x16_bf16 v[64:79], v[20:23], v[24:27], 0\n\tv_mfma_f32_32x32x16_bf16 v[80:95], v[20:23], v[24:27], 0\n\t"
#define SPINF_DIAG_CLOB                                                                                                              \
    "v20", "v21", "v22", "v23", "v24", "v25", "v26", "v27", "v28", "v29", "v32", "v33", "v34", "v35", "v36", "v37", "v38", "v39", "v40", "v41", "v42",   \
        "v43", "v44", "v45", "v46", "v47", "v48", "v49", "v50", "v51", "v52", "v53", "v54", "v55", "v56", "v57", "v58", "v59", "v60", "v61", "v62",     \
        "v63", "v64", "v65", "v66", "v67", "v68", "v69", "v70", "v71", "v72", "v73", "v74", "v75", "v76", "v77", "v78", "v79", "v80", "v81", "v82",     \
        "v83", "v84", "v85", "v86", "v87", "v88", "v89", "v90", "v91", "v92", "v93", "v94", "v95", "memory"
#define SPINF_DIAG_WRITE_B "v_mov_b32 v24, %2\n\tv_mov_b32 v25, %2\n\tv_mov_b32 v26, %2\n\tv_mov_b32 v27, %2\n\t"
#define SPINF_DIAG_CVT_B                                                                                                             \
    "v_exp_f32 v28, v29\n\ts_nop 0\n\tv_cvt_pk_bf16_f32 v24, v28, v28\n\tv_cvt_pk_bf16_f32 v25, v28, v28\n\t"                        \
    "v_cvt_pk_bf16_f32 v26, v28, v28\n\tv_cvt_pk_bf16_f32 v27, v28, v28\n\t"
#define SPINF_DIAG_MFMA "v_mfma_f32_32x32x16_bf16 %0, v[20:23], v[24:27], 0\n\t"
#define SPINF_DIAG_DRAIN "s_nop 15\n\ts_nop 15\n\t"

template <int KIND>
__device__ __forceinline__ int mfma_hazard_bad(const diag_f32x16 acc) {
    const float want = KIND == 1 ? 16.f : 32.f;   // 16 products of 1 x 1, or of 1 x 2
    bool bad = false;
#pragma unroll
    for (int i = 0; i < 16; i++) bad = bad || acc[i] != want;
    return bad ? 1 : 0;
}
#define SPINF_DIAG_CASE(KIND, G, GAPTEXT)                                                                                            \
    {                                                                                                                                \
        diag_f32x16 acc;                                                                                                             \
        if (KIND == 0) asm volatile(SPINF_DIAG_FILL SPINF_DIAG_WRITE_B GAPTEXT SPINF_DIAG_MFMA SPINF_DIAG_DRAIN : "=&v"(acc) : "v"(one2), "v"(two2) : SPINF_DIAG_CLOB);   \
        if (KIND == 1) asm volatile(SPINF_DIAG_FILL SPINF_DIAG_MFMA GAPTEXT SPINF_DIAG_WRITE_B SPINF_DIAG_DRAIN : "=&v"(acc) : "v"(one2), "v"(two2) : SPINF_DIAG_CLOB);   \
        if (KIND >= 2) asm volatile(SPINF_DIAG_FILL SPINF_DIAG_CVT_B GAPTEXT SPINF_DIAG_MFMA SPINF_DIAG_DRAIN : "=&v"(acc) : "v"(one2), "v"(two2) : SPINF_DIAG_CLOB);     \
        bad[KIND * MFMA_HAZARD_GAPS + G] += mfma_hazard_bad<KIND>(acc);                                                              \
    }
#define SPINF_DIAG_KIND(KIND)                                                                                                        \
    SPINF_DIAG_CASE(KIND, 0, "")                                                                                                     \
    SPINF_DIAG_CASE(KIND, 1, "s_nop 0\n\t")                                                                                          \
    SPINF_DIAG_CASE(KIND, 2, "s_nop 1\n\t")                                                                                          \
    SPINF_DIAG_CASE(KIND, 3, "s_nop 3\n\t")                                                                                          \
    SPINF_DIAG_CASE(KIND, 4, "s_nop 7\n\t")

__global__ __launch_bounds__(512) void mfma_hazard_kernel(const int iters, int* out) {
    const unsigned one2 = 0x3f803f80u, two2 = 0x40004000u;   // bf16 pairs of 1.0 and 2.0
    int bad[MFMA_HAZARD_KINDS * MFMA_HAZARD_GAPS] = {};
    for (int it = 0; it < iters; it++) {
        SPINF_DIAG_KIND(0)
        SPINF_DIAG_KIND(1)
        SPINF_DIAG_KIND(2)
        SPINF_DIAG_CASE(3, 0, "s_waitcnt lgkmcnt(0)\n\t")
        SPINF_DIAG_CASE(3, 1, "s_waitcnt lgkmcnt(0)\n\ts_waitcnt lgkmcnt(0)\n\t")
        SPINF_DIAG_CASE(3, 2, "s_waitcnt vmcnt(0)\n\t")
        SPINF_DIAG_CASE(3, 3, "v_nop\n\t")
        SPINF_DIAG_CASE(3, 4, "s_waitcnt lgkmcnt(0)\n\ts_nop 0\n\t")
    }
#pragma unroll
    for (int v = 0; v < MFMA_HAZARD_KINDS * MFMA_HAZARD_GAPS; v++)
        if (bad[v]) atomicAdd(&out[v], bad[v]);
    if (threadIdx.x == 0) atomicAdd(&out[MFMA_HAZARD_KINDS * MFMA_HAZARD_GAPS], 1);
}

// ---- the byte pattern of a tree-attention pass with nothing computed: what does moving the data alone cost?
// The same work items in the same static lists as the kernel with decoupled waves (tree_attn_ring.hip, head dim 256, two heads
// per item, eight waves): per item every wave loads the queries of its 32 rows (16 bytes per lane and contraction step), every
// 32-key K / V tile of the item's plan entries comes into a four-slot LDS ring by the same whole-wave DMA requests
// (issue_tile_wave, four tiles in flight, issued by waves 0 .. 3, the landing flag written by the DMA itself), and at the item's
// end every wave writes its 32 output rows in the kernel's store pattern (16-byte pieces, four lanes to a row's 64 bytes).
// No MFMA, no softmax, no mask, no LDS fragment reads: the outputs are a constant.  One workgroup barrier per tile keeps the
// ring's slots in order, which costs nothing here (the waves have nothing else to do).  status[0] += waves that gave up a bounded
// wait (never), status[1] += tiles seen landed.  parts: 1 = the K / V tiles only, 2 = the queries and outputs only, 3 = both;
// nslot (1 .. 4): slots of the ring in use = tile requests in flight.  parts 5: the tiles only, with every tile's requests dealt out
// over the eight waves and awaited by request count and barrier, as the lockstep kernel does (one wave per tile otherwise); parts 7:
// the whole pattern that way, with a landing flag per wave.
template <int D>
__global__ __launch_bounds__(512) void attn_stream_kernel(const AttnParams p, int* status, const int parts, const int nslot) {
    using G = TileGeo<D, 32, D>;
    using GK = Geo<D, 32>;
    constexpr int NSLOT = 4, NS = D / 16, NDT = D / 32, HPI = 2;
    __shared__ __attribute__((aligned(16))) char ring[NSLOT * G::BUFB];
    __shared__ int sy_abort;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wh = w >> 2, wr = w & 3;
    const int lo = p.list_ptr[blockIdx.x], hi = p.list_ptr[blockIdx.x + 1];
    auto flag_word = [&](const int slot) { return (int*)(ring + slot * G::BUFB + G::KTILEB + G::VTILEB + 768); };
    if (threadIdx.x < NSLOT * 64) flag_word(threadIdx.x >> 6)[threadIdx.x & 63] = 0;
    if (threadIdx.x == 0) sy_abort = 0;
    int total = 0;
    for (int i = lo; i < hi; i++) total += __builtin_amdgcn_readfirstlane(p.items[i].z) & 0xfffff;
    __syncthreads();

    struct Cursor { int item, e, ne, e0, kvh, tz; };
    auto open = [&](Cursor& c) {
        while (c.item < hi) {
            const int4 it = p.items[c.item];
            c.e0 = __builtin_amdgcn_readfirstlane(it.y);
            const int z = __builtin_amdgcn_readfirstlane(it.z);
            c.ne = z & 0xfffff;
            c.kvh = (int)((unsigned)z >> 20) * HPI / p.group;
            c.tz = __builtin_amdgcn_readfirstlane(it.x) | (int)((unsigned)z >> 20 << 20);
            c.e = 0;
            if (c.ne > 0) break;
            c.item++;
        }
    };
    auto step = [&](Cursor& c) {
        if (++c.e >= c.ne) {
            c.item++;
            open(c);
        }
    };
    const int lane = fresh_lane_id();
    const unsigned lane_k = (unsigned)((lane / GK::CPR) * GK::NREG * p.k_tok * 2 + (lane % GK::CPR) * 16);
    const unsigned lane_v = (unsigned)((lane / GK::CPR) * GK::NREG * p.v_tok * 2 + (lane % GK::CPR) * 16);
    auto request = [&](const Cursor& c, const int j) {   // tile j of the list into slot j % NSLOT
        const int kt = __builtin_amdgcn_readfirstlane(p.kv_idx[c.e0 + c.e]);
        issue_tile_wave<D, false>(p, lds_addr(ring + (j % nslot) * G::BUFB), kt, c.kvh, j / nslot + 1, lane, lane_k, lane_v);
    };
    auto load_q = [&](const int tz, bf16x8 (&qf)[NS]) {
        const int tok = (tz & 0xfffff) * SPINF_QTILE + 32 * wr + (lane & 31);
        const int tok_c = tok < p.n ? tok : p.n - 1;
        const int h = (int)((unsigned)tz >> 20) * HPI + wh;
        const __bf16* qp = p.q + (long)tok_c * p.q_tok + (long)h * p.q_head + 8 * (lane >> 5);
#pragma unroll
        for (int s2 = 0; s2 < NS; s2++) qf[s2] = *(const bf16x8*)(qp + 16 * s2);
    };

    Cursor ahead{lo, 0, 0, 0, 0, 0}, here{lo, 0, 0, 0, 0, 0};
    open(ahead);
    open(here);
    if (parts == 5) {   // the tiles alone, every tile's requests dealt out over the eight waves (as the lockstep kernel does over its four)
        auto share = [&](const Cursor& c, const int j) {
            const int kt = __builtin_amdgcn_readfirstlane(p.kv_idx[c.e0 + c.e]);
            issue_tile<D, 8, false, 0, 32, D>(p, lds_addr(ring + (j % nslot) * G::BUFB), kt, -1, c.kvh, w, lane, lane_k, lane_v);
        };
        for (int j = 0; j < nslot && ahead.item < hi; j++) {
            share(ahead, j);
            step(ahead);
        }
        const int mine = 4 + (w < 3);   // requests of this wave per tile
        int seen = 0;
#pragma unroll 1
        for (int j = 0; j < total; j++) {
            const int left = total - 1 - j < nslot - 1 ? total - 1 - j : nslot - 1;   // younger tiles on their way
            switch (left * mine) {
                case 0: __builtin_amdgcn_s_waitcnt(0x0f70); break;
                case 4: __builtin_amdgcn_s_waitcnt(0x0f74); break;
                case 5: __builtin_amdgcn_s_waitcnt(0x0f75); break;
                case 8: __builtin_amdgcn_s_waitcnt(0x0f78); break;
                case 10: __builtin_amdgcn_s_waitcnt(0x0f7a); break;
                case 12: __builtin_amdgcn_s_waitcnt(0x0f7c); break;
                default: __builtin_amdgcn_s_waitcnt(0x0f7f); break;   // 15
            }
            __syncthreads();   // tile j has landed, whoever requested which part of it; its slot can take tile j + nslot
            seen++;
            if (ahead.item < hi) {
                share(ahead, j + nslot);
                step(ahead);
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0f70);
        if (threadIdx.x == 0) atomicAdd(&status[1], seen);
        return;
    }
    const bool tiles = parts & 1, rows = parts & 2, dealt = parts == 7;
    // parts 7: the whole pattern with every tile's requests dealt out over the eight waves; wave w's last request of a tile writes
    // word w of the slot's flag area (one lane of a 4-byte request), and a tile has landed when all eight words show its generation
    auto share = [&](const Cursor& c, const int j) {
        const int kt = __builtin_amdgcn_readfirstlane(p.kv_idx[c.e0 + c.e]);
        const unsigned buf = lds_addr(ring + (j % nslot) * G::BUFB);
        issue_tile<D, 8, false, 0, 32, D>(p, buf, kt, -1, c.kvh, w, lane, lane_k, lane_v);
        if (lane == w) dma4_lane(ring_seq + ((j / nslot + 1) & 63), buf + G::KTILEB + G::VTILEB + 768);
    };
    if (dealt) {
        for (int j = 0; j < nslot && ahead.item < hi; j++) {
            share(ahead, j);
            step(ahead);
        }
    } else if (tiles && w < nslot) {   // wave w requests the tiles j = w, w + nslot, ...: the first one now
        for (int i = 0; i < w && ahead.item < hi; i++) step(ahead);
        if (ahead.item < hi) request(ahead, w);
    }
    bf16x8 qf[NS];
    if (rows && here.item < hi) load_q(here.tz, qf);
    int seen = 0;
#pragma unroll 1
    for (int j = 0; j < total; j++) {
        const int want = (j / nslot + 1) & 63;
        int polls = 0;
        if (dealt) {
            const volatile int* f = flag_word(j % nslot);
            while (true) {
                bool all = true;
                for (int i = 0; i < 8; i++) all = all && f[i] == want;
                if (all || *(volatile int*)&sy_abort != 0) break;
                if (++polls > (1 << 20)) {
                    sy_abort = 1;
                    if (lane == 0) atomicAdd(&status[0], 1);
                }
                __builtin_amdgcn_s_sleep(1);
            }
        } else {
            while (tiles && *(volatile int*)flag_word(j % nslot) != want && *(volatile int*)&sy_abort == 0) {
                if (++polls > (1 << 20)) {
                    sy_abort = 1;
                    if (lane == 0) atomicAdd(&status[0], 1);
                }
                __builtin_amdgcn_s_sleep(1);
            }
        }
        if (tiles) __syncthreads();   // every wave has seen tile j: its slot can take tile j + nslot
        if (*(volatile int*)&sy_abort != 0) break;
        seen++;
        if (dealt) {
            if (ahead.item < hi) {
                share(ahead, j + nslot);
                step(ahead);
            }
        } else if (tiles && w == j % nslot) {
            for (int i = 0; i < nslot && ahead.item < hi; i++) step(ahead);
            if (ahead.item < hi) request(ahead, j + nslot);
        }
        if (here.e == here.ne - 1 && !rows) {
            step(here);
        } else if (here.e == here.ne - 1) {   // the item's last tile: the next queries are requested, then this item's rows leave
            const int tz = here.tz;
            step(here);
            bf16x8 qn[NS];
            if (here.item < hi) load_q(here.tz, qn);
#pragma unroll
            for (int s2 = 0; s2 < NS; s2++) asm volatile("" ::"v"(qf[s2]));   // the queries did arrive in registers
            const int tok0 = (tz & 0xfffff) * SPINF_QTILE + 32 * wr;
            const int h = (int)((unsigned)tz >> 20) * HPI + wh;
            __bf16* ob = p.o + (long)h * p.o_head;
            bf16x8 one;
#pragma unroll
            for (int i = 0; i < 8; i++) one[i] = (__bf16)1.0f;
#pragma unroll
            for (int dt = 0; dt < NDT; dt++)
#pragma unroll
                for (int jj = 0; jj < 2; jj++) {
                    const int c = jj * 64 + lane, row = c >> 2, col = c & 3;
                    if (tok0 + row < p.n) *(bf16x8*)(ob + (long)(tok0 + row) * p.o_tok + 32 * dt + col * 8) = one;
                }
            if (here.item < hi) {
#pragma unroll
                for (int s2 = 0; s2 < NS; s2++) qf[s2] = qn[s2];
            }
        } else {
            step(here);
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);   // no DMA of this workgroup is still on its way into LDS when it ends
    if (threadIdx.x == 0) atomicAdd(&status[1], seen);
}

}  // namespace

extern "C" int spinf_diag_attn_stream(const spinf_attn_args* a, int32_t parts, int32_t nslot, int32_t* status, void* stream) {
    if (!a || !status) return spinf_fail(SPINF_E_ARG, "diag_attn_stream: null pointer");
    if ((parts < 1 || parts > 3) && parts != 5 && parts != 7)
        return spinf_fail(SPINF_E_ARG, "diag_attn_stream: parts %d not in 1 (tiles), 2 (queries and outputs), 3 (both), 5 / 7 (as 1 / 3 with a tile's requests dealt over the waves)", parts);
    if (parts >= 5 && !a->pos) return spinf_fail(SPINF_E_ARG, "diag_attn_stream: null pointer");
    if (nslot < 1 || nslot > 4) return spinf_fail(SPINF_E_ARG, "diag_attn_stream: %d slots, 1 .. 4", nslot);
    if (!a->q || !a->k || !a->v || !a->out || !a->art || !a->end || !a->kv_idx || !a->items || !a->list_ptr)
        return spinf_fail(SPINF_E_ARG, "diag_attn_stream: null pointer");
    if (a->d != 256 || a->ktile != 32 || a->n_lists <= 0 || a->n_lists > LAND_CAP || a->hkv <= 0 || a->hq % (2 * a->hkv) || a->row_of || a->grp || a->n <= 0)
        return spinf_fail(SPINF_E_ARG, "diag_attn_stream: takes what the kernel with decoupled waves takes at head dim 256: a static schedule over 32-key "
                                       "entries, an even number of query heads per key / value head, stream layout");
    const int64_t strides[8] = {a->q_tok, a->q_head, a->k_tok, a->k_head, a->v_tok, a->v_head, a->o_tok, a->o_head};
    for (int i = 0; i < 8; i++)
        if (strides[i] % 8) return spinf_fail(SPINF_E_ARG, "diag_attn_stream: strides must be multiples of 8 elements");
    const uintptr_t ptrs[4] = {(uintptr_t)a->q, (uintptr_t)a->k, (uintptr_t)a->v, (uintptr_t)a->out};
    for (int i = 0; i < 4; i++)
        if (ptrs[i] % 16) return spinf_fail(SPINF_E_ARG, "diag_attn_stream: tensors must be 16-byte aligned");
    AttnParams p = {};
    p.q = (const __bf16*)a->q; p.k = (const __bf16*)a->k; p.v = (const __bf16*)a->v; p.o = (__bf16*)a->out;
    p.q_tok = a->q_tok; p.q_head = a->q_head; p.k_tok = a->k_tok; p.k_head = a->k_head;
    p.v_tok = a->v_tok; p.v_head = a->v_head; p.o_tok = a->o_tok; p.o_head = a->o_head;
    p.n = (int)a->n; p.group = a->hq / a->hkv;
    p.art = a->art; p.end = a->end; p.pos = a->pos;
    p.kv_idx = a->kv_idx; p.kv_bits = a->kv_bits;
    p.items = (const int4*)a->items; p.list_ptr = a->list_ptr;
    hipLaunchKernelGGL(attn_stream_kernel<256>, dim3(a->n_lists), dim3(512), 0, (hipStream_t)stream, p, (int*)status, (int)parts, (int)nslot);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "diag_attn_stream: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}

extern "C" int spinf_diag_mfma_hazard(int32_t iters, int32_t workgroups, int32_t* out, void* stream) {
    if (iters <= 0 || iters > 100000 || workgroups <= 0 || workgroups > 65536 || !out)
        return spinf_fail(SPINF_E_ARG, "diag_mfma_hazard: iters in 1 .. 100,000, workgroups in 1 .. 65,536, out not null");
    hipLaunchKernelGGL(mfma_hazard_kernel, dim3(workgroups), dim3(512), 0, (hipStream_t)stream, (int)iters, (int*)out);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "diag_mfma_hazard: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}

template <int KIND>
static void launch_mfma_valu(int nv, int wgs, int threads, int iters, long long* out, hipStream_t stream) {
    switch (nv) {
        case 0: hipLaunchKernelGGL((mfma_valu_kernel<0, KIND>), dim3(wgs), dim3(threads), 0, stream, iters, out); break;
        case 2: hipLaunchKernelGGL((mfma_valu_kernel<2, KIND>), dim3(wgs), dim3(threads), 0, stream, iters, out); break;
        case 4: hipLaunchKernelGGL((mfma_valu_kernel<4, KIND>), dim3(wgs), dim3(threads), 0, stream, iters, out); break;
        case 6: hipLaunchKernelGGL((mfma_valu_kernel<6, KIND>), dim3(wgs), dim3(threads), 0, stream, iters, out); break;
        case 8: hipLaunchKernelGGL((mfma_valu_kernel<8, KIND>), dim3(wgs), dim3(threads), 0, stream, iters, out); break;
        case 12: hipLaunchKernelGGL((mfma_valu_kernel<12, KIND>), dim3(wgs), dim3(threads), 0, stream, iters, out); break;
        default: hipLaunchKernelGGL((mfma_valu_kernel<16, KIND>), dim3(wgs), dim3(threads), 0, stream, iters, out); break;
    }
}

extern "C" int spinf_diag_mfma_valu(int32_t nv, int32_t kind, int32_t waves_per_simd, int32_t iters, int64_t* out, void* stream) {
    if ((nv != 0 && nv != 2 && nv != 4 && nv != 6 && nv != 8 && nv != 12 && nv != 16) || kind < 0 || kind > 2)
        return spinf_fail(SPINF_E_ARG, "diag_mfma_valu: nv %d not in {0, 2, 4, 6, 8, 12, 16} or kind %d not in {0, 1, 2}", nv, kind);
    if ((waves_per_simd != 1 && waves_per_simd != 2 && waves_per_simd != 4) || iters <= 0 || iters > (1 << 22) || !out)
        return spinf_fail(SPINF_E_ARG, "diag_mfma_valu: waves per SIMD in {1, 2, 4}, iters in 1 .. 2^22, out not null");
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return spinf_fail(SPINF_E_HIP, "diag_mfma_valu: no device");
    const int threads = 256 * waves_per_simd;
    if (kind == 0) launch_mfma_valu<0>(nv, prop.multiProcessorCount, threads, iters, (long long*)out, (hipStream_t)stream);
    else if (kind == 2) launch_mfma_valu<2>(nv, prop.multiProcessorCount, threads, iters, (long long*)out, (hipStream_t)stream);
    else launch_mfma_valu<1>(nv, prop.multiProcessorCount, threads, iters, (long long*)out, (hipStream_t)stream);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "diag_mfma_valu: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}

extern "C" int spinf_diag_lds_order(int32_t iters, int32_t workgroups, int32_t* out, void* stream) {
    if (iters <= 0 || iters > 100000 || workgroups <= 0 || workgroups > 65536 || !out)
        return spinf_fail(SPINF_E_ARG, "diag_lds_order: iters in 1 .. 100,000, workgroups in 1 .. 65,536, out not null");
    hipLaunchKernelGGL(lds_order_kernel, dim3(workgroups), dim3(256), 0, (hipStream_t)stream, (int)iters, (int*)out);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "diag_lds_order: launch: %s", hipGetErrorString(e));
    return SPINF_OK;
}

extern "C" int spinf_diag_mfma_rate(int64_t iters, float* out, int64_t out_floats, double* flops, void* stream) {
    if (iters <= 0 || iters > (1 << 24) || !out || !flops) return spinf_fail(SPINF_E_ARG, "diag_mfma_rate: iters in 1 .. 2^24, out and flops not null");
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return spinf_fail(SPINF_E_HIP, "diag_mfma_rate: no device");
    const int wgs = prop.multiProcessorCount;
    if (out_floats < (int64_t)wgs * 512) return spinf_fail(SPINF_E_ARG, "diag_mfma_rate: out holds %lld floats, %lld needed", (long long)out_floats, (long long)wgs * 512);
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(wgs), dim3(512), 0, (hipStream_t)stream, (long)iters, out);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return spinf_fail(SPINF_E_HIP, "diag_mfma_rate: launch: %s", hipGetErrorString(e));
    *flops = (double)wgs * 8 * (double)iters * MFMA_PER_ITER * 2.0 * 32 * 32 * 16;
    return SPINF_OK;
}
