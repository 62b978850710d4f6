// LDS tile geometry, DMA and lane-exchange helpers shared by the attention kernels (tree_attn.hip, xdecode_attn.hip).
#pragma once
#include <hip/hip_runtime.h>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

__device__ __forceinline__ float lane32_max(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float lane32_sum(float x) {
    u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int D, int TK = 64>
struct Geo {
    // LDS image of one K or V tile of TK rows (64; 32 at head dim 512, where two 64-row tile buffers would not fit).  One wave-wide 16-byte DMA instruction fills 1 KiB of contiguous LDS (a
    // "region"); a region holds rows r, r + NREG, r + 2 NREG ... so that consecutive rows lie in consecutive regions, and
    // regions are padded apart: by 16 bytes for K (the b128 fragment reads of 16 consecutive rows then cover all 64
    // banks) and by 64 bytes for V (the transposing reads touch 64 bytes of each of 4 consecutive rows).  Every address
    // is a per-lane base plus a compile-time offset.
    static constexpr int ROWB = D * 2;                 // bytes of one K / V row
    static constexpr int CPR = ROWB / 16;              // 16-byte chunks per row
    static constexpr int RPI = 1024 / ROWB;            // rows per region
    static constexpr int NREG = TK / RPI;              // regions per tile
    static_assert(RPI >= 1 && NREG >= 4 && NREG <= 64, "tile geometry");
    static constexpr int KRS = 1024 + 16, VRS = 1024 + 64;
    static constexpr int KTILEB = NREG * KRS, VTILEB = NREG * VRS;
    static constexpr int METAB = 4 * 64 * 4;
    static constexpr int BUFB = KTILEB + VTILEB + METAB;   // K tile | V tile | art, end, pos, grp of the keys
    __host__ __device__ static constexpr int k_off(int row) { return (row % NREG) * KRS + (row / NREG) * ROWB; }
    __host__ __device__ static constexpr int v_off(int row) { return (row % NREG) * VRS + (row / NREG) * ROWB; }
    static constexpr int KSUB = k_off(32), VSUB = v_off(32);   // byte offsets of rows 32.. relative to rows 0..
};

// One wave-wide DMA instruction: 64 lanes x `16` (or 4) bytes from global memory straight into 1 KiB (256 B) of contiguous
// LDS at byte address `lds`.  Written as inline assembly on purpose: the compiler then does not track these LDS writes, so
// it never makes the fragment reads of the OTHER tile buffer wait for them (it cannot tell the two buffers apart once the
// buffer is chosen at run time); the kernel orders them itself with s_waitcnt vmcnt(0) + a barrier before a buffer is read.
__device__ __forceinline__ const char* uniform_ptr(const char* p) {   // a wave-uniform pointer, pinned to scalar registers
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)v), hi = __builtin_amdgcn_readfirstlane((unsigned)(v >> 32));
    return (const char*)(((unsigned long long)hi << 32) | lo);
}
__device__ __forceinline__ void dma16_uniform(const char* base, unsigned lane_off, unsigned lds) {   // base is wave-uniform
    base = uniform_ptr(base);
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %0" ::"s"(base), "v"(lane_off), "s"(lds) : "memory", "m0");
}
__device__ __forceinline__ void dma16_lane(const char* addr, unsigned lds) {
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(addr), "s"(lds) : "memory", "m0");
}
__device__ __forceinline__ void dma4_lane(const int* addr, unsigned lds) {
    lds = __builtin_amdgcn_readfirstlane(lds);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(addr), "s"(lds) : "memory", "m0");
}
__device__ __forceinline__ unsigned lds_addr(const void* p) { return (unsigned)(size_t)(const __attribute__((address_space(3))) char*)p; }
