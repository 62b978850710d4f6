// Yardstick kernels of the library's benchmark, for gfx950 (MI355X): what the matrix cores sustain on this part when nothing else
// is in the way.  No counterpart in the reference.
#include <hip/hip_runtime.h>

#include "spinf_tree.h"
#include "common.h"

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

}  // namespace

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
