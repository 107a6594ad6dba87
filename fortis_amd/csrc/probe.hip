// Issue-slot probe: does a SIMD run fp32 matrix instructions and vector instructions of different waves at the
// same time?  512-thread workgroups, two per CU: waves 0-3 of a workgroup (one per SIMD) issue independent
// chains of v_mfma_f32_16x16x4f32 (or 32x32x2), waves 4-7 (the same four SIMDs) independent chains of v_fma_f32
// (or integer add / xor).  Each side is sized to 128 issue cycles per iteration.  Measured on gfx950: both
// together take the SUM of the two alone, for floating-point and integer vector work alike -- the fp32 matrix
// peak equals the fp32 vector peak, and a vector instruction of any wave costs the SIMD its matrix cycles.  The
// roofline fractions of the fused kernels are read against that: their vector work is paid for in matrix time.
#include "common.h"

typedef float pv4f __attribute__((ext_vector_type(4)));
typedef float pv16f __attribute__((ext_vector_type(16)));

// mode bit 0: the matrix waves run; bit 1: the vector waves run.  big: 32x32x2 instead of 16x16x4.  ints: integer vector work.
__global__ __launch_bounds__(512) void issue_probe_kernel(float* out, int iters, int mode, int big, int ints)
{
    const int wave = threadIdx.x >> 6;
    const float x = threadIdx.x * 1e-3f;
    float res = 0.f;
    if (wave < 4) {
        if (!(mode & 1)) return;
        if (!big) {
            pv4f a0 = { 0, 0, 0, 0 }, a1 = a0, a2 = a0, a3 = a0;
            for (int i = 0; i < iters; i++) {
                a0 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, x, a0, 0, 0, 0);
                a1 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, x, a1, 0, 0, 0);
                a2 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, x, a2, 0, 0, 0);
                a3 = __builtin_amdgcn_mfma_f32_16x16x4f32(x, x, a3, 0, 0, 0);
            }
            res = a0[0] + a1[1] + a2[2] + a3[3];
        } else {
            pv16f a0, a1;
            for (int r = 0; r < 16; r++) { a0[r] = 0.f; a1[r] = 0.f; }
            for (int i = 0; i < iters; i++) {
                a0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x, x, a0, 0, 0, 0);
                a1 = __builtin_amdgcn_mfma_f32_32x32x2f32(x, x, a1, 0, 0, 0);
            }
            res = a0[0] + a1[1];
        }
    } else {
        if (!(mode & 2)) return;
        if (!ints) {
            float v[8];
            for (int u = 0; u < 8; u++) v[u] = x + u;
            for (int i = 0; i < iters; i++)
#pragma unroll
                for (int u = 0; u < 32; u++) v[u & 7] = __builtin_fmaf(v[u & 7], 1.0001f, 0.5f);
            for (int u = 0; u < 8; u++) res += v[u];
        } else {
            unsigned v[8];
            for (int u = 0; u < 8; u++) v[u] = threadIdx.x + u;
            for (int i = 0; i < iters; i++)
#pragma unroll
                for (int u = 0; u < 32; u++) {
                    if (u & 1) asm volatile("v_xor_b32 %0, %0, %1" : "+v"(v[u & 7]) : "v"(v[(u + 1) & 7]));
                    else asm volatile("v_add_u32 %0, %0, %1" : "+v"(v[u & 7]) : "v"(v[(u + 1) & 7]));
                }
            for (int u = 0; u < 8; u++) res += (float)v[u];
        }
    }
    out[blockIdx.x * 512 + threadIdx.x] = res;
}

// Milliseconds per launch (mean of 5 after one warm-up) of the probe on the library's stream; out[0..2] = matrix
// waves alone, vector waves alone, both.  Returns -1 when the device has no memory for the result buffer.
extern "C" int fortis_probe_issue_ms(int iters, int big, int ints, float* out_ms)
{
    if (iters < 1 || iters > (1 << 20) || !out_ms) return -1;
    hipStream_t s = fortis_stream_get();
    hipDeviceProp_t prop;
    HIP_OK(hipGetDeviceProperties(&prop, 0));
    const int grid = 2 * prop.multiProcessorCount;
    float* d = nullptr;
    if (fortis_dev_malloc((void**)&d, (size_t)grid * 512 * sizeof(float), "issue probe") != 0) return -1;
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
    for (int mode = 1; mode <= 3; mode++) {
        hipLaunchKernelGGL(issue_probe_kernel, dim3(grid), dim3(512), 0, s, d, iters, mode, big, ints);
        HIP_OK(hipEventRecord(e0, s));
        for (int r = 0; r < 5; r++) hipLaunchKernelGGL(issue_probe_kernel, dim3(grid), dim3(512), 0, s, d, iters, mode, big, ints);
        HIP_OK(hipEventRecord(e1, s));
        HIP_OK(hipEventSynchronize(e1));
        float ms = 0.f;
        HIP_OK(hipEventElapsedTime(&ms, e0, e1));
        out_ms[mode - 1] = ms / 5;
    }
    HIP_OK(hipGetLastError());
    HIP_OK(hipEventDestroy(e0)); HIP_OK(hipEventDestroy(e1));
    fortis_dev_free(d);
    return 0;
}
