// Memory-bound helpers of the step: per-feature scaling, the masked-ReLU head, the boundary
// pre/post kernels (column-major host array <-> batch-major fp32 activations with the lifted
// normalisation) and layout permutes.  All of them are HBM-bound; the transposing ones go through
// a 32 x 33 LDS tile so that both the read and the write side are coalesced (the reference's
// fortis_pre_k / fortis_post_k, trt_backend/e3sm_boundary.cu:9-20, are one-thread-per-element and
// strided on one side).
#include "common.h"
#include <type_traits>

#define EW_THREADS 256

__global__ void scale_kernel(const float* __restrict__ src, float* __restrict__ dst, const float* __restrict__ vec,
                             long total, long n, int divide)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const float v = src[idx], s = vec[idx % n];
    dst[idx] = divide ? __fdiv_rn(v, s) : __fmul_rn(v, s);
}
void fortis_launch_scale(const float* src, float* dst, const float* vec, long rows, long n, int divide, hipStream_t s)
{
    const long total = rows * n;
    if (total <= 0) return;
    hipLaunchKernelGGL(scale_kernel, dim3((unsigned)cdiv(total, EW_THREADS)), dim3(EW_THREADS), 0, s, src, dst, vec, total, n, divide);
    HIP_OK(hipGetLastError());
}

__global__ void mask_relu_kernel(const float* __restrict__ src, float* __restrict__ dst, long total, long n, long tail)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const float v = src[idx];
    dst[idx] = (idx % n >= n - tail && v < 0.f) ? 0.f : v;
}
// dst[0 .. n) = 0 as a kernel: a memset node recorded into a captured graph is not replayed reliably here.
__global__ void zero_kernel(float* __restrict__ dst, long n)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < n) dst[idx] = 0.f;
}
void fortis_launch_zero(float* dst, long n, hipStream_t s)
{
    if (n <= 0) return;
    hipLaunchKernelGGL(zero_kernel, dim3((unsigned)cdiv(n, EW_THREADS)), dim3(EW_THREADS), 0, s, dst, n);
    HIP_OK(hipGetLastError());
}
void fortis_launch_mask_relu(const float* src, float* dst, long rows, long n, long tail, hipStream_t s)
{
    const long total = rows * n;
    if (total <= 0) return;
    hipLaunchKernelGGL(mask_relu_kernel, dim3((unsigned)cdiv(total, EW_THREADS)), dim3(EW_THREADS), 0, s, src, dst, total, n, tail);
    HIP_OK(hipGetLastError());
}

// dst[c][r] = f(src[r][c], r, c) for a row-major src[R][Cc]; 32 x 32 tiles, block (32, 8).
template <typename TI, typename TO, typename F>
__global__ void transpose_kernel(const TI* __restrict__ src, TO* __restrict__ dst, long R, long Cc, F f)
{
    __shared__ TO tile[32][33];
    const long c0 = (long)blockIdx.x * 32, r0 = (long)blockIdx.y * 32;
    for (int y = threadIdx.y; y < 32; y += 8) {
        const long r = r0 + y, c = c0 + threadIdx.x;
        if (r < R && c < Cc) tile[y][threadIdx.x] = f(src[r * Cc + c], r, c);
    }
    __syncthreads();
    for (int y = threadIdx.y; y < 32; y += 8) {
        const long c = c0 + y, r = r0 + threadIdx.x;
        if (r < R && c < Cc) dst[c * R + r] = tile[threadIdx.x][y];
    }
}
// The same for fp32 on both sides with R and Cc multiples of 4 and 16-byte aligned arrays: 64 x 64 tiles, 256
// threads, 16-byte loads along the source rows and 16-byte stores along the destination rows.
template <typename F>
__global__ __launch_bounds__(256) void transpose4_kernel(const float* __restrict__ src, float* __restrict__ dst, long R, long Cc, F f)
{
    __shared__ float tile[64][65];
    const long c0 = (long)blockIdx.x * 64, r0 = (long)blockIdx.y * 64;
    const int tid = threadIdx.x;
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int idx = tid + u * 256, row = idx >> 4, c4 = (idx & 15) * 4;
        const long r = r0 + row, c = c0 + c4;
        if (r < R && c < Cc) {
            const float4 v = *(const float4*)(src + r * Cc + c);
            tile[row][c4] = f(v.x, r, c); tile[row][c4 + 1] = f(v.y, r, c + 1);
            tile[row][c4 + 2] = f(v.z, r, c + 2); tile[row][c4 + 3] = f(v.w, r, c + 3);
        }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 4; u++) {
        const int idx = tid + u * 256, crow = idx >> 4, r4 = (idx & 15) * 4;
        const long c = c0 + crow, r = r0 + r4;
        if (r < R && c < Cc)
            *(float4*)(dst + c * R + r) = make_float4(tile[r4][crow], tile[r4 + 1][crow], tile[r4 + 2][crow], tile[r4 + 3][crow]);
    }
}

// One side short (channels-last <-> channels-first with a handful of channels): a thread takes all the elements of
// one index of the long side, so its loads (ROWS: one per row, each coalesced over the threads) or its stores are
// the short run, contiguous from thread to thread; a 32 x 32 tile would be mostly empty.
template <typename TI, typename TO, typename F, bool ROWS>
__global__ void transpose_short_kernel(const TI* __restrict__ src, TO* __restrict__ dst, long R, long Cc, F f)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (ROWS) {                       // R <= 8 rows: thread per column c
        if (i >= Cc) return;
        for (long r = 0; r < R; r++) dst[i * R + r] = f(src[r * Cc + i], r, i);
    } else {                          // Cc <= 8 columns: thread per row r
        if (i >= R) return;
        for (long c = 0; c < Cc; c++) dst[c * R + i] = f(src[i * Cc + c], i, c);
    }
}

template <typename TI, typename TO, typename F>
static void launch_transpose(const TI* src, TO* dst, long R, long Cc, F f, hipStream_t s)
{
    if (R <= 0 || Cc <= 0) return;
    if (R <= 8 && Cc >= 256) {
        hipLaunchKernelGGL((transpose_short_kernel<TI, TO, F, true>), dim3((unsigned)cdiv(Cc, 256)), dim3(256), 0, s, src, dst, R, Cc, f);
        HIP_OK(hipGetLastError());
        return;
    }
    if (Cc <= 8 && R >= 256) {
        hipLaunchKernelGGL((transpose_short_kernel<TI, TO, F, false>), dim3((unsigned)cdiv(R, 256)), dim3(256), 0, s, src, dst, R, Cc, f);
        HIP_OK(hipGetLastError());
        return;
    }
    if constexpr (std::is_same<TI, float>::value && std::is_same<TO, float>::value) {
        if (R % 4 == 0 && Cc % 4 == 0 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0) {
            hipLaunchKernelGGL((transpose4_kernel<F>), dim3((unsigned)cdiv(Cc, 64), (unsigned)cdiv(R, 64)), dim3(256), 0, s, src, dst, R, Cc, f);
            HIP_OK(hipGetLastError());
            return;
        }
    }
    hipLaunchKernelGGL((transpose_kernel<TI, TO, F>), dim3((unsigned)cdiv(Cc, 32), (unsigned)cdiv(R, 32)), dim3(32, 8), 0, s,
                       src, dst, R, Cc, f);
    HIP_OK(hipGetLastError());
}

// pre: the host array (NI, NK) column-major is the row-major matrix [NK][NI]; X = its transpose
// with (a - mean[k]) / (max[k] - min[k]) evaluated in the host type, then cast to fp32.
template <typename H>
struct PreF {
    const H* mean; const H* vmax; const H* vmin;
    __device__ float operator()(H a, long k, long) const
    {
        const H m = mean ? mean[k] : (H)0, range = vmax ? (vmax[k] - (vmin ? vmin[k] : (H)0)) : (H)1;
        return (float)((a - m) / range);
    }
};
// post: Y[NI][NK] row-major -> B[NK][NI] (column-major (NI, NK)) with (H)y / scale[k].
template <typename H>
struct PostF {
    const H* scale;
    __device__ H operator()(float y, long, long k) const { return scale ? (H)y / scale[k] : (H)y; }
};
struct IdF { __device__ float operator()(float v, long, long) const { return v; } };

void fortis_launch_boundary_pre(const void* A, float* X, long NI, long NK, const void* mean, const void* vmax,
                                const void* vmin, int host_esz, hipStream_t s)
{
    if (host_esz == 8) {
        PreF<double> f = { (const double*)mean, (const double*)vmax, (const double*)vmin };
        launch_transpose((const double*)A, X, NK, NI, f, s);
    } else {
        PreF<float> f = { (const float*)mean, (const float*)vmax, (const float*)vmin };
        launch_transpose((const float*)A, X, NK, NI, f, s);
    }
}
void fortis_launch_boundary_post(const float* Y, void* B, long NI, long NK, const void* scale, int host_esz, hipStream_t s)
{
    if (host_esz == 8) {
        PostF<double> f = { (const double*)scale };
        launch_transpose(Y, (double*)B, NI, NK, f, s);
    } else {
        PostF<float> f = { (const float*)scale };
        launch_transpose(Y, (float*)B, NI, NK, f, s);
    }
}
void fortis_launch_permute(const float* src, float* dst, long C, long S, int to_channels_first, hipStream_t s)
{
    if (to_channels_first) launch_transpose(src, dst, S, C, IdF(), s);   // [S][C] -> [C][S]
    else launch_transpose(src, dst, C, S, IdF(), s);                      // [C][S] -> [S][C]
}
