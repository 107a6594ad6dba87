// Convolution family of the step, library-free: direct conv2d / conv3d (cross-correlation,
// NCHW / NCDHW, N = 1), transposed conv2d, max pooling, nearest upsample and concat-by-copy, with
// bias / folded BatchNorm / activation / residual add applied in the conv epilogue.
//
// Replaces fortis_conv2d / fortis_conv3d (cuDNN, runtime/fortis_rt.c:108-156), the direct kernels
// k_conv3d_direct / k_conv3d_direct3 (runtime/fortis_fft.cu:91-201) and the separate epilogue
// kernel fortis-fuse emits behind each of them (compiler/FortisFuse.cpp:688-692, 721-760).
//
// Direct kernel mapping: one thread per output position, CONV_FB output channels per thread in
// registers.  Consecutive lanes are consecutive x, so input reads are coalesced; the weight index
// is wave-uniform, so weights arrive through the scalar path and are broadcast.
#include "common.h"

#define CONV_THREADS 256
#define CONV_FB 8

__device__ __forceinline__ float conv_epilogue(float acc, long f, long opos, long ospatial, const ConvEpi& e)
{
    float v = acc;
    if (e.scale) v = v * e.scale[f];
    if (e.shift) v = v + e.shift[f];
    if (e.act == FORTIS_ACT_RELU) v = v > 0.f ? v : 0.f;
    else if (e.act == FORTIS_ACT_LEAKY) v = v > 0.f ? v : e.alpha * v;
    if (e.res) v = v + e.res[f * ospatial + opos];
    return v;
}

struct ConvShape {
    int C, D, H, W, F, KD, KH, KW, Do, Ho, Wo, sd, sh, sw, pd, ph, pw;
};

__global__ __launch_bounds__(CONV_THREADS) void conv_direct_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                   float* __restrict__ y, ConvShape s, ConvEpi e)
{
    const long ospatial = (long)s.Do * s.Ho * s.Wo;
    const long opos = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int f0 = blockIdx.y * CONV_FB;
    if (opos >= ospatial) return;
    const int ox = (int)(opos % s.Wo), oy = (int)((opos / s.Wo) % s.Ho), oz = (int)(opos / ((long)s.Wo * s.Ho));
    const int kvol = s.KD * s.KH * s.KW;
    float acc[CONV_FB];
#pragma unroll
    for (int f = 0; f < CONV_FB; f++) acc[f] = 0.f;
    for (int c = 0; c < s.C; c++) {
        const float* xc = x + (long)c * s.D * s.H * s.W;
        const float* wc = w + ((long)f0 * s.C + c) * kvol;
        for (int kd = 0; kd < s.KD; kd++) {
            const int iz = oz * s.sd + kd - s.pd;
            if (iz < 0 || iz >= s.D) continue;
            for (int kh = 0; kh < s.KH; kh++) {
                const int iy = oy * s.sh + kh - s.ph;
                if (iy < 0 || iy >= s.H) continue;
                for (int kw = 0; kw < s.KW; kw++) {
                    const int ix = ox * s.sw + kw - s.pw;
                    if (ix < 0 || ix >= s.W) continue;
                    const float xv = xc[((long)iz * s.H + iy) * s.W + ix];
                    const int k = (kd * s.KH + kh) * s.KW + kw;
#pragma unroll
                    for (int f = 0; f < CONV_FB; f++)
                        if (f0 + f < s.F) acc[f] = fmaf(xv, wc[(long)f * s.C * kvol + k], acc[f]);
                }
            }
        }
    }
#pragma unroll
    for (int f = 0; f < CONV_FB; f++)
        if (f0 + f < s.F) y[(long)(f0 + f) * ospatial + opos] = conv_epilogue(acc[f], f0 + f, opos, ospatial, e);
}

// Transposed conv2d in gather form: y[f][oy][ox] = sum_c sum_{kh,kw : (oy+p-kh) % s == 0, ...}
//     x[c][(oy+p-kh)/s][(ox+p-kw)/s] * w[c][f][kh][kw]
__global__ __launch_bounds__(CONV_THREADS) void convt2d_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                               float* __restrict__ y, int C, int H, int W, int F, int KH,
                                                               int KW, int Ho, int Wo, int st, int pad, ConvEpi e)
{
    const long ospatial = (long)Ho * Wo;
    const long opos = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int f0 = blockIdx.y * CONV_FB;
    if (opos >= ospatial) return;
    const int ox = (int)(opos % Wo), oy = (int)(opos / Wo);
    float acc[CONV_FB];
#pragma unroll
    for (int f = 0; f < CONV_FB; f++) acc[f] = 0.f;
    for (int c = 0; c < C; c++)
        for (int kh = 0; kh < KH; kh++) {
            const int ty = oy + pad - kh;
            if (ty < 0 || ty % st) continue;
            const int iy = ty / st;
            if (iy >= H) continue;
            for (int kw = 0; kw < KW; kw++) {
                const int tx = ox + pad - kw;
                if (tx < 0 || tx % st) continue;
                const int ix = tx / st;
                if (ix >= W) continue;
                const float xv = x[((long)c * H + iy) * W + ix];
#pragma unroll
                for (int f = 0; f < CONV_FB; f++)
                    if (f0 + f < F) acc[f] = fmaf(xv, w[(((long)c * F + f0 + f) * KH + kh) * KW + kw], acc[f]);
            }
        }
#pragma unroll
    for (int f = 0; f < CONV_FB; f++)
        if (f0 + f < F) y[(long)(f0 + f) * ospatial + opos] = conv_epilogue(acc[f], f0 + f, opos, ospatial, e);
}

__global__ void maxpool2d_kernel(const float* __restrict__ x, float* __restrict__ y, long C, int H, int W, int k)
{
    const int Ho = H / k, Wo = W / k;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= C * Ho * Wo) return;
    const int ox = (int)(idx % Wo), oy = (int)((idx / Wo) % Ho);
    const long c = idx / ((long)Wo * Ho);
    float m = -INFINITY;
    for (int a = 0; a < k; a++)
        for (int b = 0; b < k; b++) {
            const float v = x[(c * H + oy * k + a) * W + ox * k + b];
            m = v > m ? v : m;
        }
    y[idx] = m;
}

__global__ void upsample_kernel(const float* __restrict__ x, float* __restrict__ y, long C, int D, int H, int W, int s, int sd)
{
    const int Do = D * sd, Ho = H * s, Wo = W * s;
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= C * Do * Ho * Wo) return;
    const int xx = (int)(idx % Wo), yy = (int)((idx / Wo) % Ho), zz = (int)((idx / ((long)Wo * Ho)) % Do);
    const long c = idx / ((long)Wo * Ho * Do);
    y[idx] = x[((c * D + zz / sd) * H + yy / s) * W + xx / s];
}

__global__ void copy_kernel(const float* __restrict__ x, float* __restrict__ y, long n)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx < n) y[idx] = x[idx];
}

static bool fits_int(long v) { return v > 0 && v < 2147483647L; }

int fortis_launch_conv3d(const float* x, const float* w, float* y, long C, long D, long H, long Wd, long F, long KD,
                         long KH, long KW, long Do, long Ho, long Wo, long pd, long ph, long pw, const ConvEpi& e,
                         hipStream_t s)
{
    if (!fits_int(C * D * H * Wd) || !fits_int(F * Do * Ho * Wo) || KD <= 0 || KH <= 0 || KW <= 0) return -1;
    if (Do != D + 2 * pd - KD + 1 || Ho != H + 2 * ph - KH + 1 || Wo != Wd + 2 * pw - KW + 1) return -1;
    ConvShape sh = { (int)C, (int)D, (int)H, (int)Wd, (int)F, (int)KD, (int)KH, (int)KW, (int)Do, (int)Ho, (int)Wo, 1, 1, 1,
                     (int)pd, (int)ph, (int)pw };
    hipLaunchKernelGGL(conv_direct_kernel, dim3((unsigned)cdiv(Do * Ho * Wo, CONV_THREADS), (unsigned)cdiv(F, CONV_FB)),
                       dim3(CONV_THREADS), 0, s, x, w, y, sh, e);
    HIP_OK(hipGetLastError());
    return 0;
}

int fortis_launch_conv2d(const float* x, const float* w, float* y, long C, long H, long Wd, long F, long KH, long KW,
                         long Ho, long Wo, long sh_, long sw_, long ph, long pw, const ConvEpi& e, long coff, long ctot,
                         hipStream_t s)
{
    if (!fits_int(C * H * Wd) || !fits_int(ctot * Ho * Wo) || KH <= 0 || KW <= 0 || sh_ <= 0 || sw_ <= 0) return -1;
    if (Ho != (H + 2 * ph - KH) / sh_ + 1 || Wo != (Wd + 2 * pw - KW) / sw_ + 1 || coff < 0 || coff + F > ctot) return -1;
    ConvShape sh = { (int)C, 1, (int)H, (int)Wd, (int)F, 1, (int)KH, (int)KW, 1, (int)Ho, (int)Wo, 1, (int)sh_, (int)sw_,
                     0, (int)ph, (int)pw };
    hipLaunchKernelGGL(conv_direct_kernel, dim3((unsigned)cdiv(Ho * Wo, CONV_THREADS), (unsigned)cdiv(F, CONV_FB)),
                       dim3(CONV_THREADS), 0, s, x, w, y + coff * Ho * Wo, sh, e);
    HIP_OK(hipGetLastError());
    return 0;
}

int fortis_launch_convt2d(const float* x, const float* w, float* y, long C, long H, long Wd, long F, long KH, long KW,
                          long Ho, long Wo, long stride, long pad, const ConvEpi& e, long coff, long ctot, hipStream_t s)
{
    if (!fits_int(C * H * Wd) || !fits_int(ctot * Ho * Wo) || KH <= 0 || KW <= 0 || stride <= 0) return -1;
    if (coff < 0 || coff + F > ctot) return -1;
    hipLaunchKernelGGL(convt2d_kernel, dim3((unsigned)cdiv(Ho * Wo, CONV_THREADS), (unsigned)cdiv(F, CONV_FB)),
                       dim3(CONV_THREADS), 0, s, x, w, y + coff * Ho * Wo, (int)C, (int)H, (int)Wd, (int)F, (int)KH, (int)KW,
                       (int)Ho, (int)Wo, (int)stride, (int)pad, e);
    HIP_OK(hipGetLastError());
    return 0;
}

void fortis_launch_maxpool2d(const float* x, float* y, long C, long H, long Wd, long k, hipStream_t s)
{
    const long n = C * (H / k) * (Wd / k);
    hipLaunchKernelGGL(maxpool2d_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, s, x, y, C, (int)H, (int)Wd, (int)k);
    HIP_OK(hipGetLastError());
}
void fortis_launch_upsample(const float* x, float* y, long C, long D, long H, long Wd, long sfac, int nd, hipStream_t s)
{
    const int sd = nd == 3 ? (int)sfac : 1;
    const long n = C * D * sd * H * sfac * Wd * sfac;
    hipLaunchKernelGGL(upsample_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, s, x, y, C, (int)D, (int)H, (int)Wd, (int)sfac, sd);
    HIP_OK(hipGetLastError());
}
void fortis_launch_concat_copy(const float* x, float* y_at_offset, long C, long S, long, hipStream_t s)
{
    const long n = C * S;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)cdiv(n, 256)), dim3(256), 0, s, x, y_at_offset, n);
    HIP_OK(hipGetLastError());
}
