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
#define CONV_FB 8      // output channels per thread of the transposed-conv kernel and the wide direct kernel

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

// FB output channels per thread: 8 keeps an input value in a register for eight products; 1 gives a small
// problem (the 3 -> 8 channel probe on 16^3) eight times as many threads to spread over the chip.
#define CONV_WLDS 4096   // weights of a block's output channels staged in LDS when they fit (floats)
// K3: the kernel is 3 x 3 x 3 (or 1 x 3 x 3) with stride 1: the tap loops are unrolled and every load is
// issued unconditionally from a clamped coordinate (its weight is replaced by zero outside the image), so
// a thread's loads overlap instead of each waiting behind a bounds branch.
template <int FB, bool K3>
__global__ __launch_bounds__(CONV_THREADS) void conv_direct_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                   float* __restrict__ y, ConvShape s, ConvEpi e)
{
    __shared__ float sw[CONV_WLDS];
    const long ospatial = (long)s.Do * s.Ho * s.Wo;
    const long opos = (long)blockIdx.x * CONV_THREADS + threadIdx.x;
    const int f0 = blockIdx.y * FB;
    const int kvol = s.KD * s.KH * s.KW, ckv = s.C * kvol;
    // the block's weights [FB][C][taps]: one cooperative copy instead of a scalar load (and its wait) per product
    const bool wl = FB * ckv <= CONV_WLDS;
    if (wl) {
        for (int i = threadIdx.x; i < FB * ckv; i += CONV_THREADS) {
            const int f = i / ckv;
            sw[i] = f0 + f < s.F ? w[(long)f0 * ckv + i] : 0.f;
        }
        __syncthreads();
    }
    if (opos >= ospatial) return;
    const int ox = (int)(opos % s.Wo), oy = (int)((opos / s.Wo) % s.Ho), oz = (int)(opos / ((long)s.Wo * s.Ho));
    const long chan = (long)s.D * s.H * s.W;
    float acc[FB];
#pragma unroll
    for (int f = 0; f < FB; f++) acc[f] = 0.f;
    if (K3 && wl) {
        const int nkd = s.KD;                        // 3, or 1 for a 2-D convolution
        for (int c = 0; c < s.C; c++) {
            const float* xc = x + c * chan;
            for (int kd = 0; kd < nkd; kd++) {
                const int iz = oz + kd - s.pd;
                const bool vz = iz >= 0 && iz < s.D;
                const int cz = vz ? iz : 0;
                float xv[9];
                bool ok[9];
#pragma unroll
                for (int t = 0; t < 9; t++) {
                    const int iy = oy + t / 3 - s.ph, ix = ox + t % 3 - s.pw;
                    ok[t] = vz && iy >= 0 && iy < s.H && ix >= 0 && ix < s.W;
                    const int cy = iy < 0 ? 0 : iy >= s.H ? s.H - 1 : iy, cx = ix < 0 ? 0 : ix >= s.W ? s.W - 1 : ix;
                    xv[t] = xc[((long)cz * s.H + cy) * s.W + cx];
                }
#pragma unroll
                for (int t = 0; t < 9; t++)
#pragma unroll
                    for (int f = 0; f < FB; f++)
                        acc[f] = fmaf(ok[t] ? xv[t] : 0.f, sw[f * ckv + c * kvol + kd * 9 + t], acc[f]);
            }
        }
    } else {
    // taps outermost (bounds are checked once per tap), input channels innermost
    for (int kd = 0; kd < s.KD; kd++) {
        const int iz = oz * s.sd + kd - s.pd;
        if (iz < 0 || iz >= s.D) continue;
        for (int kh = 0; kh < s.KH; kh++) {
            const int iy = oy * s.sh + kh - s.ph;
            if (iy < 0 || iy >= s.H) continue;
            for (int kw = 0; kw < s.KW; kw++) {
                const int ix = ox * s.sw + kw - s.pw;
                if (ix < 0 || ix >= s.W) continue;
                const float* xp = x + ((long)iz * s.H + iy) * s.W + ix;
                const int k = (kd * s.KH + kh) * s.KW + kw;
                for (int c = 0; c < s.C; c++) {
                    const float xv = xp[c * chan];
#pragma unroll
                    for (int f = 0; f < FB; f++) {
                        const float wv = wl ? sw[f * ckv + c * kvol + k] : (f0 + f < s.F ? w[((long)(f0 + f) * s.C + c) * kvol + k] : 0.f);
                        acc[f] = fmaf(xv, wv, acc[f]);
                    }
                }
            }
        }
    }
    }
#pragma unroll
    for (int f = 0; f < FB; f++)
        if (f0 + f < s.F) y[(long)(f0 + f) * ospatial + opos] = conv_epilogue(acc[f], f0 + f, opos, ospatial, e);
}

// 3x3x3, stride 1, pad 1 convolution with at most CT_F output channels (image-space heads such as
// 64 -> 3): the matrix cores would multiply 32-row tiles that are nine tenths padding, so this one runs on
// the vector ALUs, which have the same fp32 peak on this part.
// Positions of one z-plane are linearised with pitch P = W + 1 (tap (kh, kw) of position m is element
// m + kh*P + kw of the zero-padded plane, a lane-independent offset).  A workgroup takes CT_MT positions,
// a thread CT_PT consecutive ones times all output channels in registers; per chunk of CT_CC input
// channels the three z-planes' runs are staged in LDS (double buffered through registers), and the
// chunk's weights [channel][tap][output channel] next to them; a weight read has the same address in
// every lane (LDS broadcast) and fetches one tap for all output channels.
#define CT_F 4
#define CT_PT 2
#define CT_MT (CONV_THREADS * CT_PT)
#define CT_CC 2
#define CT_NX 16     // staged elements per thread per chunk, at most

template <int NF>      // output channels computed: 3 (F <= 3) or 4
__global__ __launch_bounds__(CONV_THREADS) void conv3d_thin_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                   float* __restrict__ y, int C, int D, int H, int W, int F,
                                                                   int P, int plane, int tiles, int R, ConvEpi e)
{
    extern __shared__ float ct_lds[];                       // [2][CT_CC][3][R] inputs, then [2][CT_CC][27][CT_F] weights
    const int tid = threadIdx.x;
    const int z = blockIdx.x / tiles, tile = blockIdx.x - z * tiles;
    const int m0 = tile * CT_MT;
    const long HW = (long)H * W, chan = (long)D * HW;
    const int XCH = CT_CC * 3 * R;

    // staging map (the same for every chunk): offset of the element inside a CT_CC-channel group, or -1
    int goff[CT_NX];
#pragma unroll
    for (int i = 0; i < CT_NX; i++) {
        const int el = tid + i * CONV_THREADS;
        goff[i] = -1;
        if (el < XCH) {
            const int c = el / (3 * R), rem = el - c * (3 * R), kd = rem / R, r = rem - kd * R;
            const int v = m0 + r, yp = v / P, xp = v - yp * P;
            const int zz = z + kd - 1, yy = yp - 1, xx = xp - 1;
            if (zz >= 0 && zz < D && yy >= 0 && yy < H && xx >= 0 && xx < W)
                goff[i] = (int)(c * chan + zz * HW + (long)yy * W + xx);
        }
    }
    float rx[CT_NX];
    float rwt = 0.f;
    float* wl = ct_lds + 2 * XCH;
    // weight element this thread stages: (cc, tap, f) -> w[f][c][tap]
    const int wcc = tid / (27 * CT_F), wtap = (tid / CT_F) % 27, wf = tid % CT_F;
    auto load_chunk = [&](int ch) __attribute__((always_inline)) {
        if (tid < CT_CC * 27 * CT_F) {
            const int c = ch * CT_CC + wcc;
            rwt = (wf < F && c < C) ? w[((long)wf * C + c) * 27 + wtap] : 0.f;
        }
        const float* xsrc = x + (long)ch * CT_CC * chan;
#pragma unroll
        for (int i = 0; i < CT_NX; i++) {
            const int el = tid + i * CONV_THREADS;
            const bool ok = goff[i] >= 0 && ch * CT_CC + el / (3 * R) < C;
            const float v = xsrc[ok ? goff[i] : 0];
            rx[i] = ok ? v : 0.f;
        }
    };
    auto store_chunk = [&](int buf) __attribute__((always_inline)) {
        if (tid < CT_CC * 27 * CT_F) wl[buf * CT_CC * 27 * CT_F + tid] = rwt;
        float* dst = ct_lds + buf * XCH;
#pragma unroll
        for (int i = 0; i < CT_NX; i++) {
            const int el = tid + i * CONV_THREADS;
            if (el < XCH) dst[el] = rx[i];
        }
    };

    float acc[NF][CT_PT];
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int p = 0; p < CT_PT; p++) acc[f][p] = 0.f;

    const int nchunks = (C + CT_CC - 1) / CT_CC;
    load_chunk(0);
    store_chunk(0);
    __syncthreads();
    for (int ch = 0; ch < nchunks; ch++) {
        const int buf = ch & 1;
        if (ch + 1 < nchunks) load_chunk(ch + 1);
        const float* xs = ct_lds + buf * XCH + tid * CT_PT;
#pragma unroll
        for (int cc = 0; cc < CT_CC; cc++) {
            const int c = ch * CT_CC + cc;
            if (c >= C) break;
#pragma unroll
            for (int kd = 0; kd < 3; kd++)
#pragma unroll
                for (int kh = 0; kh < 3; kh++) {
                    float in[CT_PT + 2];
                    const float* row = xs + (cc * 3 + kd) * R + kh * P;
#pragma unroll
                    for (int t = 0; t < CT_PT + 2; t++) in[t] = row[t];
                    // the three taps' weights for all output channels: same address in every lane (LDS broadcast)
                    const float4* wt = (const float4*)(wl + ((buf * CT_CC + cc) * 27 + (kd * 3 + kh) * 3) * CT_F);
                    const float4 w0 = wt[0], w1 = wt[1], w2 = wt[2];
                    const float wa[3][CT_F] = { { w0.x, w0.y, w0.z, w0.w }, { w1.x, w1.y, w1.z, w1.w }, { w2.x, w2.y, w2.z, w2.w } };
#pragma unroll
                    for (int f = 0; f < NF; f++)
#pragma unroll
                        for (int p = 0; p < CT_PT; p++)
                            acc[f][p] = fmaf(in[p + 2], wa[2][f], fmaf(in[p + 1], wa[1][f], fmaf(in[p], wa[0][f], acc[f][p])));
                }
        }
        if (ch + 1 < nchunks) store_chunk(buf ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int p = 0; p < CT_PT; p++) {
        const int m = m0 + tid * CT_PT + p;
        if (m >= plane) continue;
        const int yy = m / P, xx = m - yy * P;
        if (xx >= W) continue;
        const long opos = ((long)z * H + yy) * W + xx;
#pragma unroll
        for (int f = 0; f < NF; f++)
            if (f < F) y[f * chan + opos] = conv_epilogue(acc[f][p], f, opos, chan, e);
    }
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

static void launch_direct(const float* x, const float* w, float* y, const ConvShape& sh, const ConvEpi& e, long ospatial, long F,
                          hipStream_t s)
{
    static int cus = 0;
    if (!cus) {
        hipDeviceProp_t prop;
        cus = hipGetDeviceProperties(&prop, 0) == hipSuccess ? prop.multiProcessorCount : 256;
    }
    const long blocks = cdiv(ospatial, CONV_THREADS);
    const bool k3 = sh.KH == 3 && sh.KW == 3 && (sh.KD == 3 || sh.KD == 1) && sh.sd == 1 && sh.sh == 1 && sh.sw == 1;
    const dim3 g1((unsigned)blocks, (unsigned)F), g8((unsigned)blocks, (unsigned)cdiv(F, 8)), b(CONV_THREADS);
    if (blocks * cdiv(F, 8) < cus) {
        if (k3) hipLaunchKernelGGL((conv_direct_kernel<1, true>), g1, b, 0, s, x, w, y, sh, e);
        else hipLaunchKernelGGL((conv_direct_kernel<1, false>), g1, b, 0, s, x, w, y, sh, e);
    } else {
        if (k3) hipLaunchKernelGGL((conv_direct_kernel<8, true>), g8, b, 0, s, x, w, y, sh, e);
        else hipLaunchKernelGGL((conv_direct_kernel<8, false>), g8, b, 0, s, x, w, y, sh, e);
    }
}

int fortis_launch_conv3d(const float* x, const float* w, float* y, long C, long D, long H, long Wd, long F, long KD,
                         long KH, long KW, long Do, long Ho, long Wo, long pd, long ph, long pw, const ConvEpi& e,
                         hipStream_t s)
{
    if (!fits_int(C * D * H * Wd) || !fits_int(F * Do * Ho * Wo) || KD <= 0 || KH <= 0 || KW <= 0) return -1;
    if (Do != D + 2 * pd - KD + 1 || Ho != H + 2 * ph - KH + 1 || Wo != Wd + 2 * pw - KW + 1) return -1;
    if (KD == 3 && KH == 3 && KW == 3 && pd == 1 && ph == 1 && pw == 1 && F <= CT_F) {
        const int P = (int)Wd + 1, plane = (int)H * P, tiles = (int)cdiv(plane, CT_MT), R = CT_MT + 2 * P + 2;
        const size_t shmem = (size_t)2 * (CT_CC * 3 * R + CT_CC * 27 * CT_F) * sizeof(float);
        if ((long)CT_CC * 3 * R <= (long)CONV_THREADS * CT_NX && shmem <= 160 * 1024) {
            static size_t attr = 0;
            if (shmem > attr) {
                HIP_OK(hipFuncSetAttribute((const void*)conv3d_thin_kernel<3>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
                HIP_OK(hipFuncSetAttribute((const void*)conv3d_thin_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
                attr = shmem;
            }
            if (F <= 3)
                hipLaunchKernelGGL(conv3d_thin_kernel<3>, dim3((unsigned)(D * tiles)), dim3(CONV_THREADS), shmem, s, x, w, y, (int)C,
                                   (int)D, (int)H, (int)Wd, (int)F, P, plane, tiles, R, e);
            else
                hipLaunchKernelGGL(conv3d_thin_kernel<4>, dim3((unsigned)(D * tiles)), dim3(CONV_THREADS), shmem, s, x, w, y, (int)C,
                                   (int)D, (int)H, (int)Wd, (int)F, P, plane, tiles, R, e);
            HIP_OK(hipGetLastError());
            return 0;
        }
    }
    ConvShape sh = { (int)C, (int)D, (int)H, (int)Wd, (int)F, (int)KD, (int)KH, (int)KW, (int)Do, (int)Ho, (int)Wo, 1, 1, 1,
                     (int)pd, (int)ph, (int)pw };
    launch_direct(x, w, y, sh, e, Do * Ho * Wo, F, s);
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
    launch_direct(x, w, y + coff * Ho * Wo, sh, e, Ho * Wo, F, s);
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
