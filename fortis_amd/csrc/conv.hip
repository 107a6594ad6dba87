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
// the vector ALUs.
// Positions of one z-plane are linearised with pitch P = W + 1 (tap (kh, kw) of position m is element
// m + kh*P + kw of the zero-padded plane, a lane-independent offset).  A workgroup takes CT_MT positions,
// a thread CT_PT consecutive ones times all output channels in registers; per chunk of CT_CC input
// channels the three z-planes' runs are staged in LDS (double buffered through registers).  A weight has
// the same address in every lane, so the weights are read through the scalar cache into scalar registers
// (LDS broadcast reads of them took more LDS time than the inputs).  With few workgroups per compute unit
// the input channels are split over blockIdx.y and a reduce kernel adds the slices.
#define CT_F 4
#define CT_PT 2
#define CT_MT (CONV_THREADS * CT_PT)
#define CT_CC 2
#define CT_NR 3      // staging rounds of a (channel, z-plane) run: it has at most CT_NR * CONV_THREADS elements

template <int NF>      // output channels computed: 3 (F <= 3) or 4
__global__ __launch_bounds__(CONV_THREADS) void conv3d_thin_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                   float* __restrict__ y, int C, int D, int H, int W, int F,
                                                                   int P, int plane, int tiles, int R, int cps, ConvEpi e)
{
    // blockIdx.y: slice of the input channels (cps chunks each); with more than one slice, slice k writes
    // its raw sums to y + k * F*D*H*W and a reduce kernel applies the epilogue
    extern __shared__ float ct_lds[];                       // [2][CT_CC][3][R] inputs
    const int tid = threadIdx.x;
    const int bx = (int)fortis_xcd_band(blockIdx.x, gridDim.x);       // neighbouring tiles and planes on one XCD
    const int z = bx / tiles, tile = bx - z * tiles;
    const int m0 = tile * CT_MT;
    const long HW = (long)H * W, chan = (long)D * HW;
    const int XCH = CT_CC * 3 * R;

    // staging map: every (channel, z-plane) run of a chunk holds the same R pixels, so a thread keeps the
    // in-plane offset of pixel tid + j * CONV_THREADS (or -1 outside the image) and the run's base is uniform
    unsigned poff[CT_NR];       // byte offset inside the plane (0 for padding)
    bool pin[CT_NR];            // inside the image
#pragma unroll
    for (int j = 0; j < CT_NR; j++) {
        const int r = tid + j * CONV_THREADS;
        const int v = m0 + r, yp = v / P, xp = v - yp * P;
        const int yy = yp - 1, xx = xp - 1;
        pin[j] = r < R && yy >= 0 && yy < H && xx >= 0 && xx < W;
        poff[j] = pin[j] ? (unsigned)(yy * W + xx) * 4u : 0u;
    }
    float rx[CT_CC * 3][CT_NR];
    // run (cc, kd) of chunk ch lies inside the tensor
    auto run_ok = [&](int ch, int cc, int kd) __attribute__((always_inline)) {
        const int zz = z + kd - 1;
        return ch * CT_CC + cc < C && zz >= 0 && zz < D;
    };
    auto load_chunk = [&](int ch) __attribute__((always_inline)) {
#pragma unroll
        for (int cc = 0; cc < CT_CC; cc++)
#pragma unroll
            for (int kd = 0; kd < 3; kd++) {
                // runs outside the tensor read the tensor's first plane and are zeroed when stored
                const char* src = (const char*)(run_ok(ch, cc, kd) ? x + (long)(ch * CT_CC + cc) * chan + (long)(z + kd - 1) * HW : x);
#pragma unroll
                for (int j = 0; j < CT_NR; j++) rx[cc * 3 + kd][j] = *(const float*)(src + poff[j]);
            }
    };
    auto store_chunk = [&](int buf, int ch) __attribute__((always_inline)) {
        float* dst = ct_lds + buf * XCH;
#pragma unroll
        for (int cc = 0; cc < CT_CC; cc++)
#pragma unroll
            for (int kd = 0; kd < 3; kd++) {
                const bool ok = run_ok(ch, cc, kd);
#pragma unroll
                for (int j = 0; j < CT_NR; j++) {
                    const int r = tid + j * CONV_THREADS;
                    if (r < R) dst[(cc * 3 + kd) * R + r] = (ok && pin[j]) ? rx[cc * 3 + kd][j] : 0.f;
                }
            }
    };

    float acc[NF][CT_PT];
#pragma unroll
    for (int f = 0; f < NF; f++)
#pragma unroll
        for (int p = 0; p < CT_PT; p++) acc[f][p] = 0.f;

    const int nall = (C + CT_CC - 1) / CT_CC;
    const int ch0 = blockIdx.y * cps, nchunks = ch0 + cps < nall ? ch0 + cps : nall;
    load_chunk(ch0);
    store_chunk(0, ch0);
    __syncthreads();
    for (int ch = ch0; ch < nchunks; ch++) {
        const int buf = (ch - ch0) & 1;
        if (ch + 1 < nchunks) load_chunk(ch + 1);
        const float* xs = ct_lds + buf * XCH + tid * CT_PT;
#pragma unroll
        for (int cc = 0; cc < CT_CC; cc++) {
            const int c = ch * CT_CC + cc;
            if (c >= C) break;
#pragma unroll
            for (int kd = 0; kd < 3; kd++) {
                // the plane's nine weights of every output channel: the address is the same in all lanes, so they
                // come through the scalar cache into scalar registers and cost no LDS or vector traffic
                // (channels beyond F repeat the last one; their sums are not stored)
                float wk[NF][9];
#pragma unroll
                for (int f = 0; f < NF; f++) {
                    const float* wr = w + ((long)(f < F ? f : F - 1) * C + c) * 27 + kd * 9;
#pragma unroll
                    for (int t = 0; t < 9; t++) wk[f][t] = wr[t];
                }
#pragma unroll
                for (int kh = 0; kh < 3; kh++) {
                    float in[CT_PT + 2];
                    const float* row = xs + (cc * 3 + kd) * R + kh * P;
#pragma unroll
                    for (int t = 0; t < CT_PT + 2; t++) in[t] = row[t];
#pragma unroll
                    for (int f = 0; f < NF; f++)
#pragma unroll
                        for (int p = 0; p < CT_PT; p++)
                            acc[f][p] = fmaf(in[p + 2], wk[f][kh * 3 + 2],
                                             fmaf(in[p + 1], wk[f][kh * 3 + 1], fmaf(in[p], wk[f][kh * 3], acc[f][p])));
                }
            }
        }
        if (ch + 1 < nchunks) store_chunk(buf ^ 1, ch + 1);
        __syncthreads();
    }
#pragma unroll
    for (int p = 0; p < CT_PT; p++) {
        const int m = m0 + tid * CT_PT + p;
        if (m >= plane) continue;
        const int yy = m / P, xx = m - yy * P;
        if (xx >= W) continue;
        const long opos = ((long)z * H + yy) * W + xx;
        if (gridDim.y > 1) {
            float* part = y + (long)blockIdx.y * F * chan;
#pragma unroll
            for (int f = 0; f < NF; f++)
                if (f < F) part[f * chan + opos] = acc[f][p];
        } else {
#pragma unroll
            for (int f = 0; f < NF; f++)
                if (f < F) y[f * chan + opos] = conv_epilogue(acc[f][p], f, opos, chan, e);
        }
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

static int thin_cus()
{
    static int cus = 0;
    if (!cus) {
        hipDeviceProp_t prop;
        cus = hipGetDeviceProperties(&prop, 0) == hipSuccess ? prop.multiProcessorCount : 256;
    }
    return cus;
}

int fortis_launch_conv3d(const float* x, const float* w, float* y, long C, long D, long H, long Wd, long F, long KD,
                         long KH, long KW, long Do, long Ho, long Wo, long pd, long ph, long pw, const ConvEpi& e,
                         hipStream_t s, long sd, long sh_, long sw_)
{
    if (!fits_int(C * D * H * Wd) || !fits_int(F * Do * Ho * Wo) || KD <= 0 || KH <= 0 || KW <= 0 || sd <= 0 || sh_ <= 0 || sw_ <= 0) return -1;
    if (Do != (D + 2 * pd - KD) / sd + 1 || Ho != (H + 2 * ph - KH) / sh_ + 1 || Wo != (Wd + 2 * pw - KW) / sw_ + 1) return -1;
    const bool unit = sd == 1 && sh_ == 1 && sw_ == 1;
    if (unit && KD == 3 && KH == 3 && KW == 3 && pd == 1 && ph == 1 && pw == 1 && F <= CT_F) {
        const int P = (int)Wd + 1, plane = (int)H * P, tiles = (int)cdiv(plane, CT_MT), R = CT_MT + 2 * P + 2;
        const size_t shmem = (size_t)2 * CT_CC * 3 * R * sizeof(float);
        if (R <= CONV_THREADS * CT_NR && shmem <= 160 * 1024) {
            static size_t attr = 0;
            if (shmem > attr) {
                HIP_OK(hipFuncSetAttribute((const void*)conv3d_thin_kernel<3>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
                HIP_OK(hipFuncSetAttribute((const void*)conv3d_thin_kernel<4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
                attr = shmem;
            }
            // a workgroup's chunks run one after another, each waiting for its loads: with few workgroups
            // per compute unit the input channels are split so that about eight are in flight on each
            const int nall = (int)cdiv(C, CT_CC);
            int ksplit = 1;
            while (ksplit < 8 && D * tiles * ksplit < 8L * thin_cus() && nall / (ksplit * 2) >= 4) ksplit *= 2;
            const int cps = (int)cdiv(nall, ksplit);
            ksplit = (int)cdiv(nall, cps);
            const long osize = F * D * H * Wd;
            float* dst = y;
            if (ksplit > 1) {
                dst = fortis_conv_split_scratch((size_t)ksplit * osize * sizeof(float));
                if (!dst) return -1;
            }
            const dim3 grid((unsigned)(D * tiles), (unsigned)ksplit);
            if (F <= 3)
                hipLaunchKernelGGL(conv3d_thin_kernel<3>, grid, dim3(CONV_THREADS), shmem, s, x, w, dst, (int)C, (int)D, (int)H,
                                   (int)Wd, (int)F, P, plane, tiles, R, cps, e);
            else
                hipLaunchKernelGGL(conv3d_thin_kernel<4>, grid, dim3(CONV_THREADS), shmem, s, x, w, dst, (int)C, (int)D, (int)H,
                                   (int)Wd, (int)F, P, plane, tiles, R, cps, e);
            HIP_OK(hipGetLastError());
            if (ksplit > 1) return fortis_launch_conv_split_reduce(dst, y, osize, D * H * Wd, ksplit, e, s);
            return 0;
        }
    }
    ConvShape sh = { (int)C, (int)D, (int)H, (int)Wd, (int)F, (int)KD, (int)KH, (int)KW, (int)Do, (int)Ho, (int)Wo, (int)sd,
                     (int)sh_, (int)sw_, (int)pd, (int)ph, (int)pw };
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
