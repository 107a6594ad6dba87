// Fused GEMM + bias + activation on the fp32 matrix cores:
//     C[B][N] = epi(A[B][K] . W[N][K]^T)
// One kernel replaces the reference's cuBLAS SGEMM (runtime/fortis_rt.c:45-75) AND the separate
// epilogue kernel fortis-fuse emits behind it (compiler/FortisFuse.cpp:685-692, 721-760: load C,
// add bias, activation, store), which re-reads and re-writes every activation once per layer.
//
// Tiling for CDNA4 (64-lane waves, v_mfma_f32_32x32x2f32, 4 SIMDs per CU):
//   workgroup tile BM x BN, 256 threads = 4 waves in a 2 x 2 grid, each wave (BM/2) x (BN/2) as
//   TM x TN MFMA tiles of 32 x 32; k is consumed in slabs of BK = 32 staged through LDS, double
//   buffered (global -> registers -> LDS while the previous slab is multiplied).
//   Both operands are k-contiguous in memory (A row-major, W[N][K]), so both are staged the same
//   way, and a lane reads 4 consecutive k as one 16-byte LDS load that feeds 4 MFMAs: MFMA step s
//   of an 8-wide k group uses k = 4h + s for lane half h, identically for A and B.
//   LDS rows are padded by 4 floats so the 16-byte reads of consecutive rows fall in different banks.
//   Workgroups are numbered so that each XCD (workgroup id mod 8) walks a contiguous band of row
//   tiles with the column tile fastest: the band's A rows and all of W stay in that XCD's L2.
#include "common.h"

typedef float v16f __attribute__((ext_vector_type(16)));

#define GM_THREADS 256
#define GM_BK 32
#define GM_LDK (GM_BK + 4)

struct GemmEpi {
    const float* bias;
    const float* out_scale;
    int act;
    float alpha;
    long mask_from;   // columns >= mask_from get ReLU (N when unused)
};

__device__ __forceinline__ float gemm_act(float v, int act, float alpha)
{
    if (act == FORTIS_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == FORTIS_ACT_LEAKY) return v > 0.f ? v : alpha * v;
    return v;
}

template <int BM, int BN>
__global__ __launch_bounds__(GM_THREADS) void gemm_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                          float* __restrict__ C, long B, long N, long K,
                                                          int tiles_n, long total_tiles, GemmEpi epi)
{
    constexpr int TM = BM / 64, TN = BN / 64;           // MFMA tiles per wave
    constexpr int LA = BM * GM_BK / 4 / GM_THREADS;     // float4 loads per thread per slab (A)
    constexpr int LW = BN * GM_BK / 4 / GM_THREADS;
    extern __shared__ float4 smem4[];
    float* sA = (float*)smem4;                          // [2][BM][GM_LDK]
    float* sW = sA + 2 * BM * GM_LDK;                   // [2][BN][GM_LDK]

    // XCD-aware tile numbering
    const long wg = blockIdx.x;
    const long per_xcd = (total_tiles + 7) / 8;
    const long logical = (wg & 7) * per_xcd + (wg >> 3);
    if (logical >= total_tiles) return;
    const long tm = logical / tiles_n, tn = logical - tm * tiles_n;
    const long m0 = tm * BM, n0 = tn * BN;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = (wave & 1) * (BM / 2), wn = (wave >> 1) * (BN / 2);
    const int lr = lane & 31, lh = lane >> 5;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    // staging map: float4 index f = tid + t*256 -> row = f / 8, kq = f % 8 (8 float4 per 32-wide row)
    float4 ra[LA], rw[LW];
    auto load_slab = [&](long k0) {
#pragma unroll
        for (int t = 0; t < LA; t++) {
            const int f = tid + t * GM_THREADS, row = f >> 3, kq = f & 7;
            const long gm = m0 + row, gk = k0 + kq * 4;
            ra[t] = (gm < B && gk < K) ? *(const float4*)(A + gm * K + gk) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int t = 0; t < LW; t++) {
            const int f = tid + t * GM_THREADS, row = f >> 3, kq = f & 7;
            const long gn = n0 + row, gk = k0 + kq * 4;
            rw[t] = (gn < N && gk < K) ? *(const float4*)(W + gn * K + gk) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    };
    auto store_slab = [&](int buf) {
        float* a = sA + buf * BM * GM_LDK;
        float* w = sW + buf * BN * GM_LDK;
#pragma unroll
        for (int t = 0; t < LA; t++) {
            const int f = tid + t * GM_THREADS, row = f >> 3, kq = f & 7;
            *(float4*)(a + row * GM_LDK + kq * 4) = ra[t];
        }
#pragma unroll
        for (int t = 0; t < LW; t++) {
            const int f = tid + t * GM_THREADS, row = f >> 3, kq = f & 7;
            *(float4*)(w + row * GM_LDK + kq * 4) = rw[t];
        }
    };

    const int nslab = (int)((K + GM_BK - 1) / GM_BK);
    load_slab(0);
    store_slab(0);
    __syncthreads();
    for (int sl = 0; sl < nslab; sl++) {
        const int buf = sl & 1;
        if (sl + 1 < nslab) load_slab((long)(sl + 1) * GM_BK);
        const float* a = sA + buf * BM * GM_LDK + (wm + lr) * GM_LDK + 4 * lh;
        const float* w = sW + buf * BN * GM_LDK + (wn + lr) * GM_LDK + 4 * lh;
#pragma unroll
        for (int kg = 0; kg < GM_BK / 8; kg++) {
            float4 fa[TM], fw[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) fa[i] = *(const float4*)(a + i * 32 * GM_LDK + kg * 8);
#pragma unroll
            for (int j = 0; j < TN; j++) fw[j] = *(const float4*)(w + j * 32 * GM_LDK + kg * 8);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].x, fw[j].x, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].y, fw[j].y, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].z, fw[j].z, acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i].w, fw[j].w, acc[i][j], 0, 0, 0);
                }
        }
        if (sl + 1 < nslab) store_slab(buf ^ 1);
        __syncthreads();
    }

    // epilogue: lane holds column n = lr of 16 rows per MFMA tile
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const long n = n0 + wn + j * 32 + lr;
        if (n >= N) continue;
        const float bv = epi.bias ? epi.bias[n] : 0.f;
        const float sv = epi.out_scale ? epi.out_scale[n] : 1.f;
        const bool relu_tail = n >= epi.mask_from;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const long m = m0 + wm + i * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
                if (m >= B) continue;
                float v = gemm_act(acc[i][j][r] + bv, epi.act, epi.alpha);
                if (epi.out_scale) v = v * sv;
                if (relu_tail) v = v > 0.f ? v : 0.f;
                C[m * N + n] = v;
            }
    }
}

// Generic guarded fallback for K not a multiple of 4 (16-byte row loads impossible): one thread
// per output element, fp32 FMA chain.  Correct for any shape; not a fast path.
__global__ void gemm_naive_kernel(const float* __restrict__ A, const float* __restrict__ W, float* __restrict__ C,
                                  long B, long N, long K, GemmEpi epi)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= B * N) return;
    const long m = idx / N, n = idx - m * N;
    float acc = 0.f;
    for (long k = 0; k < K; k++) acc = fmaf(A[m * K + k], W[n * K + k], acc);
    float v = gemm_act(acc + (epi.bias ? epi.bias[n] : 0.f), epi.act, epi.alpha);
    if (epi.out_scale) v = v * epi.out_scale[n];
    if (n >= epi.mask_from) v = v > 0.f ? v : 0.f;
    C[idx] = v;
}

template <int BM, int BN>
static void launch_tiled(const float* A, const float* W, float* C, long B, long N, long K, const GemmEpi& epi, hipStream_t s)
{
    const long tiles_m = cdiv(B, BM), tiles_n = cdiv(N, BN), total = tiles_m * tiles_n;
    const long grid = cdiv(total, 8) * 8;
    const size_t shmem = (size_t)2 * (BM + BN) * GM_LDK * sizeof(float);
    static bool attr = false;
    if (!attr) {
        HIP_OK(hipFuncSetAttribute((const void*)gemm_kernel<BM, BN>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        attr = true;
    }
    hipLaunchKernelGGL((gemm_kernel<BM, BN>), dim3((unsigned)grid), dim3(GM_THREADS), shmem, s, A, W, C, B, N, K,
                       (int)tiles_n, total, epi);
    HIP_OK(hipGetLastError());
}

int fortis_launch_gemm(const float* A, const float* W, const float* bias, float* C, long B, long N, long K,
                       int act, float alpha, const float* out_scale, long mask_tail, hipStream_t s)
{
    if (B <= 0 || N <= 0 || K <= 0) return -1;
    GemmEpi epi = { bias, out_scale, act, alpha, mask_tail > 0 ? N - mask_tail : N };
    const bool vec_ok = (K % 4 == 0) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
    if (!vec_ok) {
        hipLaunchKernelGGL(gemm_naive_kernel, dim3((unsigned)cdiv(B * N, 256)), dim3(256), 0, s, A, W, C, B, N, K, epi);
        HIP_OK(hipGetLastError());
        return 0;
    }
    static int force = -1;
    if (force < 0) { const char* e = getenv("FORTIS_GEMM_TILE"); force = e ? atoi(e) : 0; }
    // Large problems: 128 x 128 tiles; small ones use 64 x 64 so that more workgroups exist.
    const bool big = (force == 128) || (force == 0 && cdiv(B, 128) * cdiv(N, 128) >= 256);
    if (big) launch_tiled<128, 128>(A, W, C, B, N, K, epi, s);
    else launch_tiled<64, 64>(A, W, C, B, N, K, epi, s);
    return 0;
}
