// Fused MLP chain for narrow column networks (every width <= 256): the whole
// Linear+bias+activation stack runs in ONE kernel.  A workgroup owns 64 rows; their activations
// stay in LDS from the first layer to the last and never touch HBM.  Products run on the fp32
// matrix cores (v_mfma_f32_32x32x2f32); the weights are read straight from L2 into the MFMA B
// operand in a lane-ordered packing prepared once at plan time, so one 16-byte load per lane
// feeds four MFMAs.
//
// Replaces, for such networks, the reference's per-layer sequence
//   fortis_gemm (runtime/fortis_rt.c:45-75) -> epilogue kernel (compiler/FortisFuse.cpp:685-760)
// and its input-scaling / output-scaling elementwise kernels (FortisFuse.cpp:526-573).
// With STENCIL it also absorbs the gather in front of the model and the scatter behind it
// (mom6_zb/gather.cu:14-49, 58-81), so X[rows][n_in] and Y[rows][n_out] are never materialised.
//
// k ordering inside a dot product: MFMA step s of an 8-wide k group multiplies k = 4h + s for the
// two lane halves h = 0, 1.  A and B use the same order, so the result is a plain fp32 dot
// product with a different (fixed) summation order than the reference's; well inside 1e-5.
#include "stencil_dev.h"

typedef float v16f __attribute__((ext_vector_type(16)));

#define CH_ROWS 64
#define CH_THREADS 256

__device__ __forceinline__ float apply_act(float v, int act, float alpha)
{
    if (act == FORTIS_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == FORTIS_ACT_LEAKY) return v > 0.f ? v : alpha * v;
    return v;
}

template <bool STENCIL>
__global__ __launch_bounds__(CH_THREADS) void chain_kernel(ChainDesc d, const float* __restrict__ X,
                                                           float* __restrict__ Y, long rows,
                                                           const StencilDev* __restrict__ g,
                                                           const StencilDev* __restrict__ sc, PtrTab dG,
                                                           PtrTabW dS, float* __restrict__ Yraw)
{
    extern __shared__ float4 smem4[];
    const int ld = d.ld;
    float* cur = (float*)smem4;
    float* nxt = cur + CH_ROWS * ld;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long row0 = (long)blockIdx.x * CH_ROWS;
    const int K0 = d.L[0].K, K0p = d.L[0].Kp;

    // ---- phase 1: the 64 x K0 input tile into LDS ------------------------------------------
    if (STENCIL) {
        const int r = tid & (CH_ROWS - 1), part = tid / CH_ROWS;
        const long row = row0 + r;
        if (row < rows) {
            const long col = row % g->count;
            const int kk = (int)(row / g->count);
            int i, j;
            st_cell(g, col, i, j);
            float S[FORTIS_MAX_SCAL], c[FORTIS_MAX_INS];
            st_cell_values(g, dG, i, j, kk, S, c);
            for (int q = part; q < K0; q += CH_THREADS / CH_ROWS) {
                float tv = dG.p[g->refs[q].array][st_elem(g, g->refs[q], i, j, kk)];
                tv = st_chain(g, tv, S, c);
                if (d.in_div) tv = __fdiv_rn(tv, d.in_div[q]);
                cur[r * ld + q] = tv;
            }
        } else {
            for (int q = part; q < K0; q += CH_THREADS / CH_ROWS) cur[r * ld + q] = 0.f;
        }
    } else {
        const long base = row0 * K0;
        const long lim = rows * (long)K0 - base;   // valid elements from base
        for (int idx = tid; idx < CH_ROWS * K0; idx += CH_THREADS) {
            const int r = idx / K0, c = idx - r * K0;
            float v = idx < lim ? X[base + idx] : 0.f;
            if (d.in_div) v = __fdiv_rn(v, d.in_div[c]);
            cur[r * ld + c] = v;
        }
    }
    if (K0p > K0)
        for (int idx = tid; idx < CH_ROWS * (K0p - K0); idx += CH_THREADS) {
            const int r = idx / (K0p - K0), c = idx - r * (K0p - K0);
            cur[r * ld + K0 + c] = 0.f;
        }
    __syncthreads();

    // ---- phase 2: the layers, activations ping-ponging between the two LDS tiles -----------
    const int mt = wave & 1;
    for (int l = 0; l < d.nlayers; l++) {
        const int KG = d.L[l].Kp >> 3, NT = d.L[l].Np >> 5;
        const int act = d.L[l].act;
        const float alpha = d.L[l].alpha;
        const float* ap = cur + (mt * 32 + (lane & 31)) * ld + 4 * (lane >> 5);
        for (int nt = wave >> 1; nt < NT; nt += 2) {
            v16f acc;
#pragma unroll
            for (int i = 0; i < 16; i++) acc[i] = 0.f;
            const float4* wp = (const float4*)d.L[l].Wp + (size_t)nt * KG * 64 + lane;
#pragma unroll 4
            for (int kg = 0; kg < KG; kg++) {
                const float4 a = *(const float4*)(ap + kg * 8);
                const float4 b = wp[kg * 64];
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc, 0, 0, 0);
            }
            const int col = nt * 32 + (lane & 31);
            const float bv = d.L[l].bias[col];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int r = mt * 32 + 8 * (i >> 2) + 4 * (lane >> 5) + (i & 3);
                nxt[r * ld + col] = apply_act(acc[i] + bv, act, alpha);
            }
        }
        __syncthreads();
        float* t = cur; cur = nxt; nxt = t;
    }

    // ---- phase 3: results out ------------------------------------------------------------------
    const int NO = d.L[d.nlayers - 1].N;
    if (STENCIL) {
        if (tid < CH_ROWS) {
            const long row = row0 + tid;
            if (row < rows) {
                const long col = row % sc->count;
                const int kk = (int)(row / sc->count);
                int i, j;
                st_cell(sc, col, i, j);
                float S[FORTIS_MAX_SCAL], c[FORTIS_MAX_INS];
                st_cell_values(sc, dS, i, j, kk, S, c);
                for (int q = 0; q < NO; q++) {
                    float tv = cur[tid * ld + q];
                    if (d.out_mul) tv = __fmul_rn(tv, d.out_mul[q]);
                    if (Yraw) Yraw[row * NO + q] = tv;
                    tv = st_chain(sc, tv, S, c);
                    dS.p[sc->refs[q].array][st_elem(sc, sc->refs[q], i, j, kk)] = tv;
                }
            }
        }
    } else {
        const long base = row0 * NO;
        const long lim = rows * (long)NO - base;
        for (int idx = tid; idx < CH_ROWS * NO; idx += CH_THREADS) {
            if (idx >= lim) break;
            const int r = idx / NO, c = idx - r * NO;
            float v = cur[r * ld + c];
            if (d.out_mul) v = __fmul_rn(v, d.out_mul[c]);
            if (c >= NO - d.mask_tail) v = v > 0.f ? v : 0.f;
            Y[base + idx] = v;
        }
    }
}

// ---- host side ---------------------------------------------------------------------------------
float* fortis_chain_pack_weights(const float* W, long N, long K, int* Kp_out, int* Np_out)
{
    const int Kp = (int)cdiv(K, 8) * 8, Np = (int)cdiv(N, 32) * 32;
    const int KG = Kp / 8, NT = Np / 32;
    const size_t n = (size_t)Np * Kp;
    float* h = (float*)calloc(n, sizeof(float));
    for (int nt = 0; nt < NT; nt++)
        for (int kg = 0; kg < KG; kg++)
            for (int lane = 0; lane < 64; lane++)
                for (int s = 0; s < 4; s++) {
                    const long nn = nt * 32 + (lane & 31), kk = kg * 8 + 4 * (lane >> 5) + s;
                    if (nn < N && kk < K) h[(((size_t)nt * KG + kg) * 64 + lane) * 4 + s] = W[nn * K + kk];
                }
    float* dptr = nullptr;
    HIP_OK(hipMalloc((void**)&dptr, n * sizeof(float)));
    HIP_OK(hipMemcpy(dptr, h, n * sizeof(float), hipMemcpyHostToDevice));
    free(h);
    *Kp_out = Kp;
    *Np_out = Np;
    return dptr;
}

float* fortis_chain_pack_bias(const float* b, long N, int Np)
{
    float* h = (float*)calloc(Np, sizeof(float));
    if (b) memcpy(h, b, N * sizeof(float));
    float* dptr = nullptr;
    HIP_OK(hipMalloc((void**)&dptr, Np * sizeof(float)));
    HIP_OK(hipMemcpy(dptr, h, Np * sizeof(float), hipMemcpyHostToDevice));
    free(h);
    return dptr;
}

int fortis_chain_ld(const ChainDesc& d)
{
    int w = 0;
    for (int l = 0; l < d.nlayers; l++) {
        if (d.L[l].Kp > w) w = d.L[l].Kp;
        if (d.L[l].Np > w) w = d.L[l].Np;
    }
    return w + 4;   // +4 floats: consecutive rows start 4 banks apart, 16-byte reads stay aligned
}

static bool chain_check(const ChainDesc& d)
{
    if (d.nlayers < 1 || d.nlayers > FORTIS_CHAIN_MAX_LAYERS) return false;
    for (int l = 0; l < d.nlayers; l++) {
        if (d.L[l].K > FORTIS_CHAIN_MAX_WIDTH || d.L[l].N > FORTIS_CHAIN_MAX_WIDTH) return false;
        if (l && d.L[l].K != d.L[l - 1].N) return false;
        if (d.L[l].Kp % 8 || d.L[l].Np % 32 || d.L[l].Kp < d.L[l].K || d.L[l].Np < d.L[l].N) return false;
    }
    return d.ld >= fortis_chain_ld(d) && d.ld % 4 == 0;
}

template <bool ST>
static void chain_launch(const ChainDesc& d, const float* X, float* Y, long rows, const StencilDev* g,
                         const StencilDev* sc, const PtrTab& dG, const PtrTabW& dS, float* Yraw, hipStream_t s)
{
    if (!chain_check(d)) { fprintf(stderr, "fortis: MLP chain descriptor rejected by the kernel launcher\n"); return; }
    if (rows <= 0) return;
    const size_t shmem = (size_t)2 * CH_ROWS * d.ld * sizeof(float);
    static size_t attr_set[2] = { 0, 0 };
    if (shmem > attr_set[ST]) {
        HIP_OK(hipFuncSetAttribute((const void*)chain_kernel<ST>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        attr_set[ST] = shmem;
    }
    hipLaunchKernelGGL(chain_kernel<ST>, dim3((unsigned)cdiv(rows, CH_ROWS)), dim3(CH_THREADS), shmem, s, d, X, Y, rows, g,
                       sc, dG, dS, Yraw);
    HIP_OK(hipGetLastError());
}

void fortis_launch_chain(const ChainDesc& d, const float* X, float* Y, long rows, hipStream_t s)
{
    PtrTab a = {};
    PtrTabW b = {};
    chain_launch<false>(d, X, Y, rows, nullptr, nullptr, a, b, nullptr, s);
}

// g_dev / sc_dev are device copies of the lowered tables; g_host gives the row count.
void fortis_launch_chain_stencil_dev(const ChainDesc& d, const StencilDev* g_dev, const StencilDev* sc_dev,
                                     long rows, const float* const* dG, int nG, float* const* dS, int nS,
                                     float* dY, hipStream_t s)
{
    PtrTab a = {};
    PtrTabW b = {};
    for (int i = 0; i < nG; i++) a.p[i] = dG[i];
    for (int i = 0; i < nS; i++) b.p[i] = dS[i];
    chain_launch<true>(d, nullptr, nullptr, rows, g_dev, sc_dev, a, b, dY, s);
}
