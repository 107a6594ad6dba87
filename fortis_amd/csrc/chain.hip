// Fused MLP chain for narrow column networks (every width <= 256): the whole
// Linear+bias+activation stack runs in ONE kernel, and with STENCIL also the gather in front of the
// model and the scatter behind it (mom6_zb/gather.cu:14-49, 58-81), so X[rows][n_in] and
// Y[rows][n_out] are never materialised in HBM.
//
// Replaces, for such networks, the reference's per-layer sequence
//   fortis_gemm (runtime/fortis_rt.c:45-75) -> epilogue kernel (compiler/FortisFuse.cpp:685-760)
// and its input-scaling / output-scaling elementwise kernels (FortisFuse.cpp:526-573).
//
// Shape of the kernel on CDNA4:
//   * persistent workgroups: each loops over row tiles (ROWS rows), so per-workgroup set-up is paid
//     once and global-memory latency is hidden by software pipelining: the loads of tile t+1 (the
//     stencil slot values, or the X rows) are issued before the layers of tile t run;
//   * activations of a tile stay in LDS from the first layer to the last (two ping-pong tiles);
//   * weights and biases of all layers are copied into LDS once per workgroup when they fit (they
//     are read from L2 otherwise), in a lane-ordered packing prepared at plan time: one 16-byte read
//     per lane feeds four MFMAs;
//   * products run on the fp32 matrix cores with v_mfma_f32_16x16x4f32: 16-row m-tiles keep all four
//     waves busy even for a 3-wide output layer, and padding is to 16, not 32.
//
// k ordering inside a dot product: MFMA step s of a 16-wide k group multiplies k = 4q + s for the
// four lane quarters q.  A and B use the same order, so the result is a plain fp32 dot product with
// a different (fixed) summation order than the reference's; well inside 1e-5.
#include "stencil_dev.h"

typedef float v4f __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) v4f gv4f;   // 16 bytes of global memory

#define CH_THREADS 256
#define CH_NACC 4       // n-tiles a wave accumulates at once

// max(v, 0) in one instruction, on the bit pattern: a float with the sign bit set is a negative integer, so the signed
// integer maximum with 0 leaves positive values as they are and turns negative ones and -0 into +0 (a NaN keeps its
// bits if its sign is clear and becomes +0 otherwise, where apply_act below turns every NaN into 0: the forms of a
// network agree bit for bit on everything but NaN activations, which the parity contract leaves open).  fmaxf(v, 0.f) costs two instructions on an accumulator that
// comes straight from a matrix instruction: the compiler first quiets a possible signalling NaN with v_max_f32 v, v
// (it does not know that matrix results are already canonical, and it rewrites v_med3_f32(v, 0, inf) to the same
// pair).  Written in C, not as inline assembly: the compiler then keeps its own bookkeeping of the wait states between
// a matrix instruction and a reader of its result (an asm statement escapes it and read accumulators too early).
__device__ __forceinline__ float relu_acc(float v)
{
    const int b = __float_as_int(v);
    return __int_as_float(b > 0 ? b : 0);
}

__device__ __forceinline__ float apply_act(float v, int act, float alpha)
{
    if (act == FORTIS_ACT_RELU) return v > 0.f ? v : 0.f;
    if (act == FORTIS_ACT_LEAKY) return v > 0.f ? v : alpha * v;
    return v;
}

// Everything a launch needs, passed by value and copied to LDS by the kernel (params_to_lds).
struct alignas(16) ChainParams {
    ChainDesc d;
    unsigned rows, ntiles;
    const float* X;
    float* Y;
    float* Yraw;
    long pad_;
    GatherArgs g;
    ScatterArgs sc;
};
struct LayerRegs { int KG, NT, act, woff, boff; float alpha; };
__device__ __forceinline__ LayerRegs layer_regs(const ChainDesc& d, int l)
{
    LayerRegs r;
    r.KG = st_u(d.L[l].Kp >> 4); r.NT = st_u(d.L[l].Np >> 4); r.act = st_u(d.L[l].act);
    r.woff = st_u(d.L[l].woff); r.boff = st_u(d.L[l].boff);
    r.alpha = __builtin_bit_cast(float, st_u(__builtin_bit_cast(int, d.L[l].alpha)));
    return r;
}

// ---------------------------------------------------------------------------------------------------
// Workgroup-tile variant (plain X -> Y only): ROWS rows per workgroup, activations ping-pong between
// two LDS tiles, the four waves split the m-tiles (ROWS = 64) or the n-tiles of one m-tile (ROWS = 16,
// which spreads a small batch over more CUs).  Persistent over tiles, next X tile prefetched.
template <int ROWS, bool WLDS>
__global__ __launch_bounds__(CH_THREADS) __attribute__((amdgpu_waves_per_eu(1, 2)))
void chain_kernel(ChainParams params)
{
    constexpr int MT = ROWS / 16;          // m-tiles per workgroup
    constexpr int WPM = 4 / MT;            // waves sharing one m-tile (they split the n-tiles)
    constexpr int XR = 16;                 // prefetch registers: tiles up to 4096 floats
    __shared__ ChainParams P;
    extern __shared__ float4 smem4[];
    params_to_lds(&P, CH_THREADS);
    const ChainDesc& d = P.d;
    float* sWts = (float*)smem4;                               // all layers' packed weights + biases (WLDS)
    const int wfloats = st_u(d.wfloats), ld = st_u(d.ld), nlayers = st_u(d.nlayers);
    float* buf0 = sWts + (WLDS ? wfloats : 0);
    float* buf1 = buf0 + ROWS * ld;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K0 = st_u(d.L[0].K), K0p = st_u(d.L[0].Kp);
    const int NO = st_u(d.L[nlayers - 1].N), mask_tail = st_u(d.mask_tail);
    const unsigned rows = P.rows, ntiles = P.ntiles;
    const gfloat* X = st_g(P.X);
    gfloat* Y = st_g(P.Y);
    const gfloat* wall = st_g(d.wall);
    const gfloat* in_div = st_g(d.in_div);
    const gfloat* out_mul = st_g(d.out_mul);

    if (WLDS) {
        const int n4 = wfloats / 4;
        for (int i0 = tid; i0 < n4; i0 += 8 * CH_THREADS) {
            v4f r[8];
#pragma unroll
            for (int u = 0; u < 8; u++) { const int i = i0 + u * CH_THREADS; r[u] = ((const gv4f*)wall)[i < n4 ? i : n4 - 1]; }
#pragma unroll
            for (int u = 0; u < 8; u++) { const int i = i0 + u * CH_THREADS; if (i < n4) ((v4f*)sWts)[i] = r[u]; }
        }
    }
    float xr[XR];
    const bool pre = ROWS * K0 <= XR * CH_THREADS;
    auto issue = [&](unsigned tile) {
        if (!pre) return;
        const long base = (long)tile * ROWS * K0;
        const long lim = (long)rows * K0 - base;
#pragma unroll
        for (int t = 0; t < XR; t++) {
            const int idx = tid + t * CH_THREADS;
            xr[t] = (idx < ROWS * K0 && idx < lim) ? __builtin_nontemporal_load(&X[base + idx]) : 0.f;
        }
    };
    auto land = [&](unsigned tile) {
        if (pre) {
#pragma unroll
            for (int t = 0; t < XR; t++) {
                const int idx = tid + t * CH_THREADS;
                if (idx < ROWS * K0) {
                    const int r = idx / K0, c = idx - r * K0;
                    float v = xr[t];
                    if (in_div) v = __fdiv_rn(v, in_div[c]);
                    buf0[r * ld + c] = v;
                }
            }
        } else {
            // tile too wide for the prefetch registers: loaded here, latency exposed
            const long base = (long)tile * ROWS * K0;
            const long lim = (long)rows * K0 - base;
            for (int idx = tid; idx < ROWS * K0; idx += CH_THREADS) {
                const int r = idx / K0, c = idx - r * K0;
                float v = idx < lim ? X[base + idx] : 0.f;
                if (in_div) v = __fdiv_rn(v, in_div[c]);
                buf0[r * ld + c] = v;
            }
        }
        if (K0p > K0)
            for (int idx = tid; idx < ROWS * (K0p - K0); idx += CH_THREADS) {
                const int r = idx / (K0p - K0), c = idx - r * (K0p - K0);
                buf0[r * ld + K0 + c] = 0.f;
            }
    };

    unsigned tile = blockIdx.x;
    if (tile < ntiles) issue(tile);
    const int mt = wave % MT, ng = wave / MT;
    const int lrow = lane & 15, lq = lane >> 4;

    for (; tile < ntiles; tile += gridDim.x) {
        land(tile);
        __syncthreads();
        const unsigned next = tile + gridDim.x;
        if (next < ntiles) issue(next);
        float* cur = buf0;
        float* nxt = buf1;
        for (int l = 0; l < nlayers; l++) {
            const LayerRegs R = layer_regs(d, l);
            const float* ap = cur + (mt * 16 + lrow) * ld + 4 * lq;
            for (int nt0 = ng; nt0 < R.NT; nt0 += WPM * CH_NACC) {
                v4f acc[CH_NACC];
#pragma unroll
                for (int u = 0; u < CH_NACC; u++) acc[u] = (v4f){ 0.f, 0.f, 0.f, 0.f };
                for (int kg = 0; kg < R.KG; kg++) {
                    const v4f a = *(const v4f*)(ap + kg * 16);
                    v4f b[CH_NACC];
#pragma unroll
                    for (int u = 0; u < CH_NACC; u++) {
                        const int nt = nt0 + u * WPM;
                        const int off = R.woff / 4 + ((nt < R.NT ? nt : nt0) * R.KG + kg) * 64 + lane;
                        if (WLDS) b[u] = ((const v4f*)sWts)[off]; else b[u] = ((const gv4f*)wall)[off];
                    }
#pragma unroll
                    for (int u = 0; u < CH_NACC; u++) {
                        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b[u].x, acc[u], 0, 0, 0);
                        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b[u].y, acc[u], 0, 0, 0);
                        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b[u].z, acc[u], 0, 0, 0);
                        acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b[u].w, acc[u], 0, 0, 0);
                    }
                }
#pragma unroll
                for (int u = 0; u < CH_NACC; u++) {
                    const int nt = nt0 + u * WPM;
                    if (nt < R.NT) {
                        const int col = nt * 16 + lrow;
                        const float bv = WLDS ? sWts[R.boff + col] : wall[R.boff + col];
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            nxt[(mt * 16 + 4 * lq + r) * ld + col] = apply_act(acc[u][r] + bv, R.act, R.alpha);
                    }
                }
            }
            __syncthreads();
            float* t = cur; cur = nxt; nxt = t;
        }
        const long base = (long)tile * ROWS * NO;
        const long lim = (long)rows * NO - base;
        for (int idx = tid; idx < ROWS * NO; idx += CH_THREADS) {
            if (idx >= lim) break;
            const int r = idx / NO, c = idx - r * NO;
            float v = cur[r * ld + c];
            if (out_mul) v = __fmul_rn(v, out_mul[c]);
            if (c >= NO - mask_tail) v = v > 0.f ? v : 0.f;
            __builtin_nontemporal_store(v, &Y[base + idx]);
        }
        // the next land() writes buf0 while slower threads may still read `cur` above
        __syncthreads();
    }
}

// NTG n-tiles (starting at nt0) of one layer for the wave's 16 rows, in registers.
// The product is formed transposed, D = W . X^T: the weights are the MFMA's A operand and the rows'
// activations its B operand, so a lane ends up with features n = 16 nt + 4 (lane / 16) + r, r = 0..3, of
// row lane % 16 -- exactly the four consecutive k a lane must supply for k group nt of the NEXT layer.
// A layer's output registers are therefore the next layer's input registers: no LDS round trip, no
// barrier between layers.  The accumulators start at the bias.
template <int NTG, int KGMAX, bool WLDS>
__device__ __forceinline__ void layer_group(const v4f (&a)[KGMAX], v4f* o, const float* sWts, const gfloat* wall,
                                            int woff4, int boff, int nt0, int KG, int lane, int lq)
{
    v4f acc[NTG];
#pragma unroll
    for (int u = 0; u < NTG; u++) {
        const int bo = (boff + (nt0 + u) * 16) / 4 + lq;
        if (WLDS) acc[u] = ((const v4f*)sWts)[bo]; else acc[u] = ((const gv4f*)wall)[bo];
    }
#pragma unroll
    for (int kg = 0; kg < KGMAX; kg++) {
        if (kg < KG) {
            v4f w[NTG];
#pragma unroll
            for (int u = 0; u < NTG; u++) {
                const int off = woff4 + ((nt0 + u) * KG + kg) * 64 + lane;
                if (WLDS) w[u] = ((const v4f*)sWts)[off]; else w[u] = ((const gv4f*)wall)[off];
            }
#pragma unroll
            for (int u = 0; u < NTG; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].x, a[kg].x, acc[u], 0, 0, 0);
#pragma unroll
            for (int u = 0; u < NTG; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].y, a[kg].y, acc[u], 0, 0, 0);
#pragma unroll
            for (int u = 0; u < NTG; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].z, a[kg].z, acc[u], 0, 0, 0);
#pragma unroll
            for (int u = 0; u < NTG; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].w, a[kg].w, acc[u], 0, 0, 0);
        }
    }
#pragma unroll
    for (int u = 0; u < NTG; u++) o[u] = acc[u];
}

// One layer of a narrow network (at most four 16-wide k groups and n-tiles) as straight-line code: NT and KG are
// compile-time, so every weight and bias read is a per-lane base (set once per layer) plus a literal offset, no
// branch separates the reads from the MFMAs and the compiler is free to issue the reads ahead.  The activation is
// applied in place: a[0 .. NT) leave as the next layer's operand.
// RELU: the activation is known to be ReLU (no choice left in the code).
template <int NT, int KG, bool WLDS, bool RELU = false>
__device__ __forceinline__ void layer_fixed(v4f (&a)[4], const float* sWts, const gfloat* wall, int woff4, int boff, int lane,
                                            int lq, int act, float alpha)
{
    v4f acc[NT];
    const v4f* wl = (const v4f*)sWts + woff4 + lane;
    const v4f* bl = (const v4f*)sWts + boff / 4 + lq;
    const gv4f* wg = (const gv4f*)wall + woff4 + lane;
    const gv4f* bg = (const gv4f*)wall + boff / 4 + lq;
#pragma unroll
    for (int u = 0; u < NT; u++) { if (WLDS) acc[u] = bl[u * 4]; else acc[u] = bg[u * 4]; }
#pragma unroll
    for (int kg = 0; kg < KG; kg++) {
        v4f w[NT];
#pragma unroll
        for (int u = 0; u < NT; u++) { if (WLDS) w[u] = wl[(u * KG + kg) * 64]; else w[u] = wg[(u * KG + kg) * 64]; }
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].x, a[kg].x, acc[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].y, a[kg].y, acc[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].z, a[kg].z, acc[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[u].w, a[kg].w, acc[u], 0, 0, 0);
    }
    if (RELU || act == FORTIS_ACT_RELU) {
#pragma unroll
        for (int u = 0; u < NT; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) a[u][r] = relu_acc(acc[u][r]);
    } else if (act == FORTIS_ACT_NONE) {
#pragma unroll
        for (int u = 0; u < NT; u++) a[u] = acc[u];
    } else {
#pragma unroll
        for (int u = 0; u < NT; u++)
#pragma unroll
            for (int r = 0; r < 4; r++) a[u][r] = apply_act(acc[u][r], act, alpha);
    }
}
// The layer's shape picks its code once per layer (wave-uniform).
template <bool WLDS>
__device__ __forceinline__ void layer_narrow(v4f (&a)[4], const LayerRegs& R, const float* sWts, const gfloat* wall, int lane, int lq)
{
#define FORTIS_LF(NT_, KG_) case (NT_) * 4 + (KG_): layer_fixed<NT_, KG_, WLDS>(a, sWts, wall, R.woff / 4, R.boff, lane, lq, R.act, R.alpha); break;
    switch (R.NT * 4 + R.KG) {
        FORTIS_LF(1, 1) FORTIS_LF(1, 2) FORTIS_LF(1, 3) FORTIS_LF(1, 4)
        FORTIS_LF(2, 1) FORTIS_LF(2, 2) FORTIS_LF(2, 3) FORTIS_LF(2, 4)
        FORTIS_LF(3, 1) FORTIS_LF(3, 2) FORTIS_LF(3, 3) FORTIS_LF(3, 4)
        FORTIS_LF(4, 1) FORTIS_LF(4, 2) FORTIS_LF(4, 3) FORTIS_LF(4, 4)
        default: break;
    }
#undef FORTIS_LF
}

// A last layer of at most four outputs as v_mfma_f32_4x4x1 products (a quarter of the matrix time of a 16-wide
// n-tile that is mostly padding): a block of four lanes is four rows of one quarter q, lane i of it brings output
// i's weight for the feature those rows bring, and every lane ends up with its row's four outputs summed over the 16
// features per k group that its quarter carries (quarter 0 starts at the bias).  The quarters' sums are still to
// be added: last_x4_sum does it across the lanes, (q0 + q2) + (q1 + q3), and applies the activation.
template <bool WLDS, int KGX = 0>      // KGX > 0: the layer's k groups, known at compile time
__device__ __forceinline__ v4f last_x4_partial(const v4f (&a)[4], const LayerRegs& R, int x4off, const float* sWts, const gfloat* wall,
                                               int lane, int lq)
{
    const int wo = x4off / 4 + (lq * 4 + (lane & 3)) * R.KG;
    v4f acc;
    if (WLDS) acc = ((const v4f*)sWts)[R.boff / 4]; else acc = ((const gv4f*)wall)[R.boff / 4];
    if (lq) acc = (v4f)(0.f);
#pragma unroll
    for (int u = 0; u < 4; u++)
        if (KGX ? u < KGX : u < R.KG) {
            v4f w;
            if (WLDS) w = ((const v4f*)sWts)[wo + u]; else w = ((const gv4f*)wall)[wo + u];
            acc = __builtin_amdgcn_mfma_f32_4x4x1f32(w.x, a[u].x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_4x4x1f32(w.y, a[u].y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_4x4x1f32(w.z, a[u].z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_4x4x1f32(w.w, a[u].w, acc, 0, 0, 0);
        }
    return acc;
}
__device__ __forceinline__ v4f last_x4_sum(v4f acc, const LayerRegs& R)
{
#pragma unroll
    for (int r = 0; r < 4; r++) {
        float v = acc[r];
        v += __shfl_xor(v, 32);
        v += __shfl_xor(v, 16);
        acc[r] = apply_act(v, R.act, R.alpha);
    }
    return acc;
}

// All layers of a narrow network on the operand in a[]; the result is left in a[].  XSUM false: a last layer in the
// 4x4x1 form leaves each quarter's partial sums in a[0] and returns true; the caller adds them, (q0 + q2) + (q1 + q3),
// and applies the layer's activation.
// SIG: the network's shape when the launcher has matched it (chain_signature), 0 otherwise.  A matched network runs as
// straight-line code; the general path picks each layer's code by a switch on its shape, whose arms the compiler joins
// with copies of the operand registers -- 16 moves per layer and 16 rows.
//   SIG 1: Kp 32 -> 64 -> 64 -> at most 4 outputs (4x4x1 form), ReLU behind both hidden layers
//   SIG 2: Kp 32 -> 32 -> at most 4 outputs (4x4x1 form), ReLU behind the hidden layer
template <bool WLDS, bool XSUM = true, int SIG = 0>
__device__ __forceinline__ bool layers_narrow(v4f (&a)[4], const ChainDesc& d, int nlayers, const float* sWts, const gfloat* wall, int lane, int lq)
{
    if constexpr (SIG == 1 || SIG == 2) {
        asm volatile("" ::: "memory");
        const LayerRegs R0 = layer_regs(d, 0);
        if constexpr (SIG == 1) layer_fixed<4, 2, WLDS, true>(a, sWts, wall, R0.woff / 4, R0.boff, lane, lq, FORTIS_ACT_RELU, 0.f);
        else layer_fixed<2, 2, WLDS, true>(a, sWts, wall, R0.woff / 4, R0.boff, lane, lq, FORTIS_ACT_RELU, 0.f);
        if constexpr (SIG == 1) {
            asm volatile("" ::: "memory");
            const LayerRegs R1 = layer_regs(d, 1);
            layer_fixed<4, 4, WLDS, true>(a, sWts, wall, R1.woff / 4, R1.boff, lane, lq, FORTIS_ACT_RELU, 0.f);
        }
        asm volatile("" ::: "memory");
        const LayerRegs R = layer_regs(d, SIG == 1 ? 2 : 1);
        const v4f part = last_x4_partial<WLDS, SIG == 1 ? 4 : 2>(a, R, st_u(d.x4off), sWts, wall, lane, lq);
        a[0] = XSUM ? last_x4_sum(part, R) : part;
        return true;
    }
    const int x4off = st_u(d.x4off);
    const int nfull = x4off >= 0 ? nlayers - 1 : nlayers;
    for (int l = 0; l < nfull; l++) {
        asm volatile("" ::: "memory");
        const LayerRegs R = layer_regs(d, l);
        layer_narrow<WLDS>(a, R, sWts, wall, lane, lq);
    }
    if (x4off >= 0) {
        asm volatile("" ::: "memory");
        const LayerRegs R = layer_regs(d, nlayers - 1);
        const v4f part = last_x4_partial<WLDS>(a, R, x4off, sWts, wall, lane, lq);
        a[0] = XSUM ? last_x4_sum(part, R) : part;
    }
    return x4off >= 0;
}

// ---------------------------------------------------------------------------------------------------
// Wave-independent, register-resident variant: ONE WAVE owns 16 rows from the gather (or the X load)
// to the scatter (or the Y store), and the activations never leave its registers (see layer_group).
// Lane (row = lane % 16, q = lane / 16) holds, per 16-wide k group, the four features 4q..4q+3 of its
// row: the gather loads exactly those slots, the last layer leaves exactly those outputs.  The four
// waves of a workgroup only share the LDS copies of the parameter block and of the weights.  The grid
// is persistent; the global loads of a wave's next tile are issued before the current one is computed.
template <bool STENCIL, bool WLDS, int NTMAX, int SIG = 0>
__global__ __launch_bounds__(CH_THREADS) __attribute__((amdgpu_waves_per_eu(NTMAX <= 4 ? 4 : 2, NTMAX <= 4 ? 4 : 2)))
void chain_wave_kernel(ChainParams params)
{
    constexpr int KG0 = STENCIL ? ST_KREFS / 16 : NTMAX;   // k groups the first layer can read
    constexpr bool PREFETCH = KG0 <= 4;                           // wide inputs: no second register set
    constexpr int NTO = STENCIL ? ST_KREFS / 16 : NTMAX;   // n-tiles the output stage can write
    __shared__ ChainParams P;
    extern __shared__ float4 smem4[];
    params_to_lds(&P, CH_THREADS);
    const ChainDesc& d = P.d;
    const GatherArgs& g = P.g;
    const ScatterArgs& sc = P.sc;
    float* sWts = (float*)smem4;
    const int wfloats = st_u(d.wfloats), nlayers = st_u(d.nlayers);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K0 = st_u(d.L[0].K);
    const int NO = st_u(d.L[nlayers - 1].N), mask_tail = st_u(d.mask_tail);
    const unsigned rows = (unsigned)st_u((int)P.rows);
    const int lrow = lane & 15, lq = lane >> 4;
    const gfloat* wall = st_g(d.wall);
    const gfloat* in_div = st_g(d.in_div);
    const gfloat* out_mul = st_g(d.out_mul);
    const bool g_uniform = STENCIL && st_u(g.uniform) != 0;
    const bool s_uniform = STENCIL && st_u(sc.uniform) != 0;
    const bool s_refs_uniform = STENCIL && st_u(sc.refs_uniform) != 0;     // one store offset per cell
    // gather and scatter usually visit the same cells in the same order: decode a row once
    const bool same_cells = STENCIL && st_u((int)(g.count == sc.count && g.ni == sc.ni && g.ilo == sc.ilo && g.jlo == sc.jlo &&
                                                  g.sx == sc.sx && g.cells == sc.cells)) != 0;
    const bool xvec = !STENCIL && st_u((int)((K0 & 3) == 0 && ((uintptr_t)P.X & 15) == 0)) != 0;   // 16-byte X loads
    const bool yvec = !STENCIL && st_u((int)((NO & 3) == 0 && ((uintptr_t)P.Y & 15) == 0)) != 0;   // 16-byte Y stores

    // Everything a tile reads from global memory, as registers: the first layer's operand (slot values
    // or X), and for the stencil form the gather scalars and scatter scalars of the lane's cell.
    struct TileIn {
        v4f x[KG0];
        float gS[ST_SCAL_MAX], sS[ST_SCAL_MAX];
        int si, sj, skk;
        unsigned row0;
    };
    // ---- issues every global load of the tile at row0 ---------------------------------------------------
    auto issue = [&](TileIn& in, unsigned row0) __attribute__((always_inline)) {
        in.row0 = row0;
        in.si = in.sj = in.skk = 0;
        const unsigned row = row0 + lrow;
        if (STENCIL) {
            const unsigned rc = row < rows ? row : 0;
            int i, j, kk;
            st_row(g, rc, i, j, kk);
            if (same_cells) { in.si = i; in.sj = j; in.skk = kk; }
            else st_row(sc, rc, in.si, in.sj, in.skk);
            if (g_uniform) {
                // one element offset per cell; a slot is then its pointer plus that offset
                const long off = st_off(g.refs[0], i, j, kk);
#pragma unroll
                for (int kg = 0; kg < KG0; kg++)
#pragma unroll
                    for (int s4 = 0; s4 < 4; s4++) {
                        const int q = 16 * kg + 4 * lq + s4;
                        in.x[kg][s4] = st_g(g.refs[q].p)[off];      // entries past nrefs repeat slot 0
                    }
#pragma unroll
                for (int s = 0; s < ST_SCAL_MAX; s++) in.gS[s] = st_g(g.scal[s].p)[off];
            } else {
#pragma unroll
                for (int kg = 0; kg < KG0; kg++)
#pragma unroll
                    for (int s4 = 0; s4 < 4; s4++) {
                        const int q = 16 * kg + 4 * lq + s4;
                        const StSlotT<const float*> sl = g.refs[q < K0 ? q : 0];
                        in.x[kg][s4] = st_g(sl.p)[st_off(sl, i, j, kk)];
                    }
#pragma unroll
                for (int s = 0; s < ST_SCAL_MAX; s++) {
                    const StSlotT<const float*> sl = g.scal[s < g.nscal ? s : 0];
                    in.gS[s] = st_g(sl.p)[st_off(sl, i, j, kk)];
                }
            }
            if (s_uniform) {
                const long off = st_off(sc.refs[0], in.si, in.sj, in.skk);
#pragma unroll
                for (int s = 0; s < ST_SCAL_MAX; s++) in.sS[s] = st_g(sc.scal[s].p)[off];
            } else {
#pragma unroll
                for (int s = 0; s < ST_SCAL_MAX; s++) {
                    const StSlotT<float*> sl = sc.scal[s];
                    in.sS[s] = st_g(sl.p)[st_off(sl, in.si, in.sj, in.skk)];
                }
            }
        } else {
            // X is read once and Y written once: both go through non-temporal accesses so that a row stream of
            // gigabytes does not push the neighbouring kernels' grids out of the 256 MB memory-side cache (the
            // stencil gather that follows a 1028 x 1028 x 15 step ran 0.43 ms behind plain accesses, 0.30 ms now).
            // The price, for rows that are not whole 16-byte vectors: the 4-byte loads of a row come back to lines
            // that have already left the cache, and the fetch counter reads 1.12 times X (1.00 with plain loads).
            const gfloat* xrow = st_g(P.X) + (size_t)(row < rows ? row : 0) * K0;
#pragma unroll
            for (int kg = 0; kg < KG0; kg++) {
                const int c = 16 * kg + 4 * lq;
                if (xvec) {
                    in.x[kg] = c < K0 ? __builtin_nontemporal_load((const gv4f*)(xrow + c)) : (v4f)(0.f);
                } else {
#pragma unroll
                    for (int s4 = 0; s4 < 4; s4++) in.x[kg][s4] = c + s4 < K0 ? __builtin_nontemporal_load(xrow + c + s4) : 0.f;
                }
            }
        }
    };
    // ---- one tile: first operand from the loaded values, the layers in registers, results out ----------
    auto process = [&](TileIn& in) __attribute__((always_inline)) {
        const unsigned row = in.row0 + lrow;
        const bool valid = row < rows;
        v4f a[NTMAX], o[NTMAX];
#pragma unroll
        for (int kg = 0; kg < NTMAX; kg++) a[kg] = (v4f)(0.f);
        if (STENCIL) {
            StCell cell;
#pragma unroll
            for (int s = 0; s < ST_SCAL_MAX; s++) cell.S[s] = in.gS[s];
            st_cell_program(g, cell);
            float tv[KG0 * 4];
#pragma unroll
            for (int t = 0; t < KG0 * 4; t++) tv[t] = in.x[t >> 2][t & 3];
            st_chain_apply(g, cell, tv);
#pragma unroll
            for (int t = 0; t < KG0 * 4; t++) {
                const int q = 16 * (t >> 2) + 4 * lq + (t & 3);
                float v = (valid && q < K0) ? tv[t] : 0.f;
                if (in_div && q < K0) v = __fdiv_rn(v, in_div[q]);
                if ((t >> 2) < NTMAX) a[(t >> 2) < NTMAX ? (t >> 2) : 0][t & 3] = v;
            }
        } else {
#pragma unroll
            for (int kg = 0; kg < KG0; kg++)
#pragma unroll
                for (int s4 = 0; s4 < 4; s4++) {
                    const int c = 16 * kg + 4 * lq + s4;
                    float v = (valid && c < K0) ? in.x[kg][s4] : 0.f;
                    if (in_div && c < K0) v = __fdiv_rn(v, in_div[c]);
                    a[kg][s4] = v;
                }
        }
        if constexpr (NTMAX == 4 && !STENCIL) {           // (the general stencil form has no registers to spare for it)
            __builtin_amdgcn_s_setprio(3);          // as in the fused forms: the matrix phase outranks the other waves' loads and stores
            layers_narrow<WLDS, true, SIG>(a, d, nlayers, sWts, wall, lane, lq);
            __builtin_amdgcn_s_setprio(0);
        } else
        for (int l = 0; l < nlayers; l++) {
            asm volatile("" ::: "memory");
            const LayerRegs R = layer_regs(d, l);
            if constexpr (NTMAX == 4) {
                // a last layer of at most four outputs in its 4x4x1 form, as in layers_narrow: every form of the
                // narrow-network kernels then ends the network on the same arithmetic
                if (l == nlayers - 1 && st_u(d.x4off) >= 0) {
                    a[0] = last_x4_sum(last_x4_partial<WLDS>(a, R, st_u(d.x4off), sWts, wall, lane, lq), R);
                    break;
                }
            }
            // n-tiles in groups of four independent accumulators; the size of the last group is
            // dispatched once per layer
#pragma unroll
            for (int gq = 0; gq < NTMAX / 4; gq++) {
                const int rem = R.NT - gq * 4;
                if (rem >= 4) layer_group<4, NTMAX, WLDS>(a, o + gq * 4, sWts, wall, R.woff / 4, R.boff, gq * 4, R.KG, lane, lq);
                else if (rem == 3) layer_group<3, NTMAX, WLDS>(a, o + gq * 4, sWts, wall, R.woff / 4, R.boff, gq * 4, R.KG, lane, lq);
                else if (rem == 2) layer_group<2, NTMAX, WLDS>(a, o + gq * 4, sWts, wall, R.woff / 4, R.boff, gq * 4, R.KG, lane, lq);
                else if (rem == 1) layer_group<1, NTMAX, WLDS>(a, o + gq * 4, sWts, wall, R.woff / 4, R.boff, gq * 4, R.KG, lane, lq);
            }
            // activation, chosen once per layer; the outputs become the next layer's operand
            auto next_in = [&](auto actf) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < NTMAX; u++)      // tiles past R.NT hold stale values no later stage reads
#pragma unroll
                    for (int r = 0; r < 4; r++) a[u][r] = actf(o[u][r]);
            };
            if (R.act == FORTIS_ACT_RELU) next_in([](float v) { return relu_acc(v); });
            else if (R.act == FORTIS_ACT_NONE) next_in([](float v) { return v; });
            else next_in([&](float v) { return apply_act(v, R.act, R.alpha); });
        }
        // ---- results out: the lane holds outputs n = 16 nt + 4 lq + r of its row ----------------------
        asm volatile("" ::: "memory");
        if (STENCIL) {
            gfloat* Yraw = st_g(P.Yraw);
            StCell cell;
#pragma unroll
            for (int s = 0; s < ST_SCAL_MAX; s++) cell.S[s] = in.sS[s];
            st_cell_program(sc, cell);
#pragma unroll
            for (int nt = 0; nt < (NTO < NTMAX ? NTO : NTMAX); nt++) {
                if (nt * 16 >= NO) break;
                float ov[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int n = nt * 16 + 4 * lq + r;
                    ov[r] = a[nt][r];
                    if (out_mul && n < NO) ov[r] = __fmul_rn(ov[r], out_mul[n]);
                    if (Yraw && valid && n < NO) Yraw[(size_t)row * NO + n] = ov[r];
                }
                st_chain_apply(sc, cell, ov);
                const long soff = st_off(sc.refs[0], in.si, in.sj, in.skk);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int n = nt * 16 + 4 * lq + r;
                    if (valid && n < NO) {
                        const StSlotT<float*> sl = sc.refs[n];
                        st_g(sl.p)[s_refs_uniform ? soff : st_off(sl, in.si, in.sj, in.skk)] = ov[r];
                    }
                }
            }
        } else if (NO < 4) {
            // Thin outputs (one to three per row): the tile's 16 rows are 16 NO consecutive floats of Y, held by the
            // lanes of the first quarter of the wave (lane = row, NO values each).  They change lanes so that lane t
            // holds float t of the run and the tile leaves in one store of whole, consecutive bytes; a lane storing its
            // row's values one by one left 12-byte pieces that reached memory as separate partial writes (2.4 times
            // the bytes of Y by the write counter).
            v4f v = a[0];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                if (out_mul && r < NO) v[r] = __fmul_rn(v[r], out_mul[r]);
                if (r >= NO - mask_tail) v[r] = v[r] > 0.f ? v[r] : 0.f;
            }
            const int src = NO == 3 ? (lane * 171) >> 9 : NO == 2 ? lane >> 1 : lane, rr = lane - src * NO;   // lane / NO
            float out = 0.f;
#pragma unroll
            for (int r = 0; r < 3; r++) {
                const float pr = __int_as_float(__builtin_amdgcn_ds_bpermute(src << 2, __float_as_int(v[r])));
                out = rr == r ? pr : out;
            }
            if (lane < 16 * NO && in.row0 + (unsigned)src < rows)
                __builtin_nontemporal_store(out, st_g(P.Y) + (size_t)in.row0 * NO + lane);
        } else {
            gfloat* yrow = st_g(P.Y) + (size_t)row * NO;
#pragma unroll
            for (int nt = 0; nt < NTMAX; nt++) {
                if (nt * 16 >= NO) break;
                const int n0 = nt * 16 + 4 * lq;
                v4f v = a[nt];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (out_mul && n0 + r < NO) v[r] = __fmul_rn(v[r], out_mul[n0 + r]);
                    if (n0 + r >= NO - mask_tail) v[r] = v[r] > 0.f ? v[r] : 0.f;
                }
                if (!valid) continue;
                if (yvec) { if (n0 < NO) __builtin_nontemporal_store(v, (gv4f*)(yrow + n0)); }
                else {
#pragma unroll
                    for (int r = 0; r < 4; r++) if (n0 + r < NO) __builtin_nontemporal_store(v[r], yrow + n0 + r);
                }
            }
        }
    };

    const unsigned long long ntile = ((unsigned long long)rows + 15) / 16;
    const unsigned long long stride = (unsigned long long)gridDim.x * 4;
    unsigned long long t = (unsigned long long)(STENCIL ? st_xcd_band_block() : blockIdx.x) * 4 + wave;
    TileIn cur, nxt;
    if (t < ntile) issue(cur, (unsigned)(t * 16));      // in flight while the weights are staged
    if (WLDS) {
        // weights into LDS: requests batched eight at a time so their latencies overlap
        const int n4 = wfloats / 4;
        for (int i0 = tid; i0 < n4; i0 += 8 * CH_THREADS) {
            v4f r[8];
#pragma unroll
            for (int u = 0; u < 8; u++) { const int i = i0 + u * CH_THREADS; r[u] = ((const gv4f*)wall)[i < n4 ? i : n4 - 1]; }
#pragma unroll
            for (int u = 0; u < 8; u++) { const int i = i0 + u * CH_THREADS; if (i < n4) ((v4f*)sWts)[i] = r[u]; }
        }
        __syncthreads();
    }
    for (; t < ntile; t += stride) {
        // Table values (slot pointers, strides, layer shapes) are re-read from LDS per tile: hoisted out of
        // this loop they would occupy more registers than the tile itself.
        asm volatile("" ::: "memory");
        const bool more = t + stride < ntile;
        if (PREFETCH) {
            if (more) issue(nxt, (unsigned)((t + stride) * 16));
            process(cur);
            if (more) cur = nxt;
        } else {
            process(cur);
            if (more) issue(cur, (unsigned)((t + stride) * 16));
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// The stencil form for the tables that lifted column physics usually gives (the ZB step is one): every gather
// slot has the same strides, the scatter's stores share theirs, gather and scatter visit the same cells, each
// table has at most two same-cell scalars and two per-cell instructions, the network is narrow (every width at
// most 64) with at most four outputs, and every array spans less than 4 GiB.  Same arithmetic and same
// wave-per-16-rows layout as chain_wave_kernel<true>, with what those conditions allow taken out of the tile
// loop: the lane's eight slot pointers stay in registers for the life of the (persistent) wave, scalar and store
// pointers and all strides are wave-uniform scalar registers, a cell is decoded once and its element offsets are
// 32-bit, and the expression interpreter looks at two scalars and two per-cell results instead of four and six.
// PF: the next tile's loads are issued before the current tile is processed (two sets of tile inputs in registers:
// four waves per SIMD).  Without it the kernel fits five waves per SIMD, which is what a launch of a little more than
// four tiles per SIMD wants: each tile then has a wave of its own and no wave runs a second tile after the others
// have finished.
template <bool WLDS, int SIG = 0, bool PF = true>
__global__ __launch_bounds__(CH_THREADS) __attribute__((amdgpu_waves_per_eu(PF ? 4 : 5, PF ? 4 : 5)))
void chain_stencil_fast_kernel(ChainParams params)
{
    constexpr int NS = 2, NC = 2;
    __shared__ ChainParams P;
    extern __shared__ float4 smem4[];
    params_to_lds(&P, CH_THREADS);
    const ChainDesc& d = P.d;
    const GatherArgs& g = P.g;
    const ScatterArgs& sc = P.sc;
    float* sWts = (float*)smem4;
    const int wfloats = st_u(d.wfloats), nlayers = st_u(d.nlayers);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K0 = st_u(d.L[0].K), NO = st_u(d.L[nlayers - 1].N);
    const unsigned rows = (unsigned)st_u((int)P.rows);
    const int lrow = lane & 15, lq = lane >> 4;
    const gfloat* wall = st_g(d.wall);
    const gfloat* in_div = st_g(d.in_div);
    const gfloat* out_mul = st_g(d.out_mul);
    // ---- hoisted table values -------------------------------------------------------------------------------
    const gfloat* gp[PF ? 8 : 1];                          // this lane's slots q = 16 (t / 4) + 4 lq + t % 4
#pragma unroll
    for (int t = 0; t < (PF ? 8 : 1); t++) gp[t] = st_g(g.refs[16 * (t >> 2) + 4 * lq + (t & 3)].p);   // (without prefetch: read per tile)
    const unsigned g_si = (unsigned)st_u(g.refs[0].si), g_sj = (unsigned)st_u(g.refs[0].sj), g_pl = (unsigned)st_u((int)g.refs[0].plane);
    const unsigned o_si = (unsigned)st_u(sc.refs[0].si), o_sj = (unsigned)st_u(sc.refs[0].sj), o_pl = (unsigned)st_u((int)sc.refs[0].plane);
    const bool o_as_g = g_si == o_si && g_sj == o_sj && g_pl == o_pl;
    const gfloat* gsp[NS];
    const gfloat* ssp[NS];
    unsigned s_si[NS], s_sj[NS], s_pl[NS];
    bool s_as_o[NS];
#pragma unroll
    for (int q = 0; q < NS; q++) {
        gsp[q] = st_uptr(st_g(g.scal[q].p));
        ssp[q] = st_uptr(st_g(sc.scal[q].p));
        s_si[q] = (unsigned)st_u(sc.scal[q].si); s_sj[q] = (unsigned)st_u(sc.scal[q].sj); s_pl[q] = (unsigned)st_u((int)sc.scal[q].plane);
        s_as_o[q] = s_si[q] == o_si && s_sj[q] == o_sj && s_pl[q] == o_pl;
    }
    gfloat* op[4];
#pragma unroll
    for (int n = 0; n < 4; n++) op[n] = st_uptr(st_g(sc.refs[n].p));       // entries past the outputs repeat store 0

    struct TileIn { float x[8], gS[NS], sS[NS]; unsigned soff, row0; };
    auto issue = [&](TileIn& in, unsigned row0) __attribute__((always_inline)) {
        in.row0 = row0;
        const unsigned row = row0 + lrow;
        int i, j, kk;
        st_row(g, row < rows ? row : 0, i, j, kk);
        const unsigned goff = (unsigned)i * g_si + (unsigned)j * g_sj + (unsigned)kk * g_pl;
        in.soff = o_as_g ? goff : (unsigned)i * o_si + (unsigned)j * o_sj + (unsigned)kk * o_pl;
#pragma unroll
        for (int t = 0; t < 8; t++) in.x[t] = (PF ? gp[PF ? t : 0] : st_g(g.refs[16 * (t >> 2) + 4 * lq + (t & 3)].p))[goff];
#pragma unroll
        for (int q = 0; q < NS; q++) in.gS[q] = gsp[q][goff];
#pragma unroll
        for (int q = 0; q < NS; q++) {
            const unsigned off = s_as_o[q] ? in.soff : (unsigned)i * s_si[q] + (unsigned)j * s_sj[q] + (unsigned)kk * s_pl[q];
            in.sS[q] = ssp[q][off];
        }
    };
    // the input divisors of the lane's eight slots: the same for every tile, loaded once (slots past the network's
    // inputs take slot 0's; their quotients are replaced by zero)
    // (the form without prefetch has no registers for them and reads them per tile)
    float dv[PF ? 8 : 1];
#pragma unroll
    for (int t = 0; t < (PF ? 8 : 1); t++) dv[t] = 1.f;
    if (PF && in_div) {
#pragma unroll
        for (int t = 0; t < (PF ? 8 : 1); t++) {
            const int q = 16 * (t >> 2) + 4 * lq + (t & 3);
            dv[t] = in_div[q < K0 ? q : 0];
        }
    }
    auto process = [&](TileIn& in) __attribute__((always_inline)) {
        const unsigned row = in.row0 + lrow;
        const bool valid = row < rows;
        v4f a[4];
        {
            StCellT<NS, NC> cell;
#pragma unroll
            for (int q = 0; q < NS; q++) cell.S[q] = in.gS[q];
            st_cell_program(g, cell);
            float tv[8];
#pragma unroll
            for (int t = 0; t < 8; t++) tv[t] = in.x[t];
            st_chain_apply(g, cell, tv);
#pragma unroll
            for (int t = 0; t < 8; t++) {
                const int q = 16 * (t >> 2) + 4 * lq + (t & 3);
                a[t >> 2][t & 3] = (valid && q < K0) ? tv[t] : 0.f;
            }
            if (in_div) {
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    const int q = 16 * (t >> 2) + 4 * lq + (t & 3);
                    const float dq = PF ? dv[PF ? t : 0] : (float)in_div[q < K0 ? q : 0];
                    a[t >> 2][t & 3] = (valid && q < K0) ? __fdiv_rn(tv[t], dq) : 0.f;
                }
            }
            a[2] = a[3] = (v4f)(0.f);
        }
        // the matrix phase outranks the other waves' vector phases at the issue port: a wave that has its operands
        // streams its MFMAs while the others decode and divide in the gaps (2.5 % on the 15.7 M-column grid)
        __builtin_amdgcn_s_setprio(3);
        layers_narrow<WLDS, true, SIG>(a, d, nlayers, sWts, wall, lane, lq);
        __builtin_amdgcn_s_setprio(0);
        asm volatile("" ::: "memory");
        // outputs 0..3 of the row are in the lanes of the first quarter
        float ov[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            ov[r] = a[0][r];
        }
        if (out_mul) {
#pragma unroll
            for (int r = 0; r < 4; r++) ov[r] = __fmul_rn(ov[r], st_c(d.out_mul)[r < NO ? r : 0]);      // (outputs past the last are not stored)
        }
        gfloat* Yraw = st_g(P.Yraw);
        if (Yraw && valid && lq == 0) {
#pragma unroll
            for (int r = 0; r < 4; r++) if (r < NO) Yraw[(size_t)row * NO + r] = ov[r];
        }
        StCellT<NS, NC> cell;
#pragma unroll
        for (int q = 0; q < NS; q++) cell.S[q] = in.sS[q];
        st_cell_program(sc, cell);
        st_chain_apply(sc, cell, ov);
        if (valid && lq == 0) {
#pragma unroll
            for (int r = 0; r < 4; r++) if (r < NO) op[r][in.soff] = ov[r];
        }
    };

    const unsigned long long ntile = ((unsigned long long)rows + 15) / 16;
    // Each XCD (workgroups b % 8 == x run on XCD x) walks its own contiguous eighth of the tiles, its workgroups
    // side by side: a cell's 3 x 3 neighbourhood is read through one L2, and the halo rows of one round are the
    // interior rows of that XCD's next.  Grids that are not a multiple of eight workgroups walk all tiles together.
    unsigned long long t, tend, stride;
    if (gridDim.x % 8 == 0) {
        const unsigned long long per = (ntile + 7) / 8, x = blockIdx.x % 8;
        t = x * per + (unsigned long long)(blockIdx.x / 8) * 4 + wave;
        tend = (x + 1) * per < ntile ? (x + 1) * per : ntile;
        stride = (unsigned long long)(gridDim.x / 8) * 4;
    } else {
        t = (unsigned long long)blockIdx.x * 4 + wave; tend = ntile; stride = (unsigned long long)gridDim.x * 4;
    }
    TileIn cur;
    if (t < tend) issue(cur, (unsigned)(t * 16));       // in flight while the weights are staged
    if (WLDS) {
        const int n4 = wfloats / 4;
        for (int i0 = tid; i0 < n4; i0 += 8 * CH_THREADS) {
            v4f r[8];
#pragma unroll
            for (int u = 0; u < 8; u++) { const int i = i0 + u * CH_THREADS; r[u] = ((const gv4f*)wall)[i < n4 ? i : n4 - 1]; }
#pragma unroll
            for (int u = 0; u < 8; u++) { const int i = i0 + u * CH_THREADS; if (i < n4) ((v4f*)sWts)[i] = r[u]; }
        }
        __syncthreads();
    }
    if constexpr (PF) {
        TileIn nxt;
        for (; t < tend; t += stride) {
            asm volatile("" ::: "memory");
            const bool more = t + stride < tend;
            if (more) issue(nxt, (unsigned)((t + stride) * 16));
            process(cur);
            if (more) cur = nxt;
        }
    } else {
        for (; t < tend; t += stride) {
            asm volatile("" ::: "memory");
            process(cur);
            if (t + stride < tend) issue(cur, (unsigned)((t + stride) * 16));
        }
    }
}

// ---------------------------------------------------------------------------------------------------
// Same conditions and same arithmetic as chain_stencil_fast_kernel, other division of labour: a wave takes 64
// rows at a time and LANE = ROW for everything that is per row -- decoding the cell, loading its NQ slots and
// scalars, the lifted expressions (the divisions), and at the end the scatter expressions and stores -- so each
// of those instructions serves 64 rows instead of 16.  The evaluated slot values go through a per-wave LDS tile
// ([64 rows][36 floats]: the pitch keeps the 16-byte reads of an m-tile conflict free) into the MFMA operand
// layout; the four 16-row m-tiles then run the layers in registers as before and leave their outputs in a
// second small LDS tile from which every lane picks up its own row.  The next 64 rows' loads are issued as soon
// as the slot registers are free, i.e. before the four m-tiles are multiplied.
#define CSR_PITCH 36
#define CSR_THREADS 512      // eight waves share one LDS copy of the weights: four waves per SIMD stay resident
template <bool WLDS, int NQ, int SIG = 0>
__global__ __launch_bounds__(CSR_THREADS) __attribute__((amdgpu_waves_per_eu(4, 4)))
void chain_stencil_rows_kernel(ChainParams params)
{
    constexpr int NS = 2, NC = 2;
    __shared__ ChainParams P;
    extern __shared__ float4 smem4[];
    params_to_lds(&P, CSR_THREADS);
    const ChainDesc& d = P.d;
    const GatherArgs& g = P.g;
    const ScatterArgs& sc = P.sc;
    const int wfloats = st_u(d.wfloats), nlayers = st_u(d.nlayers);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float* sWts = (float*)smem4;
    float* sOp = sWts + (WLDS ? wfloats : 0) + wave * (32 * CSR_PITCH + 64 * 4);   // this wave's operand tile (32 rows at a time)
    float* sOut = sOp + 32 * CSR_PITCH;                                            // and its output tile [64][4]
    const int K0 = st_u(d.L[0].K), NO = st_u(d.L[nlayers - 1].N);
    const unsigned rows = (unsigned)st_u((int)P.rows);
    const int lrow = lane & 15, lq = lane >> 4;
    const gfloat* wall = st_g(d.wall);
    const gfloat* in_div = st_g(d.in_div);
    const gfloat* in_rcp = st_g(d.in_rcp);
    const gfloat* out_mul = st_g(d.out_mul);
    const unsigned g_si = (unsigned)st_u(g.refs[0].si), g_sj = (unsigned)st_u(g.refs[0].sj), g_pl = (unsigned)st_u((int)g.refs[0].plane);
    const unsigned o_si = (unsigned)st_u(sc.refs[0].si), o_sj = (unsigned)st_u(sc.refs[0].sj), o_pl = (unsigned)st_u((int)sc.refs[0].plane);
    const bool o_as_g = g_si == o_si && g_sj == o_sj && g_pl == o_pl;

    struct RowIn { float x[NQ], gS[NS], sS[NS]; unsigned soff, row; };
    // ---- every global load of the 64 rows at row0; lane = row ----------------------------------------------
    auto issue = [&](RowIn& in, unsigned row0) __attribute__((always_inline)) {
        in.row = row0 + lane;
        int i, j, kk;
        st_row(g, in.row < rows ? in.row : 0, i, j, kk);
        const unsigned goff = (unsigned)i * g_si + (unsigned)j * g_sj + (unsigned)kk * g_pl;
        in.soff = o_as_g ? goff : (unsigned)i * o_si + (unsigned)j * o_sj + (unsigned)kk * o_pl;
        // every array spans less than 2^30 elements (checked by the launcher): a 32-bit byte offset beside a uniform
        // base pointer, so a load needs no per-lane 64-bit address
        const unsigned gbyte = goff << 2;
        typedef __attribute__((address_space(1))) char gchar;
#pragma unroll
        // (the slot pointers straight from the kernel arguments, by literal index: scalar loads, where the copy of the
        // arguments in LDS costs a vector read and two v_readfirstlane per pointer and tile)
        for (int q = 0; q < NQ; q++) in.x[q] = *(const gfloat*)((const gchar*)st_uptr(st_g(params.g.refs[q].p)) + gbyte);   // entries past the table's repeat slot 0
#pragma unroll
        for (int q = 0; q < NS; q++) in.gS[q] = *(const gfloat*)((const gchar*)st_uptr(st_g(params.g.scal[q].p)) + gbyte);
#pragma unroll
        for (int q = 0; q < NS; q++) {
            const unsigned ssi = (unsigned)st_u(params.sc.scal[q].si), ssj = (unsigned)st_u(params.sc.scal[q].sj), spl = (unsigned)st_u((int)params.sc.scal[q].plane);
            const unsigned off = (ssi == o_si && ssj == o_sj && spl == o_pl) ? in.soff : (unsigned)i * ssi + (unsigned)j * ssj + (unsigned)kk * spl;
            in.sS[q] = st_uptr(st_g(params.sc.scal[q].p))[off];
        }
    };

    // per-XCD contiguous ranges of 64-row groups (see chain_stencil_fast_kernel)
    const unsigned long long ngroup = ((unsigned long long)rows + 63) / 64;
    unsigned long long t, tend, stride;
    if (gridDim.x % 8 == 0) {
        const unsigned long long per = (ngroup + 7) / 8, x = blockIdx.x % 8;
        t = x * per + (unsigned long long)(blockIdx.x / 8) * 8 + wave;
        tend = (x + 1) * per < ngroup ? (x + 1) * per : ngroup;
        stride = (unsigned long long)(gridDim.x / 8) * 8;
    } else {
        t = (unsigned long long)blockIdx.x * 8 + wave; tend = ngroup; stride = (unsigned long long)gridDim.x * 8;
    }
    RowIn in;
    if (t < tend) issue(in, (unsigned)(t * 64));        // in flight while the weights are staged
    if (WLDS) {
        const int n4 = wfloats / 4;
        for (int i0 = tid; i0 < n4; i0 += 4 * CSR_THREADS) {
            v4f r[4];
#pragma unroll
            for (int u = 0; u < 4; u++) { const int i = i0 + u * CSR_THREADS; r[u] = ((const gv4f*)wall)[i < n4 ? i : n4 - 1]; }
#pragma unroll
            for (int u = 0; u < 4; u++) { const int i = i0 + u * CSR_THREADS; if (i < n4) ((v4f*)sWts)[i] = r[u]; }
        }
        __syncthreads();
    }
    for (; t < tend; t += stride) {
        asm volatile("" ::: "memory");
        // ---- lane = row: expressions, then the row's operands into the wave's LDS tile -----------------------
        const unsigned row = in.row, soff = in.soff;
        const bool valid = row < rows;
        float sS[NS];
#pragma unroll
        for (int q = 0; q < NS; q++) sS[q] = in.sS[q];
        {
            StCellT<NS, NC> cell;
#pragma unroll
            for (int q = 0; q < NS; q++) cell.S[q] = in.gS[q];
            st_cell_program(g, cell);
            st_chain_apply<NQ, true>(g, cell, in.x);
            // (slots past the network's inputs, which hold a copy of slot 0, are zeroed in the LDS tile below; rows past
            // the end hold the first cell's values and their results are never stored: no per-slot select here)
            // The divisors are the same for every row: scalar loads, all of them out before the first division.  Slots
            // past the network's inputs (zeroed below) divide by slot 0's divisor rather than sit behind a branch each.
            if (in_rcp && st_div_wave_in_range(in.x, 1.f)) {
                // divisors in range (checked when the step was built), numerators too: the short form of the division
                const cfloat* cd = st_c(d.in_div);
                const cfloat* cr = st_c(d.in_rcp);
#pragma unroll
                for (int q = 0; q < NQ; q++) { const int qc = q < K0 ? q : 0; in.x[q] = st_div_inrange(in.x[q], cd[qc], cr[qc]); }
            } else if (in_div) {
                const cfloat* cd = st_c(d.in_div);
#pragma unroll
                for (int q = 0; q < NQ; q++) { const int qc = q < K0 ? q : 0; in.x[q] = __fdiv_rn(in.x[q], cd[qc]); }
            }
        }
        // ---- two halves of 32 rows: their operands through the LDS tile, two m-tiles through the layers ------
        __builtin_amdgcn_s_setprio(3);
#pragma unroll 1
        for (int half = 0; half < 2; half++) {
            if ((lane >> 5) == half) {
                v4f* dst = (v4f*)(sOp + (lane & 31) * CSR_PITCH);
#pragma unroll
                for (int q4 = 0; q4 < 8; q4++) {
                    v4f v;
#pragma unroll
                    for (int r = 0; r < 4; r++) v[r] = 4 * q4 + r < NQ ? in.x[4 * q4 + r] : 0.f;
                    dst[q4] = v;
                }
                for (int c = K0; c < NQ; c++) ((float*)dst)[c] = 0.f;
            }
            asm volatile("" ::: "memory");
            // the slot registers are free once the second half is written: the next 64 rows' loads go out here
            if (half == 1 && t + stride < tend) issue(in, (unsigned)((t + stride) * 64));
#pragma unroll 1
            for (int T = 0; T < 2; T++) {
                v4f a[4];
                const v4f* src = (const v4f*)(sOp + (16 * T + lrow) * CSR_PITCH) + lq;
                a[0] = src[0]; a[1] = src[4];      // (a[2], a[3]: a layer reads as many k groups as the one before it wrote n-tiles)
                if (layers_narrow<WLDS, false, SIG>(a, d, nlayers, sWts, wall, lane, lq)) {
                    // the quarters' partial sums of the last layer meet in the tile's own operand rows (consumed above)
                    v4f* tmp = (v4f*)(sOp + 16 * T * CSR_PITCH);
                    tmp[lq * 16 + lrow] = a[0];
                    asm volatile("" ::: "memory");
                    if (lq == 0) {
                        const LayerRegs R = layer_regs(d, nlayers - 1);
                        v4f o = (tmp[lrow] + tmp[32 + lrow]) + (tmp[16 + lrow] + tmp[48 + lrow]);
#pragma unroll
                        for (int r = 0; r < 4; r++) o[r] = apply_act(o[r], R.act, R.alpha);
                        ((v4f*)sOut)[32 * half + 16 * T + lrow] = o;
                    }
                } else if (lq == 0) ((v4f*)sOut)[32 * half + 16 * T + lrow] = a[0];
            }
            asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_s_setprio(0);
        asm volatile("" ::: "memory");
        // ---- lane = row again: the row's outputs, scatter expressions, stores --------------------------------
        const v4f o4 = ((const v4f*)sOut)[lane];
        float ov[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            ov[r] = o4[r];
        }
        if (out_mul) {
#pragma unroll
            for (int r = 0; r < 4; r++) ov[r] = __fmul_rn(ov[r], st_c(d.out_mul)[r < NO ? r : 0]);      // (outputs past the last are not stored)
        }
        gfloat* Yraw = st_g(P.Yraw);
        if (Yraw && valid) {
#pragma unroll
            for (int r = 0; r < 4; r++) if (r < NO) Yraw[(size_t)row * NO + r] = ov[r];
        }
        StCellT<NS, NC> cell;
#pragma unroll
        for (int q = 0; q < NS; q++) cell.S[q] = sS[q];
        st_cell_program(sc, cell);
        st_chain_apply(sc, cell, ov);
        if (valid) {
#pragma unroll
            for (int r = 0; r < 4; r++) if (r < NO) st_uptr(st_g(params.sc.refs[r].p))[soff] = ov[r];
        }
    }
}

__global__ void chain_rcp_kernel(const float* __restrict__ div, float* __restrict__ rcp, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) rcp[i] = st_div_rcp(div[i]);
}
void fortis_chain_fill_rcp(const float* div, float* rcp, int n, hipStream_t s)
{
    hipLaunchKernelGGL(chain_rcp_kernel, dim3((unsigned)cdiv(n, 64)), dim3(64), 0, s, div, rcp, n);
    HIP_OK(hipGetLastError());
}

// ---- host side ---------------------------------------------------------------------------------------
// Packs all layers into one device blob: for each layer the weights W[N][K] in B-operand order
// [Np/16][Kp/16][64 lanes][4] (lane = 16*q + j holds W[nt*16 + j][kg*16 + 4q + s], s = 0..3), then the
// zero-padded bias [Np].  Fills d->L[].{K,N,Kp,Np,woff,boff}, d->wall, d->wfloats, d->ld.
int fortis_chain_build(ChainDesc* d, int nlayers, const float* const* W, const float* const* b, const int* K,
                       const int* N, float** blob_out)
{
    if (nlayers < 1 || nlayers > FORTIS_CHAIN_MAX_LAYERS) return -1;
    long total = 0;
    int wmax = 0;
    for (int l = 0; l < nlayers; l++) {
        if (K[l] < 1 || N[l] < 1 || K[l] > FORTIS_CHAIN_MAX_WIDTH || N[l] > FORTIS_CHAIN_MAX_WIDTH) return -1;
        if (l && K[l] != N[l - 1]) return -1;
        ChainLayer& L = d->L[l];
        L.K = K[l]; L.N = N[l];
        L.Kp = (int)cdiv(K[l], 16) * 16; L.Np = (int)cdiv(N[l], 16) * 16;
        L.woff = (int)total; total += (long)L.Kp * L.Np;
        L.boff = (int)total; total += L.Np;
        if (L.Kp > wmax) wmax = L.Kp;
        if (L.Np > wmax) wmax = L.Np;
    }
    total = cdiv(total, 4) * 4;
    // A last layer of at most four outputs a second time, for v_mfma_f32_4x4x1: [q][n][k group][4] holds
    // W[n][16 group + 4 q + s], the 16 features a lane of quarter q carries per k group.
    const ChainLayer& LL = d->L[nlayers - 1];
    d->x4off = -1;
    if (LL.N <= 4 && LL.Kp <= 64) { d->x4off = (int)total; total += 16L * LL.Kp / 16 * 4; }
    float* h = (float*)calloc(total, sizeof(float));
    if (d->x4off >= 0) {
        const int KG = LL.Kp / 16;
        for (int q = 0; q < 4; q++)
            for (int n = 0; n < LL.N; n++)
                for (int u = 0; u < KG; u++)
                    for (int r = 0; r < 4; r++) {
                        const int k = 16 * u + 4 * q + r;
                        if (k < LL.K) h[d->x4off + ((q * 4 + n) * KG + u) * 4 + r] = W[nlayers - 1][(long)n * LL.K + k];
                    }
    }
    for (int l = 0; l < nlayers; l++) {
        const ChainLayer& L = d->L[l];
        const int KG = L.Kp / 16, NT = L.Np / 16;
        for (int nt = 0; nt < NT; nt++)
            for (int kg = 0; kg < KG; kg++)
                for (int lane = 0; lane < 64; lane++)
                    for (int s = 0; s < 4; s++) {
                        const long n = nt * 16 + (lane & 15), k = kg * 16 + 4 * (lane >> 4) + s;
                        if (n < L.N && k < L.K) h[L.woff + (((long)nt * KG + kg) * 64 + lane) * 4 + s] = W[l][n * L.K + k];
                    }
        if (b && b[l]) memcpy(h + L.boff, b[l], L.N * sizeof(float));
    }
    float* dev = nullptr;
    if (fortis_dev_malloc((void**)&dev, total * sizeof(float), "MLP chain weights") != 0) { free(h); return -1; }
    if (hipMemcpy(dev, h, total * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        fprintf(stderr, "fortis: copying the MLP chain weights to the device failed\n");
        fortis_dev_free(dev);
        free(h);
        return -1;
    }
    free(h);
    d->nlayers = nlayers;
    d->wall = dev;
    d->wfloats = (int)total;
    d->ld = wmax + 4;   // +4 floats: the 16 rows of an m-tile start 4 banks apart, 16-byte reads stay aligned
    *blob_out = dev;
    return 0;
}

static bool chain_check(const ChainDesc& d)
{
    if (d.nlayers < 1 || d.nlayers > FORTIS_CHAIN_MAX_LAYERS || !d.wall) return false;
    int wmax = 0;
    for (int l = 0; l < d.nlayers; l++) {
        if (d.L[l].K > FORTIS_CHAIN_MAX_WIDTH || d.L[l].N > FORTIS_CHAIN_MAX_WIDTH) return false;
        if (l && d.L[l].K != d.L[l - 1].N) return false;
        if (d.L[l].Kp % 16 || d.L[l].Np % 16 || d.L[l].Kp < d.L[l].K || d.L[l].Np < d.L[l].N) return false;
        if (d.L[l].Kp > wmax) wmax = d.L[l].Kp;
        if (d.L[l].Np > wmax) wmax = d.L[l].Np;
    }
    return d.ld >= wmax + 4 && d.ld % 4 == 0 && d.wfloats % 4 == 0;
}

static int num_cus()
{
    static int n = 0;
    if (!n) {
        hipDeviceProp_t prop;
        n = hipGetDeviceProperties(&prop, 0) == hipSuccess ? prop.multiProcessorCount : 256;
    }
    return n;
}

static void fill_params(ChainParams* P, const ChainDesc& d, const float* X, float* Y, long rows, float* Yraw)
{
    memset(P, 0, sizeof *P);
    P->d = d; P->rows = (unsigned)rows; P->X = X; P->Y = Y; P->Yraw = Yraw;
}

template <int ROWS, bool WLDS>
static void launch_variant(ChainParams& P, hipStream_t s)
{
    const ChainDesc& d = P.d;
    const size_t shmem = ((size_t)(WLDS ? d.wfloats : 0) + (size_t)2 * ROWS * d.ld) * sizeof(float);
    static size_t attr = 0;
    if (shmem > attr) {
        HIP_OK(hipFuncSetAttribute((const void*)chain_kernel<ROWS, WLDS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        attr = shmem;
    }
    P.ntiles = (unsigned)cdiv(P.rows, ROWS);
    // persistent grid: as many workgroups as the chip holds at once (LDS-limited), never more than tiles
    long per_cu = (160L * 1024) / (long)(shmem + sizeof(ChainParams) + 512);
    per_cu = per_cu < 1 ? 1 : per_cu > 4 ? 4 : per_cu;
    long grid = (long)num_cus() * per_cu;
    if (grid > P.ntiles) grid = P.ntiles;
    hipLaunchKernelGGL((chain_kernel<ROWS, WLDS>), dim3((unsigned)grid), dim3(CH_THREADS), shmem, s, P);
    HIP_OK(hipGetLastError());
}

static bool chain_ok(const ChainDesc& d, long rows)
{
    if (!chain_check(d)) { fprintf(stderr, "fortis: MLP chain descriptor rejected by the kernel launcher\n"); return false; }
    if (rows >= 4294967295L - 1024) { fprintf(stderr, "fortis: too many rows for one MLP chain launch\n"); return false; }
    return rows > 0;
}
// weights live in LDS when they leave room for at least two workgroups per CU
static bool chain_wlds(const ChainDesc& d) { return ((size_t)d.wfloats + 2 * 64 * d.ld) * sizeof(float) <= 72 * 1024; }

template <bool ST, bool WLDS, int NTMAX, int SIG_ = 0>
static void launch_wave_variant(ChainParams& P, hipStream_t s)
{
    constexpr int SIG = SIG_;
    const ChainDesc& d = P.d;
    const size_t shmem = (size_t)(WLDS ? d.wfloats : 0) * sizeof(float);
    static size_t attr = 0;
    static long slots = 0;
    if (shmem > attr || !slots) {
        HIP_OK(hipFuncSetAttribute((const void*)chain_wave_kernel<ST, WLDS, NTMAX, SIG>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        attr = shmem;
        int occ = 0;
        HIP_OK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void*)chain_wave_kernel<ST, WLDS, NTMAX, SIG>, CH_THREADS, shmem));
        slots = (long)(occ < 1 ? 1 : occ) * num_cus();
    }
    // persistent grid: as many workgroups as the chip holds at once, never more than 64-row groups
    long grid = cdiv(P.rows, 64);
    if (grid > slots) grid = slots;
    hipLaunchKernelGGL((chain_wave_kernel<ST, WLDS, NTMAX, SIG>), dim3((unsigned)grid), dim3(CH_THREADS), shmem, s, P);
    HIP_OK(hipGetLastError());
}
static int chain_ntmax(const ChainDesc& d)
{
    int nt = d.L[0].Kp / 16;
    for (int l = 0; l < d.nlayers; l++) if (d.L[l].Np / 16 > nt) nt = d.L[l].Np / 16;
    return nt;
}
// weights go to LDS in the wave kernel when three workgroups still fit on a CU
static bool chain_wave_wlds(const ChainDesc& d)
{
    static int force = -2;
    if (force == -2) { const char* e = getenv("FORTIS_CHAIN_WLDS"); force = e ? atoi(e) : -1; }
    if (force >= 0) return force != 0;
    return (size_t)d.wfloats * sizeof(float) + sizeof(ChainParams) <= 52 * 1024;
}

// The shapes layers_narrow has straight-line code for (its SIG), 0 for any other network.
static int chain_signature(const ChainDesc& d)
{
    static const int off = getenv("FORTIS_CHAIN_SIGNATURE") != nullptr && atoi(getenv("FORTIS_CHAIN_SIGNATURE")) == 0;
    if (off || d.x4off < 0) return 0;
    auto hidden = [&](int l, int Kp, int Np) { return d.L[l].Kp == Kp && d.L[l].Np == Np && d.L[l].act == FORTIS_ACT_RELU; };
    if (d.nlayers == 3 && hidden(0, 32, 64) && hidden(1, 64, 64) && d.L[2].Kp == 64) return 1;
    if (d.nlayers == 2 && hidden(0, 32, 32) && d.L[1].Kp == 32) return 2;
    return 0;
}

template <bool ST>
static void launch_wave(ChainParams& P, hipStream_t s)
{
    const bool wlds = chain_wave_wlds(P.d);
    if (chain_ntmax(P.d) <= 4) {
        if constexpr (!ST) {
            const int sig = wlds ? chain_signature(P.d) : 0;
            if (sig == 1) { launch_wave_variant<ST, true, 4, 1>(P, s); return; }
            if (sig == 2) { launch_wave_variant<ST, true, 4, 2>(P, s); return; }
        }
        if (wlds) launch_wave_variant<ST, true, 4>(P, s);
        else launch_wave_variant<ST, false, 4>(P, s);
    } else {
        if (wlds) launch_wave_variant<ST, true, 16>(P, s);
        else launch_wave_variant<ST, false, 16>(P, s);
    }
}

// form_rows: the row count that picks the kernel form (0: rows).  A caller that runs a batch in row bands passes the
// whole batch's, so that every band is computed by the kernel -- and in the summation order -- of the whole batch.
void fortis_launch_chain(const ChainDesc& d, const float* X, float* Y, long rows, hipStream_t s, long form_rows)
{
    if (!chain_ok(d, rows)) return;
    ChainParams P;
    fill_params(&P, d, X, Y, rows, nullptr);
    if (form_rows <= 0) form_rows = rows;
    // many rows of a narrow input: the wave-independent kernel
    if (form_rows >= 64L * num_cus()) { launch_wave<false>(P, s); return; }
    const bool wlds = chain_wlds(d);
    // few rows: 16-row tiles spread the work over more CUs (the four waves then split the n-tiles)
    if (form_rows < 64L * num_cus()) {
        if (wlds) launch_variant<16, true>(P, s);
        else launch_variant<16, false>(P, s);
    } else {
        if (wlds) launch_variant<64, true>(P, s);
        else launch_variant<64, false>(P, s);
    }
}

// Whether the tables and the network meet the conditions of chain_stencil_fast_kernel (see there).
static bool stencil_fast_ok(const ChainParams& P, const StencilDev& g, const StencilDev& sc)
{
    static int off = -1;
    if (off < 0) off = getenv("FORTIS_STENCIL_GENERIC") != nullptr;
    if (off || chain_ntmax(P.d) > 4 || P.d.L[P.d.nlayers - 1].N > 4 || P.d.mask_tail) return false;
    if (!P.g.uniform || !P.sc.refs_uniform) return false;
    if (g.nscal > 2 || sc.nscal > 2 || g.ncell > 2 || sc.ncell > 2) return false;
    if (P.g.count != P.sc.count || P.g.ni != P.sc.ni || P.g.ilo != P.sc.ilo || P.g.jlo != P.sc.jlo || P.g.sx != P.sc.sx || P.g.cells != P.sc.cells) return false;
    // 32-bit element offsets: every array the kernel indexes spans less than 2^30 elements, strides are not negative
    auto fits = [](const StencilDev& t) {
        for (int a = 0; a < t.narrays; a++) if (t.plane[a] * (long)t.nk >= (1L << 30)) return false;
        for (int r = 0; r < t.nrefs + t.nscal; r++) {
            const fortis_ref_t& f = r < t.nrefs ? t.refs[r] : t.scal[r - t.nrefs];
            if (f.si < 0 || f.sj < 0) return false;
        }
        return true;
    };
    return fits(g) && fits(sc);
}

template <bool WLDS, int SIG = 0, bool PF = true>
static long stencil_fast_slots(size_t shmem)
{
    static size_t attr = 0;
    static long slots = 0;
    if (shmem > attr || !slots) {
        HIP_OK(hipFuncSetAttribute((const void*)chain_stencil_fast_kernel<WLDS, SIG, PF>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        attr = shmem;
        int occ = 0;
        HIP_OK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void*)chain_stencil_fast_kernel<WLDS, SIG, PF>, CH_THREADS, shmem));
        slots = (long)(occ < 1 ? 1 : occ) * num_cus();
    }
    return slots;
}
template <bool WLDS, int SIG = 0>
static void launch_stencil_fast(ChainParams& P, hipStream_t s)
{
    const size_t shmem = (size_t)(WLDS ? P.d.wfloats : 0) * sizeof(float);
    const long slots = stencil_fast_slots<WLDS, SIG, true>(shmem);
    long grid = cdiv(P.rows, 64);
    static const int pf_only = getenv("FORTIS_STENCIL_PF") != nullptr;
    if (WLDS && grid > slots && !pf_only) {
        // more tiles than the prefetching form has waves: if the form with five waves per SIMD holds them all at
        // once, every tile gets a wave of its own (the grid rounded up to whole rounds of the eight XCDs)
        const long slots5 = stencil_fast_slots<WLDS, SIG, false>(shmem);
        if (grid <= slots5) {
            grid = (grid + 7) / 8 * 8;
            hipLaunchKernelGGL((chain_stencil_fast_kernel<WLDS, SIG, false>), dim3((unsigned)(grid < slots5 ? grid : slots5)), dim3(CH_THREADS), shmem, s, P);
            HIP_OK(hipGetLastError());
            return;
        }
    }
    if (grid > slots) grid = slots;
    hipLaunchKernelGGL((chain_stencil_fast_kernel<WLDS, SIG>), dim3((unsigned)grid), dim3(CH_THREADS), shmem, s, P);
    HIP_OK(hipGetLastError());
}

template <bool WLDS, int NQ, int SIG = 0>
static void launch_stencil_rows(ChainParams& P, hipStream_t s)
{
    const size_t shmem = ((size_t)(WLDS ? P.d.wfloats : 0) + (CSR_THREADS / 64) * (32 * CSR_PITCH + 64 * 4)) * sizeof(float);
    static size_t attr = 0;
    static long slots = 0;
    if (shmem > attr || !slots) {
        HIP_OK(hipFuncSetAttribute((const void*)chain_stencil_rows_kernel<WLDS, NQ, SIG>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        attr = shmem;
        int occ = 0;
        HIP_OK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void*)chain_stencil_rows_kernel<WLDS, NQ, SIG>, CSR_THREADS, shmem));
        slots = (long)(occ < 1 ? 1 : occ) * num_cus();
    }
    long grid = cdiv(P.rows, CSR_THREADS);
    if (grid > slots) grid = slots;
    hipLaunchKernelGGL((chain_stencil_rows_kernel<WLDS, NQ, SIG>), dim3((unsigned)grid), dim3(CSR_THREADS), shmem, s, P);
    HIP_OK(hipGetLastError());
}

void fortis_launch_chain_stencil(const ChainDesc& d, const StencilDev& g, const StencilDev& sc, long rows,
                                 const float* const* dG, float* const* dS, float* dY, hipStream_t s)
{
    if (!chain_ok(d, rows)) return;
    ChainParams P;
    fill_params(&P, d, nullptr, nullptr, rows, dY);
    st_make_args<const float*>(g, g.cells, dG, &P.g);
    st_make_args<float*>(sc, sc.cells, dS, &P.sc);
    if (stencil_fast_ok(P, g, sc)) {
        // lane-per-row form from three of its rounds of the chip on (64 rows x 16 waves x CUs); below that the
        // wave-per-16-rows form spreads the rows over more waves and finishes a partial round sooner.
        // FORTIS_STENCIL_FORM=16|64 forces one of them.
        static int form = -1;
        if (form < 0) { const char* e = getenv("FORTIS_STENCIL_FORM"); form = e ? atoi(e) : 0; }
        const bool v1 = form == 16 || (form != 64 && rows < 3L * 64 * 16 * num_cus());
        const bool wlds = chain_wave_wlds(P.d);
        const int k0 = P.d.L[0].K;
        // the two ZB networks (27 -> 64 -> 64 -> 3 and the reference's 27 -> 20 -> 3) as straight-line code
        const int sig = wlds && k0 > 16 && k0 <= 28 ? chain_signature(P.d) : 0;
        if (v1) {
            // (the reference's small network measured 5 % slower as straight-line code in this form: 12.9 against 12.3 us)
            if (sig == 1) launch_stencil_fast<true, 1>(P, s);
            else if (wlds) launch_stencil_fast<true>(P, s);
            else launch_stencil_fast<false>(P, s);
            return;
        }
        if (sig == 1) { launch_stencil_rows<true, 28, 1>(P, s); return; }
        if (sig == 2) { launch_stencil_rows<true, 28, 2>(P, s); return; }
        if (wlds) { if (k0 <= 16) launch_stencil_rows<true, 16>(P, s); else if (k0 <= 28) launch_stencil_rows<true, 28>(P, s); else launch_stencil_rows<true, 32>(P, s); }
        else { if (k0 <= 16) launch_stencil_rows<false, 16>(P, s); else if (k0 <= 28) launch_stencil_rows<false, 28>(P, s); else launch_stencil_rows<false, 32>(P, s); }
        return;
    }
    launch_wave<true>(P, s);
}
