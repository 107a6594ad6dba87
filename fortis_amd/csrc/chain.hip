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
            xr[t] = (idx < ROWS * K0 && idx < lim) ? X[base + idx] : 0.f;
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
            Y[base + idx] = v;
        }
        // the next land() writes buf0 while slower threads may still read `cur` above
        __syncthreads();
    }
}

// One m-tile (16 rows at ap) times NT n-tiles starting at nt0, NT known at compile time: no branch
// inside the k loop, MFMAs interleaved over the NT independent accumulators.
template <int NT, bool WLDS>
__device__ __forceinline__ void mma_ntiles(const float* ap, const float* sWts, const gfloat* wall, int woff4, int nt0,
                                           int KG, int lane, v4f* acc)
{
#pragma unroll
    for (int u = 0; u < NT; u++) acc[u] = (v4f){ 0.f, 0.f, 0.f, 0.f };
#pragma unroll 2
    for (int kg = 0; kg < KG; kg++) {
        const v4f a = *(const v4f*)(ap + kg * 16);
        v4f b[NT];
#pragma unroll
        for (int u = 0; u < NT; u++) {
            const int off = woff4 + ((nt0 + u) * KG + kg) * 64 + lane;
            if (WLDS) b[u] = ((const v4f*)sWts)[off]; else b[u] = ((const gv4f*)wall)[off];
        }
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, b[u].x, acc[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, b[u].y, acc[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, b[u].z, acc[u], 0, 0, 0);
#pragma unroll
        for (int u = 0; u < NT; u++) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, b[u].w, acc[u], 0, 0, 0);
    }
}

// ---------------------------------------------------------------------------------------------------
// Wave-independent variant: ONE WAVE owns 16 rows from the gather (or the X load) to the scatter (or
// the Y store).  Every layer is computed in place in the wave's private 16 x ld LDS tile (all n-tiles
// are accumulated in registers before anything is written back), so no workgroup barrier separates
// the layers and the waves of a CU drift apart: while one waits for its slot loads another runs its
// MFMAs.  The four waves of a workgroup only share the LDS copies of the parameter block and of the
// weights.  All global loads a wave needs (slot values, gather scalars, scatter scalars) are issued
// up front, before the weights are staged.
template <bool STENCIL, bool WLDS, int NTMAX>
__global__ __launch_bounds__(CH_THREADS) __attribute__((amdgpu_waves_per_eu(1, 4)))
void chain_wave_kernel(ChainParams params)
{
    constexpr int QMAX = FORTIS_MAX_REFS / 4;
    constexpr int XR = 16;                                      // plain: 16 rows x K0 <= 64 floats = 16 per lane
    __shared__ ChainParams P;
    extern __shared__ float4 smem4[];
    params_to_lds(&P, CH_THREADS);
    const ChainDesc& d = P.d;
    const GatherArgs& g = P.g;
    const ScatterArgs& sc = P.sc;
    float* sWts = (float*)smem4;
    const int wfloats = st_u(d.wfloats), ld = st_u(d.ld), nlayers = st_u(d.nlayers);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float* act = sWts + (WLDS ? wfloats : 0) + wave * 16 * ld;
    const int K0 = st_u(d.L[0].K), K0p = st_u(d.L[0].Kp);
    const int NO = st_u(d.L[nlayers - 1].N), mask_tail = st_u(d.mask_tail);
    const unsigned rows = P.rows;
    const int lrow = lane & 15, lq = lane >> 4;
    const gfloat* wall = st_g(d.wall);
    const gfloat* in_div = st_g(d.in_div);
    const gfloat* out_mul = st_g(d.out_mul);

    const bool g_uniform = STENCIL && st_u(g.uniform) != 0;
    // gather and scatter usually visit the same cells in the same order: decode a row once
    const bool same_cells = STENCIL && st_u((int)(g.count == sc.count && g.ni == sc.ni && g.ilo == sc.ilo && g.jlo == sc.jlo &&
                                                  g.sx == sc.sx && g.cells == sc.cells)) != 0;
    // Everything a tile reads from global memory, as registers: slot values, gather scalars, scatter
    // scalars (stencil form) or the 16 x K0 input block (plain form).
    struct TileIn {
        float tv[QMAX], gS[ST_SCAL_MAX], sS[ST_SCAL_MAX], xr[XR];
        int si, sj, skk;
        unsigned row0;
    };
    // ---- issues every global load of the tile at row0 ---------------------------------------------------
    auto issue = [&](TileIn& in, unsigned row0) __attribute__((always_inline)) {
        in.row0 = row0;
        in.si = in.sj = in.skk = 0;
        if (STENCIL) {
            const unsigned row = row0 + lrow;
            const unsigned rc = row < rows ? row : 0;
            int i, j, kk;
            st_row(g, rc, i, j, kk);
            if (same_cells) { in.si = i; in.sj = j; in.skk = kk; }
            else st_row(sc, rc, in.si, in.sj, in.skk);
            if (g_uniform) {
                // one element offset per cell; a slot is then its pointer plus that offset
                const long off = st_off(g.refs[0], i, j, kk);
#pragma unroll
                for (int t = 0; t < QMAX; t++) {
                    const int q = lq + 4 * t;
                    in.tv[t] = st_g(g.refs[q < K0 ? q : 0].p)[off];
                }
#pragma unroll
                for (int s = 0; s < ST_SCAL_MAX; s++) in.gS[s] = st_g(g.scal[s < g.nscal ? s : 0].p)[off];
            } else {
#pragma unroll
                for (int t = 0; t < QMAX; t++) {
                    const int q = lq + 4 * t;
                    const StSlotT<const float*> sl = g.refs[q < K0 ? q : 0];
                    in.tv[t] = st_g(sl.p)[st_off(sl, i, j, kk)];
                }
#pragma unroll
                for (int s = 0; s < ST_SCAL_MAX; s++) {
                    const StSlotT<const float*> sl = g.scal[s < g.nscal ? s : 0];
                    in.gS[s] = st_g(sl.p)[st_off(sl, i, j, kk)];
                }
            }
#pragma unroll
            for (int s = 0; s < ST_SCAL_MAX; s++) {
                const StSlotT<float*> sl = sc.scal[s < sc.nscal ? s : 0];
                in.sS[s] = st_g(sl.p)[st_off(sl, in.si, in.sj, in.skk)];
            }
        } else {
            const gfloat* X = st_g(P.X);
            const long base = (long)row0 * K0;
            const long lim = (long)rows * K0 - base;
#pragma unroll
            for (int t = 0; t < XR; t++) {
                const int idx = lane + t * 64;
                in.xr[t] = (idx < 16 * K0 && idx < lim) ? X[base + idx] : 0.f;
            }
        }
    };
    // ---- one tile: input into the wave's LDS tile, the layers in place, results out --------------------
    auto process = [&](TileIn& in) __attribute__((always_inline)) {
        const unsigned row0 = in.row0, row = row0 + lrow;
        const bool valid = row < rows;
        if (STENCIL) {
            StCell cell;
#pragma unroll
            for (int s = 0; s < ST_SCAL_MAX; s++) cell.S[s] = in.gS[s];
            st_cell_program(g, cell);
            st_chain_apply(g, cell, in.tv);
#pragma unroll
            for (int t = 0; t < QMAX; t++) {
                const int q = lq + 4 * t;
                if (q < K0) {
                    float v = valid ? in.tv[t] : 0.f;
                    if (in_div) v = __fdiv_rn(v, in_div[q]);
                    act[lrow * ld + q] = v;
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < XR; t++) {
                const int idx = lane + t * 64;
                if (idx < 16 * K0) {
                    const int r = idx / K0, c = idx - r * K0;
                    float v = in.xr[t];
                    if (in_div) v = __fdiv_rn(v, in_div[c]);
                    act[r * ld + c] = v;
                }
            }
        }
        for (int idx = lane; idx < 16 * (K0p - K0); idx += 64) {
            const int r = idx / (K0p - K0), c = idx - r * (K0p - K0);
            act[r * ld + K0 + c] = 0.f;
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const float* ap = act + lrow * ld + 4 * lq;
        for (int l = 0; l < nlayers; l++) {
            const LayerRegs R = layer_regs(d, l);
            v4f acc[NTMAX];
#pragma unroll
            for (int u = 0; u < NTMAX; u++) acc[u] = (v4f){ 0.f, 0.f, 0.f, 0.f };
            // n-tiles in groups of four; the size of the last group is dispatched once per layer so that
            // the k loop itself is branch-free
#pragma unroll
            for (int gq = 0; gq < NTMAX / 4; gq++) {
                const int rem = R.NT - gq * 4;
                if (rem >= 4) mma_ntiles<4, WLDS>(ap, sWts, wall, R.woff / 4, gq * 4, R.KG, lane, acc + gq * 4);
                else if (rem == 3) mma_ntiles<3, WLDS>(ap, sWts, wall, R.woff / 4, gq * 4, R.KG, lane, acc + gq * 4);
                else if (rem == 2) mma_ntiles<2, WLDS>(ap, sWts, wall, R.woff / 4, gq * 4, R.KG, lane, acc + gq * 4);
                else if (rem == 1) mma_ntiles<1, WLDS>(ap, sWts, wall, R.woff / 4, gq * 4, R.KG, lane, acc + gq * 4);
            }
            // every read of the tile is done (the accumulators depend on them): overwrite it
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            auto write_back = [&](auto actf) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < NTMAX; u++)
                    if (u < R.NT) {
                        const int col = u * 16 + lrow;
                        const float bv = WLDS ? sWts[R.boff + col] : wall[R.boff + col];
#pragma unroll
                        for (int r = 0; r < 4; r++) act[(4 * lq + r) * ld + col] = actf(acc[u][r] + bv);
                    }
            };
            // the activation is chosen once per layer, not per element
            if (R.act == FORTIS_ACT_RELU) write_back([](float v) { return fmaxf(v, 0.f); });
            else if (R.act == FORTIS_ACT_NONE) write_back([](float v) { return v; });
            else write_back([&](float v) { return apply_act(v, R.act, R.alpha); });
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
        if (STENCIL) {
            gfloat* Yraw = st_g(P.Yraw);
            if (lq == 0 && valid) {
                StCell cell;
#pragma unroll
                for (int s = 0; s < ST_SCAL_MAX; s++) cell.S[s] = in.sS[s];
                st_cell_program(sc, cell);
                for (int q0 = 0; q0 < NO; q0 += 4) {
                    float ov[4];
#pragma unroll
                    for (int t = 0; t < 4; t++) {
                        ov[t] = q0 + t < NO ? act[lrow * ld + q0 + t] : 0.f;
                        if (out_mul && q0 + t < NO) ov[t] = __fmul_rn(ov[t], out_mul[q0 + t]);
                        if (Yraw && q0 + t < NO) Yraw[(size_t)row * NO + q0 + t] = ov[t];
                    }
                    st_chain_apply(sc, cell, ov);
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        if (q0 + t < NO) {
                            const StSlotT<float*> sl = sc.refs[q0 + t];
                            st_g(sl.p)[st_off(sl, in.si, in.sj, in.skk)] = ov[t];
                        }
                }
            }
        } else {
            gfloat* Y = st_g(P.Y);
            const long base = (long)row0 * NO;
            const long lim = (long)rows * NO - base;
            for (int idx = lane; idx < 16 * NO; idx += 64) {
                if (idx >= lim) break;
                const int r = idx / NO, c = idx - r * NO;
                float v = act[r * ld + c];
                if (out_mul) v = __fmul_rn(v, out_mul[c]);
                if (c >= NO - mask_tail) v = v > 0.f ? v : 0.f;
                Y[base + idx] = v;
            }
        }
        // the next tile's input overwrites the LDS tile: every lane is done reading it
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    // The grid is persistent: this wave takes tiles first, first + stride, ...  The first tile's loads
    // are in flight while the workgroup stages the weights; after that the loads of the next tile are
    // issued before the current one is computed.
    const unsigned long long ntile = ((unsigned long long)rows + 15) / 16;
    const unsigned long long stride = (unsigned long long)gridDim.x * 4;
    unsigned long long t = (unsigned long long)blockIdx.x * 4 + wave;
    TileIn cur, nxt;
    if (t < ntile) issue(cur, (unsigned)(t * 16));
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
        const bool more = t + stride < ntile;
        if (more) issue(nxt, (unsigned)((t + stride) * 16));
        process(cur);
        if (more) cur = nxt;
    }
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
    float* h = (float*)calloc(total, sizeof(float));
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
    HIP_OK(hipMalloc((void**)&dev, total * sizeof(float)));
    HIP_OK(hipMemcpy(dev, h, total * sizeof(float), hipMemcpyHostToDevice));
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

template <bool ST, bool WLDS, int NTMAX>
static void launch_wave_variant(ChainParams& P, hipStream_t s)
{
    const ChainDesc& d = P.d;
    const size_t shmem = ((size_t)(WLDS ? d.wfloats : 0) + (size_t)4 * 16 * d.ld) * sizeof(float);
    static size_t attr = 0;
    static long slots = 0;
    if (shmem > attr || !slots) {
        HIP_OK(hipFuncSetAttribute((const void*)chain_wave_kernel<ST, WLDS, NTMAX>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        attr = shmem;
        int occ = 0;
        HIP_OK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void*)chain_wave_kernel<ST, WLDS, NTMAX>, CH_THREADS, shmem));
        slots = (long)(occ < 1 ? 1 : occ) * num_cus();
    }
    // persistent grid: as many workgroups as the chip holds at once, never more than 64-row groups
    long grid = cdiv(P.rows, 64);
    if (grid > slots) grid = slots;
    hipLaunchKernelGGL((chain_wave_kernel<ST, WLDS, NTMAX>), dim3((unsigned)grid), dim3(CH_THREADS), shmem, s, P);
    HIP_OK(hipGetLastError());
}
static int chain_ntmax(const ChainDesc& d)
{
    int nt = 0;
    for (int l = 0; l < d.nlayers; l++) if (d.L[l].Np / 16 > nt) nt = d.L[l].Np / 16;
    return nt;
}
// weights go to LDS in the wave kernel when three workgroups still fit on a CU
static bool chain_wave_wlds(const ChainDesc& d)
{
    static int force = -2;
    if (force == -2) { const char* e = getenv("FORTIS_CHAIN_WLDS"); force = e ? atoi(e) : -1; }
    if (force >= 0) return force != 0;
    return ((size_t)d.wfloats + 4 * 16 * d.ld) * sizeof(float) + sizeof(ChainParams) <= 52 * 1024;
}

template <bool ST>
static void launch_wave(ChainParams& P, hipStream_t s)
{
    const bool wlds = chain_wave_wlds(P.d);
    if (chain_ntmax(P.d) <= 4) {
        if (wlds) launch_wave_variant<ST, true, 4>(P, s);
        else launch_wave_variant<ST, false, 4>(P, s);
    } else {
        if (wlds) launch_wave_variant<ST, true, 16>(P, s);
        else launch_wave_variant<ST, false, 16>(P, s);
    }
}

void fortis_launch_chain(const ChainDesc& d, const float* X, float* Y, long rows, hipStream_t s)
{
    if (!chain_ok(d, rows)) return;
    ChainParams P;
    fill_params(&P, d, X, Y, rows, nullptr);
    // many rows of a narrow input: the wave-independent kernel
    if (rows >= 64L * num_cus() && d.L[0].K <= 64) { launch_wave<false>(P, s); return; }
    const bool wlds = chain_wlds(d);
    // few rows: 16-row tiles spread the work over more CUs (the four waves then split the n-tiles)
    if (rows < 64L * num_cus()) {
        if (wlds) launch_variant<16, true>(P, s);
        else launch_variant<16, false>(P, s);
    } else {
        if (wlds) launch_variant<64, true>(P, s);
        else launch_variant<64, false>(P, s);
    }
}

void fortis_launch_chain_stencil(const ChainDesc& d, const StencilDev& g, const StencilDev& sc, long rows,
                                 const float* const* dG, float* const* dS, float* dY, hipStream_t s)
{
    if (!chain_ok(d, rows)) return;
    ChainParams P;
    fill_params(&P, d, nullptr, nullptr, rows, dY);
    st_make_args<const float*>(g, g.cells, dG, &P.g);
    st_make_args<float*>(sc, sc.cells, dS, &P.sc);
    launch_wave<true>(P, s);
}
