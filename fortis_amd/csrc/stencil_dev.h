// Device-side helpers shared by the stencil gather/scatter kernels and the fused
// gather -> MLP -> scatter kernel.  The tables (StencilDev) live in device memory and are read
// with wave-uniform addresses; all expression arithmetic is explicit round-to-nearest fp32 with
// no contraction, matching the reference's `-fmad=false` gather.cu.
#pragma once
#include "common.h"

struct PtrTab { const float* p[FORTIS_MAX_ARRAYS]; };
struct PtrTabW { float* p[FORTIS_MAX_ARRAYS]; };

// cell number -> 1-based (i, j): the rectangle of mom6_zb/gather.cu:15-16, or the cell list.
__device__ __forceinline__ void st_cell(const StencilDev* d, long col, int& i, int& j)
{
    if (d->cells) { int c = d->cells[col]; i = 1 + c % d->sx; j = 1 + c / d->sx; }
    else { i = d->ilo + (int)(col % d->ni); j = d->jlo + (int)(col / d->ni); }
}
__device__ __forceinline__ long st_elem(const StencilDev* d, const fortis_ref_t& r, int i, int j, int kk)
{
    return r.base + (long)i * r.si + (long)j * r.sj + (r.planar ? (long)kk * d->plane[r.array] : 0L);
}
__device__ __forceinline__ float st_arith(int op, float a, float b)
{
    switch (op) {
        case 0: return __fadd_rn(a, b);
        case 1: return __fsub_rn(a, b);
        case 2: return __fmul_rn(a, b);
        default: return __fdiv_rn(a, b);
    }
}
// operand of per-cell code: 1..8 scalar, 16+ constant, 32+ earlier per-cell result
__device__ __forceinline__ float st_operand(const StencilDev* d, int code, const float (&S)[FORTIS_MAX_SCAL],
                                            const float (&c)[FORTIS_MAX_INS])
{
    float v = 0.f;
    if (code >= 32) {
#pragma unroll
        for (int m = 0; m < FORTIS_MAX_INS; m++) if (code - 32 == m) v = c[m];
    } else if (code >= 16) {
        v = d->consts[code - 16];
    } else {
#pragma unroll
        for (int s = 0; s < FORTIS_MAX_SCAL; s++) if (code - 1 == s) v = S[s];
    }
    return v;
}
// Loads the same-cell scalars and evaluates the per-cell instructions.
template <typename Tab>
__device__ __forceinline__ void st_cell_values(const StencilDev* d, const Tab& A, int i, int j, int kk,
                                               float (&S)[FORTIS_MAX_SCAL], float (&c)[FORTIS_MAX_INS])
{
#pragma unroll
    for (int s = 0; s < FORTIS_MAX_SCAL; s++) {
        S[s] = 0.f;
        if (s < d->nscal) S[s] = A.p[d->scal[s].array][st_elem(d, d->scal[s], i, j, kk)];
    }
#pragma unroll
    for (int n = 0; n < FORTIS_MAX_INS; n++) {
        c[n] = 0.f;
        if (n < d->ncell) c[n] = st_arith(d->cell[n].op, st_operand(d, d->cell[n].a, S, c), st_operand(d, d->cell[n].b, S, c));
    }
}
// Runs the tv chain on one slot value.
__device__ __forceinline__ float st_chain(const StencilDev* d, float tv, const float (&S)[FORTIS_MAX_SCAL],
                                          const float (&c)[FORTIS_MAX_INS])
{
    for (int n = 0; n < d->nchain; n++) {
        float o = st_operand(d, d->chain[n].code, S, c);
        tv = d->chain[n].tv_left ? st_arith(d->chain[n].op, tv, o) : st_arith(d->chain[n].op, o, tv);
    }
    return tv;
}
