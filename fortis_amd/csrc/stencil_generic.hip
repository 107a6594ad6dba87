// General stencil gather / scatter: every table the reference's lifter can produce, including what the
// fused kernels do not take -- fp64 host arrays, double literals, the lifter's functions (sqrtf, expf,
// logf, tanhf, fmaxf, fminf, negation) and expressions that are not one chain on the slot value.
//
// Reference: the kernels driver/fortis_gather_emit.py:49-61 (gather) and :71-81 (scatter) print, one
// thread per row / per cell, with the lifted expressions pasted in as C.  Here the expressions are
// interpreted from the table with C's types: a value is held as a double, an operation whose C type is
// float converts its operands to float and is done in fp32, one whose C type is double
// (FORTIS_INS_F64) is done in fp64; every operation is a single correctly rounded IEEE operation,
// never fused.  The index arithmetic is the same exact integer arithmetic as in the fused kernels.
#include "stencil_dev.h"

#define SG_THREADS 256

struct GenSlot { const void* p; long si, sj, plane; int f64, pad_; };   // p: array base with the element offset folded in
struct alignas(16) GenArgs {
    int nrefs, nscal, nins, pad0_;
    GenSlot refs[FORTIS_MAX_REFS];
    GenSlot scal[FORTIS_MAX_SCAL];
    int op[FORTIS_MAX_INS], a[FORTIS_MAX_INS], b[FORTIS_MAX_INS];
    double consts[FORTIS_MAX_CONST];
    unsigned count;
    int ilo, jlo, ni, sx, pad1_;
    const int* cells;
    StMagic mcount, mni, msx;
};

typedef __attribute__((address_space(1))) double gdouble;

__device__ __forceinline__ double sg_load(const GenSlot& s, long off)
{
    return s.f64 ? (double)((const gdouble*)s.p)[off] : (double)((const gfloat*)s.p)[off];
}
__device__ __forceinline__ void sg_store(const GenSlot& s, long off, float v)
{
    if (s.f64) ((gdouble*)s.p)[off] = (double)v;
    else ((gfloat*)s.p)[off] = v;
}

// Runs the instruction list on one slot value.  r: this thread's column of the result scratch in LDS.
__device__ __forceinline__ float sg_eval(const GenArgs& d, float tv, const double (&S)[FORTIS_MAX_SCAL],
                                         double (*r)[SG_THREADS], int tid)
{
    const int nins = st_u(d.nins);
    double last = (double)tv;
    for (int n = 0; n < nins; n++) {
        const int opw = st_u(d.op[n]), ca = st_u(d.a[n]), cb = st_u(d.b[n]);
        auto operand = [&](int code) -> double {
            if (code == 0) return (double)tv;
            if (code < 16) {
                double v = S[0];
#pragma unroll
                for (int s = 1; s < FORTIS_MAX_SCAL; s++) v = (code == 1 + s) ? S[s] : v;
                return v;
            }
            if (code < 32) return d.consts[code - 16];
            return r[code - 32][tid];
        };
        const double x = operand(ca), y = operand(cb);
        const float xf = (float)x, yf = (float)y;
        const bool f64 = (opw & FORTIS_INS_F64) != 0;
        double v;
        switch (opw & 0xff) {
            case FORTIS_OP_ADD: v = f64 ? __dadd_rn(x, y) : (double)__fadd_rn(xf, yf); break;
            case FORTIS_OP_SUB: v = f64 ? __dsub_rn(x, y) : (double)__fsub_rn(xf, yf); break;
            case FORTIS_OP_MUL: v = f64 ? __dmul_rn(x, y) : (double)__fmul_rn(xf, yf); break;
            case FORTIS_OP_DIV: v = f64 ? __ddiv_rn(x, y) : (double)__fdiv_rn(xf, yf); break;
            case FORTIS_OP_MAX: v = (double)fmaxf(xf, yf); break;
            case FORTIS_OP_MIN: v = (double)fminf(xf, yf); break;
            case FORTIS_OP_NEG: v = f64 ? -x : (double)(-xf); break;
            case FORTIS_OP_SQRT: v = (double)__builtin_sqrtf(xf); break;   // correctly rounded (the rn intrinsic is the approximate one here)
            case FORTIS_OP_EXP: v = (double)expf(xf); break;
            case FORTIS_OP_LOG: v = (double)logf(xf); break;
            case FORTIS_OP_TANH: v = (double)tanhf(xf); break;
            default: v = (double)xf; break;          // FORTIS_OP_F32
        }
        r[n][tid] = v;
        last = v;
    }
    return (float)last;
}

__global__ __launch_bounds__(SG_THREADS) void gather_generic_kernel(GenArgs args, float* __restrict__ X, unsigned rows)
{
    __shared__ GenArgs d;
    __shared__ double r[FORTIS_MAX_INS][SG_THREADS];
    params_to_lds(&d, SG_THREADS);
    const int tid = threadIdx.x;
    const unsigned row = blockIdx.x * SG_THREADS + tid;
    if (row >= rows) return;
    int i, j, kk;
    st_row(d, row, i, j, kk);
    double S[FORTIS_MAX_SCAL];
#pragma unroll
    for (int s = 0; s < FORTIS_MAX_SCAL; s++) {
        S[s] = 0.0;
        if (s < d.nscal) S[s] = sg_load(d.scal[s], (long)i * d.scal[s].si + (long)j * d.scal[s].sj + (long)kk * d.scal[s].plane);
    }
    const int n = st_u(d.nrefs);
    float* out = X + (size_t)row * n;
    for (int q = 0; q < n; q++) {
        const GenSlot& sl = d.refs[q];
        const float tv = (float)sg_load(sl, (long)i * sl.si + (long)j * sl.sj + (long)kk * sl.plane);   // float tv = A[...]
        out[q] = sg_eval(d, tv, S, r, tid);
    }
}

__global__ __launch_bounds__(SG_THREADS) void scatter_generic_kernel(GenArgs args, const float* __restrict__ Y, int kk)
{
    __shared__ GenArgs d;
    __shared__ double r[FORTIS_MAX_INS][SG_THREADS];
    params_to_lds(&d, SG_THREADS);
    const int tid = threadIdx.x;
    const unsigned col = blockIdx.x * SG_THREADS + tid;
    if (col >= d.count) return;
    int i, j;
    st_cell(d, col, i, j);
    double S[FORTIS_MAX_SCAL];
#pragma unroll
    for (int s = 0; s < FORTIS_MAX_SCAL; s++) {
        S[s] = 0.0;
        if (s < d.nscal) S[s] = sg_load(d.scal[s], (long)i * d.scal[s].si + (long)j * d.scal[s].sj + (long)kk * d.scal[s].plane);
    }
    const int n = st_u(d.nrefs);
    const float* in = Y + (size_t)col * n;
    for (int q = 0; q < n; q++) {
        const GenSlot& sl = d.refs[q];
        sg_store(sl, (long)i * sl.si + (long)j * sl.sj + (long)kk * sl.plane, sg_eval(d, in[q], S, r, tid));
    }
}

// ---- host side ---------------------------------------------------------------------------------------
static inline int sg_esz(const fortis_stencil_t& t, int a) { return t.elt[a] == 8 ? 8 : 4; }

// Range and operand checks of a table for the general kernels.
int fortis_stencil_validate(const fortis_stencil_t* t)
{
    if (t->narrays < 1 || t->narrays > FORTIS_MAX_ARRAYS || t->nrefs < 1 || t->nrefs > FORTIS_MAX_REFS || t->nscal < 0 ||
        t->nscal > FORTIS_MAX_SCAL || t->nins < 0 || t->nins > FORTIS_MAX_INS || t->nconst < 0 ||
        t->nconst > FORTIS_MAX_CONST || t->count < 1 || t->nk < 1 || t->count * t->nk >= 4294967295L / FORTIS_MAX_REFS) {
        fprintf(stderr, "fortis: stencil table out of range\n");
        return -1;
    }
    for (int a = 0; a < t->narrays; a++)
        if (t->elt[a] != 0 && t->elt[a] != 4 && t->elt[a] != 8) { fprintf(stderr, "fortis: stencil array %d has element size %d\n", a, t->elt[a]); return -1; }
    for (int r = 0; r < t->nrefs + t->nscal; r++) {
        const fortis_ref_t& f = r < t->nrefs ? t->refs[r] : t->scal[r - t->nrefs];
        if (f.array < 0 || f.array >= t->narrays) { fprintf(stderr, "fortis: stencil ref names array %d\n", f.array); return -1; }
    }
    // Every element a kernel will touch must lie inside its array's plane: base + i*si + j*sj in [0, plane) for
    // every visited cell (the plane index kk only adds whole planes).  A descriptor that fails this would make
    // the kernels read or write outside the arrays.
    const long ni = t->ni > 0 ? t->ni : 1, sx = t->sx > 0 ? t->sx : 1;
    for (int r = 0; r < t->nrefs + t->nscal; r++) {
        const fortis_ref_t& f = r < t->nrefs ? t->refs[r] : t->scal[r - t->nrefs];
        long lo, hi;
        if (t->cells) {
            lo = hi = f.base + (1 + t->cells[0] % sx) * f.si + (1 + t->cells[0] / sx) * f.sj;
            for (long c = 0; c < t->count; c++) {
                if (t->cells[c] < 0) { fprintf(stderr, "fortis: negative entry in the stencil cell list\n"); return -1; }
                const long e = f.base + (1 + t->cells[c] % sx) * f.si + (1 + t->cells[c] / sx) * f.sj;
                lo = e < lo ? e : lo;
                hi = e > hi ? e : hi;
            }
        } else {
            const long i0 = t->ilo, i1 = t->ilo + (t->count < ni ? t->count : ni) - 1;
            const long j0 = t->jlo, j1 = t->jlo + (t->count + ni - 1) / ni - 1;
            lo = f.base + (f.si >= 0 ? i0 : i1) * f.si + (f.sj >= 0 ? j0 : j1) * f.sj;
            hi = f.base + (f.si >= 0 ? i1 : i0) * f.si + (f.sj >= 0 ? j1 : j0) * f.sj;
        }
        if (lo < 0 || hi >= t->plane[f.array]) {
            fprintf(stderr, "fortis: stencil %s %d reaches elements %ld..%ld of array %d, whose plane has %ld\n",
                    r < t->nrefs ? "slot" : "scalar", r < t->nrefs ? r : r - t->nrefs, lo, hi, f.array, t->plane[f.array]);
            return -1;
        }
    }
    for (int n = 0; n < t->nins; n++) {
        const int op = t->ins[n].op & 0xff, codes[2] = { t->ins[n].a, t->ins[n].b };
        bool ok = op <= FORTIS_OP_F32 && (t->ins[n].op & ~(0xff | FORTIS_INS_F64)) == 0;
        for (int s = 0; s < 2; s++) {
            const int c = codes[s];
            ok = ok && (c == 0 || (c >= 1 && c <= t->nscal) || (c >= 16 && c < 16 + t->nconst) || (c >= 32 && c < 32 + n));
        }
        if (!ok) { fprintf(stderr, "fortis: bad stencil instruction %d\n", n); return -1; }
    }
    return 0;
}

// True if the table needs C's mixed types or an operator the fused kernels do not have.
bool fortis_stencil_typed(const fortis_stencil_t* t)
{
    for (int a = 0; a < t->narrays; a++) if (t->elt[a] == 8) return true;
    for (int c = 0; c < t->nconst; c++) if (t->cdouble[c]) return true;
    for (int n = 0; n < t->nins; n++) if (t->ins[n].op > FORTIS_OP_DIV) return true;   // any flag or any later operator
    return t->nscal > ST_SCAL_MAX;
}

static void sg_make_args(const fortis_stencil_t& t, const int* dcells, const void* const* arrays, GenArgs* g)
{
    memset(g, 0, sizeof *g);
    g->nrefs = t.nrefs; g->nscal = t.nscal; g->nins = t.nins;
    for (int r = 0; r < t.nrefs + t.nscal; r++) {
        const fortis_ref_t& f = r < t.nrefs ? t.refs[r] : t.scal[r - t.nrefs];
        GenSlot& s = r < t.nrefs ? g->refs[r] : g->scal[r - t.nrefs];
        s.p = (const char*)arrays[f.array] + f.base * sg_esz(t, f.array);
        s.si = f.si; s.sj = f.sj;
        s.plane = f.planar ? t.plane[f.array] : 0;
        s.f64 = sg_esz(t, f.array) == 8;
    }
    for (int n = 0; n < t.nins; n++) { g->op[n] = t.ins[n].op; g->a[n] = t.ins[n].a; g->b[n] = t.ins[n].b; }
    for (int c = 0; c < t.nconst; c++) g->consts[c] = t.cdouble[c] ? t.dconsts[c] : (double)t.consts[c];
    g->count = (unsigned)t.count;
    g->ilo = t.ilo; g->jlo = t.jlo; g->ni = t.ni > 0 ? t.ni : 1; g->sx = t.sx > 0 ? t.sx : 1;
    g->cells = dcells;
    g->mcount = st_magic((unsigned)t.count);
    g->mni = st_magic((unsigned)g->ni);
    g->msx = st_magic((unsigned)g->sx);
}

void fortis_launch_gather_generic(const fortis_stencil_t& t, const int* dcells, const void* const* dA, float* dX, hipStream_t s)
{
    GenArgs g;
    sg_make_args(t, dcells, dA, &g);
    const unsigned rows = (unsigned)(t.count * t.nk);
    hipLaunchKernelGGL(gather_generic_kernel, dim3((unsigned)cdiv(rows, SG_THREADS)), dim3(SG_THREADS), 0, s, g, dX, rows);
    HIP_OK(hipGetLastError());
}
void fortis_launch_scatter_generic(const fortis_stencil_t& t, const int* dcells, void* const* dA, const float* dY, int kk, hipStream_t s)
{
    GenArgs g;
    sg_make_args(t, dcells, (const void* const*)dA, &g);
    hipLaunchKernelGGL(scatter_generic_kernel, dim3((unsigned)cdiv(t.count, SG_THREADS)), dim3(SG_THREADS), 0, s, g, dY, kk);
    HIP_OK(hipGetLastError());
}
