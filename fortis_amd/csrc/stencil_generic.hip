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
#define SG_CHAIN_MAX 8

struct GenSlot { const void* p; long si, sj, plane; int f64, pad_; };   // p: array base with the element offset folded in
struct alignas(16) GenArgs {
    int nrefs, nscal, nins, cellmask;      // cellmask: bit n set = instruction n does not depend on the slot value
    GenSlot refs[ST_KREFS];                // the slots of this launch (a larger table goes in several launches)
    GenSlot scal[FORTIS_MAX_SCAL];
    int op[FORTIS_MAX_INS], a[FORTIS_MAX_INS], b[FORTIS_MAX_INS];
    double consts[FORTIS_MAX_CONST];
    unsigned count;
    int ilo, jlo, ni, sx, uniform;          // uniform: every slot has the strides of slot 0
    const int* cells;
    StMagic mcount, mni, msx;
    int slotkind;                           // slot arrays: 0 all fp32, 1 all fp64, 2 mixed
    // Chain form of the slot-dependent instructions (nchain < 0: not of that form): step s applies ch_op[s] to the
    // running slot value and one operand that is the same for every slot of the row (ch_other[s], an operand
    // code, -1 for a unary operator); ch_left[s]: the running value is the left operand.
    int nchain, pad_[2];
    int ch_op[SG_CHAIN_MAX], ch_other[SG_CHAIN_MAX], ch_left[SG_CHAIN_MAX];
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
// Instructions that do not depend on the slot value (bit set in d.cellmask) are the same for every slot of a
// row: phase 1 runs those once per row, phase 0 the others once per slot; both leave their results in r.
// The row's scalars are rows nins .. nins + nscal - 1 of r, so that an operand of any kind is one read.
__device__ __forceinline__ float sg_eval(const GenArgs& d, float tv, double (*r)[SG_THREADS], int tid, int phase)
{
    const int nins = st_u(d.nins), cellmask = st_u(d.cellmask);
    for (int n = 0; n < nins; n++) {
        if (((cellmask >> n) & 1) != phase) continue;
        const int opw = st_u(d.op[n]), ca = st_u(d.a[n]), cb = st_u(d.b[n]);
        auto operand = [&](int code) -> double {
            if (code == 0) return (double)tv;
            if (code < 16) return r[nins + code - 1][tid];
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
    }
    return nins ? (float)r[nins - 1][tid] : tv;
}

// An operand that does not involve the slot value: a scalar of the row, a constant, or an earlier result.
__device__ __forceinline__ double sg_cell_operand(const GenArgs& d, double (*r)[SG_THREADS], int tid, int code)
{
    const int nins = st_u(d.nins);
    if (code < 16) return r[nins + code - 1][tid];
    if (code < 32) return d.consts[code - 16];
    return r[code - 32][tid];
}

template <typename F>
__device__ __forceinline__ void sg_apply(float* mine, int n, bool left, double c, F f)
{
    if (left) for (int q = 0; q < n; q++) mine[q] = (float)f((double)mine[q], c);
    else for (int q = 0; q < n; q++) mine[q] = (float)f(c, (double)mine[q]);
}

// fp64 division of fp32 slot values by one divisor: the compiler's sequence (v_div_scale_f64 of both operands,
// v_rcp_f64 with two Newton steps, quotient, residual, v_div_fmas_f64, v_div_fixup_f64) neither scales nor fixes
// anything up when the numerators are finite non-zero floats (as doubles their exponents lie in [-149, 127]) and the
// divisor's exponent lies in [-400, 400]: no operand, reciprocal or quotient comes near the ends of the double range.
// A numerator of +0 also comes out right through the short form (0 * r carries the quotient's sign, the residual is
// +0); -0 does not (the last fma adds zeros of opposite sign) and goes the long way with infinities and NaNs.
// True when the short form holds for every active lane of the wave.
__device__ __forceinline__ bool sg_div_wave_in_range(const float* mine, int n, double c)
{
    const unsigned ce = ((unsigned)(__double_as_longlong(c) >> 52)) & 0x7ffu;
    unsigned lo = 0xffffffffu, hi = 0;
    for (int q = 0; q < n; q++) {
        // sign rotated to the bottom and flipped: -0 -> 0, +0 -> 1, infinities and NaNs -> 0xff000000 and above
        const unsigned k = __builtin_rotateleft32(__float_as_uint(mine[q]), 1) ^ 1u;
        lo = k < lo ? k : lo;
        hi = k > hi ? k : hi;
    }
    const bool out = ce < 1023u - 400u || ce > 1023u + 400u || lo == 0u || hi >= 0xff000000u;
    return __builtin_amdgcn_ballot_w64(out) == 0;
}

// One step of the chain form on all n slot values of the row: the operator is decoded once, not once per slot.
// Same arithmetic as sg_eval: operands as doubles, an fp32 operation converts them to float first.
__device__ __forceinline__ void sg_chain_step(int opw, bool left, double c, float* mine, int n)
{
    const bool f64 = (opw & FORTIS_INS_F64) != 0;
    switch (opw & 0xff) {
        case FORTIS_OP_ADD:
            if (f64) sg_apply(mine, n, left, c, [](double x, double y) { return __dadd_rn(x, y); });
            else sg_apply(mine, n, left, c, [](double x, double y) { return (double)__fadd_rn((float)x, (float)y); });
            break;
        case FORTIS_OP_SUB:
            if (f64) sg_apply(mine, n, left, c, [](double x, double y) { return __dsub_rn(x, y); });
            else sg_apply(mine, n, left, c, [](double x, double y) { return (double)__fsub_rn((float)x, (float)y); });
            break;
        case FORTIS_OP_MUL:
            if (f64) sg_apply(mine, n, left, c, [](double x, double y) { return __dmul_rn(x, y); });
            else sg_apply(mine, n, left, c, [](double x, double y) { return (double)__fmul_rn((float)x, (float)y); });
            break;
        case FORTIS_OP_DIV:
            if (f64 && left && sg_div_wave_in_range(mine, n, c)) {
                // every slot value of the row over the same divisor, all operands clear of the ranges in which the
                // IEEE sequence would scale or fix up (see sg_div_wave_in_range): its reciprocal and two Newton steps
                // once per row, then a multiply and two fmas per slot -- the same operations, hence the same bits
                double r = __builtin_amdgcn_rcp(c);
                r = __fma_rn(r, __fma_rn(-c, r, 1.0), r);
                r = __fma_rn(r, __fma_rn(-c, r, 1.0), r);
                for (int q = 0; q < n; q++) {
                    const double x = (double)mine[q], q0 = __dmul_rn(x, r);
                    mine[q] = (float)__fma_rn(__fma_rn(-c, q0, x), r, q0);
                }
            } else if (f64) sg_apply(mine, n, left, c, [](double x, double y) { return __ddiv_rn(x, y); });
            else sg_apply(mine, n, left, c, [](double x, double y) { return (double)__fdiv_rn((float)x, (float)y); });
            break;
        case FORTIS_OP_MAX: sg_apply(mine, n, left, c, [](double x, double y) { return (double)fmaxf((float)x, (float)y); }); break;
        case FORTIS_OP_MIN: sg_apply(mine, n, left, c, [](double x, double y) { return (double)fminf((float)x, (float)y); }); break;
        case FORTIS_OP_NEG: sg_apply(mine, n, true, c, [](double x, double) { return (double)(-(float)x); }); break;   // exact in either type
        case FORTIS_OP_SQRT: sg_apply(mine, n, true, c, [](double x, double) { return (double)__builtin_sqrtf((float)x); }); break;
        case FORTIS_OP_EXP: sg_apply(mine, n, true, c, [](double x, double) { return (double)expf((float)x); }); break;
        case FORTIS_OP_LOG: sg_apply(mine, n, true, c, [](double x, double) { return (double)logf((float)x); }); break;
        case FORTIS_OP_TANH: sg_apply(mine, n, true, c, [](double x, double) { return (double)tanhf((float)x); }); break;
        default: break;                                        // FORTIS_OP_F32: the running value is a float already
    }
}

// Loads the row's scalars into their rows of r.
__device__ __forceinline__ void sg_scalars(const GenArgs& d, double (*r)[SG_THREADS], int tid, int i, int j, int kk)
{
    const int nins = st_u(d.nins), nscal = st_u(d.nscal);
    for (int s = 0; s < nscal; s++)
        r[nins + s][tid] = sg_load(d.scal[s], (long)i * d.scal[s].si + (long)j * d.scal[s].sj + (long)kk * d.scal[s].plane);
}
// Element offset of slot sl at cell (i, j, kk); off0 serves every slot when they share their strides.
__device__ __forceinline__ long sg_off(const GenArgs& d, const GenSlot& sl, long off0, int i, int j, int kk)
{
    return st_u(d.uniform) ? off0 : (long)i * sl.si + (long)j * sl.sj + (long)kk * sl.plane;
}

// Loads the row's n slot values into mine[], four loads in flight at a time.  T: element type of every slot's array.
template <typename T>
__device__ __forceinline__ void sg_load_slots(const GenArgs& d, float* mine, int n, long off0, int i, int j, int kk)
{
    typedef __attribute__((address_space(1))) T gT;
    int q = 0;
    for (; q + 4 <= n; q += 4) {
        T v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const GenSlot& sl = d.refs[q + u];
            v[u] = ((const gT*)sl.p)[sg_off(d, sl, off0, i, j, kk)];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) mine[q + u] = (float)v[u];          // float tv = A[...]
    }
    for (; q < n; q++) {
        const GenSlot& sl = d.refs[q];
        mine[q] = (float)((const gT*)sl.p)[sg_off(d, sl, off0, i, j, kk)];
    }
}

// One thread per row.  The row's slot values are loaded first (independent loads, several in flight), then
// evaluated in place in the workgroup's tile of X in LDS; the tile -- SG_THREADS consecutive rows, contiguous
// in X -- is written out with coalesced 16-byte stores (a thread storing its own row strides by the row length).
// Dynamic LDS: [nins + nscal][SG_THREADS] doubles (expression results, then the row's scalars), then the tile [SG_THREADS][nrefs] floats.
// A table of more than ST_KREFS slots is gathered in several launches: a launch holds slots q0 .. q0 + nrefs - 1 of the
// table and writes those columns of X, whose rows are `pitch` floats long.
__global__ __launch_bounds__(SG_THREADS) void gather_generic_kernel(GenArgs args, float* __restrict__ X, unsigned rows, unsigned pitch,
                                                                    unsigned q0)
{
    __shared__ GenArgs d;
    extern __shared__ __attribute__((aligned(16))) double sg_dyn[];
    params_to_lds(&d, SG_THREADS);
    const int tid = threadIdx.x;
    const int n = st_u(d.nrefs), nins = st_u(d.nins);
    double (*r)[SG_THREADS] = (double (*)[SG_THREADS])sg_dyn;
    float* tile = (float*)(sg_dyn + (size_t)(nins + st_u(d.nscal)) * SG_THREADS);
    const unsigned row0 = st_xcd_band_block() * SG_THREADS, row = row0 + tid;
    if (row < rows) {
        int i, j, kk;
        st_row(d, row, i, j, kk);
        sg_scalars(d, r, tid, i, j, kk);
        const long off0 = (long)i * d.refs[0].si + (long)j * d.refs[0].sj + (long)kk * d.refs[0].plane;
        float* mine = tile + tid * n;
        const int kind = st_u(d.slotkind);
        if (kind == 1) sg_load_slots<double>(d, mine, n, off0, i, j, kk);
        else if (kind == 0) sg_load_slots<float>(d, mine, n, off0, i, j, kk);
        else
            for (int q = 0; q < n; q++) {
                const GenSlot& sl = d.refs[q];
                mine[q] = (float)sg_load(sl, sg_off(d, sl, off0, i, j, kk));   // float tv = A[...]
            }
        sg_eval(d, 0.f, r, tid, 1);
        const int nchain = st_u(d.nchain);
        if (nchain >= 0) {
            for (int c = 0; c < nchain; c++) {
                const int other = st_u(d.ch_other[c]);
                sg_chain_step(st_u(d.ch_op[c]), st_u(d.ch_left[c]) != 0, other >= 0 ? sg_cell_operand(d, r, tid, other) : 0.0, mine, n);
            }
        } else {
            for (int q = 0; q < n; q++) mine[q] = sg_eval(d, mine[q], r, tid, 0);
        }
    }
    __syncthreads();
    const unsigned nr = rows - row0 < SG_THREADS ? rows - row0 : SG_THREADS, total = nr * n;
    float* dst = X + (size_t)row0 * n;
    if (pitch != (unsigned)n) {
        // a column band of X: element e of the tile is slot e % n of row e / n
        for (unsigned e = tid; e < total; e += SG_THREADS) X[(size_t)(row0 + e / n) * pitch + q0 + e % n] = tile[e];
    } else if (((uintptr_t)dst & 15) == 0) {
        const unsigned t4 = total / 4;
        typedef float sg_v4f __attribute__((ext_vector_type(4)));
        // X is written once and read by another kernel: non-temporal stores
        for (unsigned v = tid; v < t4; v += SG_THREADS) __builtin_nontemporal_store(((const sg_v4f*)tile)[v], (sg_v4f*)dst + v);
        for (unsigned e = t4 * 4 + tid; e < total; e += SG_THREADS) dst[e] = tile[e];
    } else {
        for (unsigned e = tid; e < total; e += SG_THREADS) dst[e] = tile[e];
    }
}

// One thread per cell of layer kk.  Dynamic LDS: [nins + nscal][SG_THREADS] doubles (expression results, scalars).
__global__ __launch_bounds__(SG_THREADS) void scatter_generic_kernel(GenArgs args, const float* __restrict__ Y, int kk, unsigned pitch,
                                                                     unsigned q0)
{
    __shared__ GenArgs d;
    extern __shared__ __attribute__((aligned(16))) double sg_dyn[];
    params_to_lds(&d, SG_THREADS);
    double (*r)[SG_THREADS] = (double (*)[SG_THREADS])sg_dyn;
    const int tid = threadIdx.x;
    const unsigned col = blockIdx.x * SG_THREADS + tid;
    if (col >= d.count) return;
    int i, j;
    st_cell(d, col, i, j);
    sg_scalars(d, r, tid, i, j, kk);
    const long off0 = (long)i * d.refs[0].si + (long)j * d.refs[0].sj + (long)kk * d.refs[0].plane;
    const int n = st_u(d.nrefs);
    const float* in = Y + (size_t)col * pitch + q0;          // this launch's outputs of the cell's row
    sg_eval(d, 0.f, r, tid, 1);
    for (int q = 0; q < n; q++) {
        const GenSlot& sl = d.refs[q];
        sg_store(sl, sg_off(d, sl, off0, i, j, kk), sg_eval(d, in[q], r, tid, 0));
    }
}

// ---- host side ---------------------------------------------------------------------------------------
static inline int sg_esz(const fortis_stencil_t& t, int a) { return t.elt[a] == 8 ? 8 : 4; }

// Range and operand checks of a table for the general kernels.
int fortis_stencil_validate(const fortis_stencil_t* t)
{
    if (t->narrays < 1 || t->narrays > FORTIS_MAX_ARRAYS || t->nrefs < 1 || t->nrefs > FORTIS_MAX_REFS || t->nscal < 0 ||
        t->nscal > FORTIS_MAX_SCAL || t->nins < 0 || t->nins > FORTIS_MAX_INS || t->nconst < 0 ||
        t->nconst > FORTIS_MAX_CONST || t->count < 1 || t->nk < 1 || t->count * t->nk >= 4294967295L / t->nrefs) {
        fprintf(stderr, "fortis: stencil table out of range\n");
        return -1;
    }
    for (int a = 0; a < t->narrays; a++)
        if (t->elt[a] != 0 && t->elt[a] != 4 && t->elt[a] != 8) { fprintf(stderr, "fortis: stencil array %d has element size %d\n", a, t->elt[a]); return -1; }
    for (int r = 0; r < t->nrefs + t->nscal; r++) {
        const fortis_ref_t& f = r < t->nrefs ? t->refs[r] : t->scal[r - t->nrefs];
        if (f.array < 0 || f.array >= t->narrays) { fprintf(stderr, "fortis: stencil ref names array %d\n", f.array); return -1; }
    }
    // An array with a plane per enclosing-loop iteration must hold the nk planes starting at klo: the host-array
    // entries copy exactly those, and the kernels index them.
    for (int a = 0; a < t->narrays; a++) {
        if (t->plane[a] < 1 || t->total[a] < t->plane[a]) { fprintf(stderr, "fortis: stencil array %d has %ld elements in planes of %ld\n", a, t->total[a], t->plane[a]); return -1; }
        if (t->total[a] > t->plane[a] && ((long)(t->klo > 1 ? t->klo : 1) - 1 + t->nk) * t->plane[a] > t->total[a]) {
            fprintf(stderr, "fortis: stencil array %d holds %ld elements, fewer than the %d planes of %ld from iteration %d on\n",
                    a, t->total[a], t->nk, t->plane[a], t->klo > 1 ? t->klo : 1);
            return -1;
        }
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

// Kernel arguments for slots q0 .. q0 + nq - 1 of the table.
static void sg_make_args(const fortis_stencil_t& t, const int* dcells, const void* const* arrays, GenArgs* g, int q0, int nq)
{
    memset(g, 0, sizeof *g);
    g->nrefs = nq; g->nscal = t.nscal; g->nins = t.nins;
    for (int r = 0; r < nq + t.nscal; r++) {
        const fortis_ref_t& f = r < nq ? t.refs[q0 + r] : t.scal[r - nq];
        GenSlot& s = r < nq ? g->refs[r] : g->scal[r - nq];
        s.p = (const char*)arrays[f.array] + f.base * sg_esz(t, f.array);
        s.si = f.si; s.sj = f.sj;
        s.plane = f.planar ? t.plane[f.array] : 0;
        s.f64 = sg_esz(t, f.array) == 8;
    }
    for (int n = 0; n < t.nins; n++) {
        g->op[n] = t.ins[n].op; g->a[n] = t.ins[n].a; g->b[n] = t.ins[n].b;
        // depends on the slot value: reads it, or reads the result of an instruction that does
        auto dep = [&](int code) { return code == 0 || (code >= 32 && !((g->cellmask >> (code - 32)) & 1)); };
        const bool binary = (t.ins[n].op & 0xff) <= FORTIS_OP_MIN;
        if (!dep(t.ins[n].a) && !(binary && dep(t.ins[n].b))) g->cellmask |= 1u << n;
    }
    for (int c = 0; c < t.nconst; c++) g->consts[c] = t.cdouble[c] ? t.dconsts[c] : (double)t.consts[c];
    // Chain form: every slot-dependent instruction combines the previous one's result (the slot value for the
    // first) with an operand that is the same for all slots, the last instruction is the last step, and no fp64
    // step feeds another fp64 step (the running values are kept as floats).
    {
        int prev = -1, nch = 0;
        bool ok = t.nins == 0 || !((g->cellmask >> (t.nins - 1)) & 1);
        for (int n = 0; n < t.nins && ok; n++) {
            if ((g->cellmask >> n) & 1) continue;
            const int op = t.ins[n].op & 0xff, a = t.ins[n].a, b = t.ins[n].b, run = prev < 0 ? 0 : 32 + prev;
            const bool binary = op <= FORTIS_OP_MIN;
            auto dep = [&](int code) { return code == 0 || (code >= 32 && !((g->cellmask >> (code - 32)) & 1)); };
            if (nch == SG_CHAIN_MAX) { ok = false; break; }
            if (a == run && !(binary && dep(b))) { g->ch_left[nch] = 1; g->ch_other[nch] = binary ? b : -1; }
            else if (binary && b == run && !dep(a)) { g->ch_left[nch] = 0; g->ch_other[nch] = a; }
            else { ok = false; break; }
            // a double handed from one fp64 step to the next would be cut to a float (an fp32 step converts its
            // operands to float anyway)
            if (prev >= 0 && (t.ins[prev].op & FORTIS_INS_F64) && (t.ins[n].op & FORTIS_INS_F64)) { ok = false; break; }
            g->ch_op[nch++] = t.ins[n].op;
            prev = n;
        }
        g->nchain = ok ? nch : -1;
    }
    g->slotkind = g->refs[0].f64;
    for (int r = 1; r < nq; r++) if (g->refs[r].f64 != g->refs[0].f64) g->slotkind = 2;
    g->uniform = 1;
    for (int r = 1; r < nq; r++)
        if (g->refs[r].si != g->refs[0].si || g->refs[r].sj != g->refs[0].sj || g->refs[r].plane != g->refs[0].plane) g->uniform = 0;
    g->count = (unsigned)t.count;
    g->ilo = t.ilo; g->jlo = t.jlo; g->ni = t.ni > 0 ? t.ni : 1; g->sx = t.sx > 0 ? t.sx : 1;
    g->cells = dcells;
    g->mcount = st_magic((unsigned)t.count);
    g->mni = st_magic((unsigned)g->ni);
    g->msx = st_magic((unsigned)g->sx);
}

void fortis_launch_gather_generic(const fortis_stencil_t& t, const int* dcells, const void* const* dA, float* dX, hipStream_t s)
{
    const unsigned rows = (unsigned)(t.count * t.nk);
    static bool sized = false;
    if (!sized) {
        HIP_OK(hipFuncSetAttribute((const void*)gather_generic_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   SG_THREADS * (int)((FORTIS_MAX_INS + FORTIS_MAX_SCAL) * sizeof(double) + ST_KREFS * sizeof(float))));   // 112 KB
        HIP_OK(hipFuncSetAttribute((const void*)scatter_generic_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   SG_THREADS * (int)((FORTIS_MAX_INS + FORTIS_MAX_SCAL) * sizeof(double))));
        sized = true;
    }
    for (int q0 = 0; q0 < t.nrefs; q0 += ST_KREFS) {
        const int nq = t.nrefs - q0 < ST_KREFS ? t.nrefs - q0 : ST_KREFS;
        GenArgs g;
        sg_make_args(t, dcells, dA, &g, q0, nq);
        const size_t shmem = (size_t)SG_THREADS * ((t.nins + t.nscal) * sizeof(double) + nq * sizeof(float));
        hipLaunchKernelGGL(gather_generic_kernel, dim3((unsigned)cdiv(rows, SG_THREADS)), dim3(SG_THREADS), shmem, s, g, dX, rows,
                           (unsigned)t.nrefs, (unsigned)q0);
        HIP_OK(hipGetLastError());
    }
}
void fortis_launch_scatter_generic(const fortis_stencil_t& t, const int* dcells, void* const* dA, const float* dY, int kk, hipStream_t s)
{
    static bool sized = false;
    if (!sized) {
        HIP_OK(hipFuncSetAttribute((const void*)scatter_generic_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   SG_THREADS * (int)((FORTIS_MAX_INS + FORTIS_MAX_SCAL) * sizeof(double))));
        sized = true;
    }
    for (int q0 = 0; q0 < t.nrefs; q0 += ST_KREFS) {
        const int nq = t.nrefs - q0 < ST_KREFS ? t.nrefs - q0 : ST_KREFS;
        GenArgs g;
        sg_make_args(t, dcells, (const void* const*)dA, &g, q0, nq);
        hipLaunchKernelGGL(scatter_generic_kernel, dim3((unsigned)cdiv(t.count, SG_THREADS)), dim3(SG_THREADS),
                           (size_t)SG_THREADS * (t.nins + t.nscal) * sizeof(double), s, g, dY, kk, (unsigned)t.nrefs, (unsigned)q0);
        HIP_OK(hipGetLastError());
    }
}
