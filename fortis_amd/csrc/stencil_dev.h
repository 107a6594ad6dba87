// Device-side helpers shared by the stencil gather/scatter kernels and the fused
// gather -> MLP -> scatter kernel.
//
// The tables travel as kernel arguments (StencilArgs, ~1.3 KB) and every kernel first copies its
// argument block from the kernarg segment into LDS with one 16-byte vector load per thread
// (params_to_lds); after that a table read is an LDS read.  Reading the tables in place (scalar loads
// from the kernarg segment, each followed by a wait) cost a wave ~80 serialized round trips and was
// what bounded the first versions of these kernels.  Each slot carries its final device pointer
// (array base + element offset folded in on the host), so slot loads need no second table.
// All expression arithmetic is explicit round-to-nearest fp32 with no contraction, matching the
// reference's `-fmad=false` gather.cu.
#pragma once
#include "common.h"

#define ST_CHAIN_MAX 6   // operations chained on the slot value
#define ST_CELL_MAX 6    // per-cell instructions (no slot value involved)
#define ST_SCAL_MAX 4    // same-cell scalars the kernels load

template <typename P>
struct StSlotT { P p; int si, sj; long plane; };      // elem = p[i*si + j*sj + kk*plane]

// Copies the kernel's first (by-value, 16-byte aligned) argument from the kernarg segment into LDS.
template <typename T>
__device__ __forceinline__ void params_to_lds(T* dst, int nthreads)
{
    static_assert(sizeof(T) % 16 == 0, "parameter block must be a multiple of 16 bytes");
    const float4* src = (const float4*)__builtin_amdgcn_kernarg_segment_ptr();
    for (int i = threadIdx.x; i < (int)(sizeof(T) / 16); i += nthreads) ((float4*)dst)[i] = src[i];
    __syncthreads();
}
__device__ __forceinline__ unsigned st_xcd_band_block() { return fortis_xcd_band(blockIdx.x, gridDim.x); }
// A pointer read back from LDS has lost its address space; device arrays are global memory.
typedef __attribute__((address_space(1))) float gfloat;
__device__ __forceinline__ const gfloat* st_g(const float* p) { return (const gfloat*)p; }
__device__ __forceinline__ gfloat* st_g(float* p) { return (gfloat*)p; }
// A table that no kernel writes, read at an index that is the same in every lane: through the constant address
// space such reads are scalar loads (one request per wave, neighbours fetched together), where a global load of a
// uniform address is a vector instruction that every lane waits for.
typedef __attribute__((address_space(4))) float cfloat;
__device__ __forceinline__ const cfloat* st_c(const float* p) { return (const cfloat*)p; }
__device__ __forceinline__ int st_u(int v) { return __builtin_amdgcn_readfirstlane(v); }   // wave-uniform value
struct StIns { int op, a, b; float ca, cb; };          // per-cell instruction, constants inlined
struct StStep { int op, code, tv_left; float cv; };    // tv chain step, constant inlined

// Exact unsigned division by a divisor fixed for the launch: q = (n * m) >> 64 with m = ceil(2^64 / d),
// exact for every 32-bit n (n * (m d - 2^64) < 2^64).  d == 1 has no 64-bit m and is flagged.
struct StMagic { unsigned mh, ml, d, one; };
static inline StMagic st_magic(unsigned d)
{
    StMagic m = { 0u, 0u, d ? d : 1u, d <= 1u ? 1u : 0u };
    if (!m.one) {
        const unsigned __int128 v = (((unsigned __int128)1 << 64) + d - 1) / d;
        m.mh = (unsigned)(v >> 32); m.ml = (unsigned)v;
    }
    return m;
}
__device__ __forceinline__ void st_divmod(unsigned n, const StMagic& m, unsigned& q, unsigned& r)
{
    if (st_u((int)m.one)) { q = n; r = 0; return; }
    const unsigned long long t = (unsigned long long)n * m.mh + __umulhi(n, m.ml);
    q = (unsigned)(t >> 32);
    r = n - q * m.d;
}

template <typename P>
struct alignas(16) StencilArgsT {
    int nrefs, nscal, ncell, nchain;
    StSlotT<P> refs[ST_KREFS];
    StSlotT<P> scal[ST_SCAL_MAX];
    StIns cell[ST_CELL_MAX];
    StStep chain[ST_CHAIN_MAX];
    unsigned count;
    int ilo, jlo, ni, sx;
    const int* cells;
    StMagic mcount, mni, msx;   // exact division by count, ni, sx
    int uniform;                // every slot and scalar has the same (si, sj, plane): one offset per cell
    int refs_uniform;           // every slot does (the scalars may differ, e.g. a 2-D plane among 3-D arrays)
    int pad_[2];
};
typedef StencilArgsT<const float*> GatherArgs;
typedef StencilArgsT<float*> ScatterArgs;

// cell number -> 1-based (i, j): the rectangle of mom6_zb/gather.cu:15-16, or the cell list.
template <typename A>
__device__ __forceinline__ void st_cell(const A& d, unsigned col, int& i, int& j)
{
    unsigned q, r;
    if (d.cells) { const unsigned c = (unsigned)((const __attribute__((address_space(1))) int*)d.cells)[col]; st_divmod(c, d.msx, q, r); i = 1 + (int)r; j = 1 + (int)q; }
    else { st_divmod(col, d.mni, q, r); i = d.ilo + (int)r; j = d.jlo + (int)q; }
}
// row of the flattened (cell, iteration) space -> iteration kk and 1-based (i, j)
template <typename A>
__device__ __forceinline__ void st_row(const A& d, unsigned row, int& i, int& j, int& kk)
{
    unsigned q, col;
    st_divmod(row, d.mcount, q, col);
    kk = (int)q;
    st_cell(d, col, i, j);
}
template <typename S>
__device__ __forceinline__ long st_off(const S& r, int i, int j, int kk)
{
    return (long)i * r.si + (long)j * r.sj + (long)kk * r.plane;
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
// operand of per-cell code: 1..8 scalar, 16+ constant (value inlined as cv), 32+ earlier result.
// NS / NC: how many scalars / per-cell results the caller's tables can hold (the full table sizes by default; the
// kernels for small tables pass less and save a select per slot they do not have).
template <int NS, int NC>
__device__ __forceinline__ float st_operand(int code, float cv, const float (&S)[NS], const float (&c)[NC])
{
    float v = cv;
#pragma unroll
    for (int m = 0; m < NC; m++) v = (code == 32 + m) ? c[m] : v;
#pragma unroll
    for (int s = 0; s < NS; s++) v = (code == 1 + s) ? S[s] : v;
    return v;
}
// Same-cell scalars and per-cell instruction results of one cell.
template <int NS = ST_SCAL_MAX, int NC = ST_CELL_MAX>
struct StCellT { float S[NS]; float c[NC]; };
typedef StCellT<> StCell;

// Evaluates the per-cell instructions on scalars already in cell.S.
template <typename A, int NS, int NC>
__device__ __forceinline__ void st_cell_program(const A& d, StCellT<NS, NC>& cell)
{
    const int ncell = st_u(d.ncell);
#pragma unroll
    for (int n = 0; n < NC; n++) {
        cell.c[n] = 0.f;
        if (n < ncell) {
            const StIns ci = d.cell[n];
            cell.c[n] = st_arith(st_u(ci.op), st_operand<NS, NC>(st_u(ci.a), ci.ca, cell.S, cell.c), st_operand<NS, NC>(st_u(ci.b), ci.cb, cell.S, cell.c));
        }
    }
}
// Loads the same-cell scalars and evaluates the per-cell instructions.
template <typename A>
__device__ __forceinline__ void st_prepare(const A& d, int i, int j, int kk, StCell& cell)
{
    // unconditional loads (an unused scalar re-reads scalar 0): no branch separates them, so they are
    // issued together with the slot loads and waited for once
#pragma unroll
    for (int s = 0; s < ST_SCAL_MAX; s++) {
        const StSlotT<decltype(d.scal[0].p)> sl = d.scal[s < d.nscal ? s : 0];
        cell.S[s] = st_g(sl.p)[st_off(sl, i, j, kk)];
    }
    st_cell_program(d, cell);
}
// ---- many numerators over one divisor ------------------------------------------------------------------------
// The compiler's IEEE fp32 division is eleven instructions: v_div_scale_f32 of both operands, v_rcp_f32, a Newton
// step on the reciprocal, the quotient with two residual corrections (the last one in v_div_fmas_f32) and
// v_div_fixup_f32.  When numerator and divisor both lie in [2^-40, 2^40] neither v_div_scale scales (no operand or
// quotient comes near the ends of the exponent range), v_div_fmas is a plain fma and v_div_fixup returns its input,
// so the same result, bit for bit, comes from the reciprocal's two fmas once per divisor and a multiply and four
// fmas per numerator.  st_div_key maps a value to its bit pattern without the sign: the range is then an unsigned
// interval (zeros, denormals, infinities and NaNs fall outside), and a whole set of values is checked through its
// smallest and largest key.
#define ST_DIV_KEY_LO (87u << 24)       // 2^-40
#define ST_DIV_KEY_HI (168u << 24)      // 2^41: keys below it have exponents up to 2^40
__device__ __forceinline__ unsigned st_div_key(float v) { return __float_as_uint(v) << 1; }
__device__ __forceinline__ float st_div_rcp(float d)
{
    const float r = __builtin_amdgcn_rcpf(d);
    return fmaf(fmaf(-d, r, 1.f), r, r);
}
// n / d given rcp = st_div_rcp(d); both operands in range
__device__ __forceinline__ float st_div_inrange(float n, float d, float rcp)
{
    const float q0 = __fmul_rn(n, rcp);
    const float q1 = fmaf(fmaf(-d, q0, n), rcp, q0);
    return fmaf(fmaf(-d, q1, n), rcp, q1);
}
// true when every lane of the wave has all its N values (and `also`) in range
template <int N>
__device__ __forceinline__ bool st_div_wave_in_range(const float (&v)[N], float also)
{
    unsigned lo = st_div_key(also), hi = lo;
#pragma unroll
    for (int t = 0; t < N; t++) {
        const unsigned k = st_div_key(v[t]);
        lo = k < lo ? k : lo;
        hi = k > hi ? k : hi;
    }
    const bool out = lo < ST_DIV_KEY_LO || hi >= ST_DIV_KEY_HI;
    return __builtin_amdgcn_ballot_w64(out) == 0;
}

// Runs the tv chain on N slot values at once: the loop over chain steps is a real loop (one table
// read and one wave-uniform switch per step), each arm handles all N values, so the generated code
// holds each operation once per arm instead of once per slot and step.
// FASTDIV: a division of all N values by the step's operand takes the short in-range form when the whole wave allows it.
template <int N, bool FASTDIV = false, typename A, int NS, int NC>
__device__ __forceinline__ void st_chain_apply(const A& d, const StCellT<NS, NC>& cell, float (&tv)[N])
{
    const int nchain = st_u(d.nchain);
    for (int n = 0; n < nchain; n++) {
        const StStep st = d.chain[n];
        const float o = st_operand<NS, NC>(st_u(st.code), st.cv, cell.S, cell.c);
        switch (st_u(st.op * 2 + (st.tv_left ? 1 : 0))) {
            case 0: case 1:
#pragma unroll
                for (int t = 0; t < N; t++) tv[t] = __fadd_rn(tv[t], o);
                break;
            case 2:
#pragma unroll
                for (int t = 0; t < N; t++) tv[t] = __fsub_rn(o, tv[t]);
                break;
            case 3:
#pragma unroll
                for (int t = 0; t < N; t++) tv[t] = __fsub_rn(tv[t], o);
                break;
            case 4: case 5:
#pragma unroll
                for (int t = 0; t < N; t++) tv[t] = __fmul_rn(tv[t], o);
                break;
            case 6:
#pragma unroll
                for (int t = 0; t < N; t++) tv[t] = __fdiv_rn(o, tv[t]);
                break;
            default:
                if (FASTDIV && st_div_wave_in_range(tv, o)) {
                    const float rcp = st_div_rcp(o);
#pragma unroll
                    for (int t = 0; t < N; t++) tv[t] = st_div_inrange(tv[t], o, rcp);
                    break;
                }
#pragma unroll
                for (int t = 0; t < N; t++) tv[t] = __fdiv_rn(tv[t], o);
                break;
        }
    }
}
// A wave-uniform pointer, told to the compiler: it then lives in scalar registers and a load through it takes its
// per-lane part as a 32-bit offset.
template <typename T>
__device__ __forceinline__ T* st_uptr(T* p)
{
    const unsigned long long v = (unsigned long long)p;
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)v), hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(v >> 32));
    return (T*)(((unsigned long long)hi << 32) | lo);
}

// Host: lowered table + device array pointers -> kernel arguments.
template <typename P>
static inline void st_make_args(const StencilDev& low, const int* dcells, P const* arrays, StencilArgsT<P>* a)
{
    memset(a, 0, sizeof *a);
    a->nrefs = low.nrefs; a->nscal = low.nscal; a->ncell = low.ncell; a->nchain = low.nchain;
    for (int r = 0; r < low.nrefs + low.nscal; r++) {
        const fortis_ref_t& f = r < low.nrefs ? low.refs[r] : low.scal[r - low.nrefs];
        StSlotT<P>& s = r < low.nrefs ? a->refs[r] : a->scal[r - low.nrefs];
        s.p = arrays[f.array] + f.base;
        s.si = (int)f.si; s.sj = (int)f.sj;
        s.plane = f.planar ? low.plane[f.array] : 0;
    }
    auto cval = [&](int code) { return (code >= 16 && code < 32) ? low.consts[code - 16] : 0.f; };
    for (int n = 0; n < low.ncell; n++) {
        StIns i = { low.cell[n].op, low.cell[n].a, low.cell[n].b, cval(low.cell[n].a), cval(low.cell[n].b) };
        a->cell[n] = i;
    }
    for (int n = 0; n < low.nchain; n++) {
        StStep s = { low.chain[n].op, low.chain[n].code, low.chain[n].tv_left, cval(low.chain[n].code) };
        a->chain[n] = s;
    }
    // unused table entries repeat slot 0, so that a kernel may load through any of them without a clamp
    for (int r = low.nrefs; r < ST_KREFS; r++) a->refs[r] = a->refs[0];
    for (int r = low.nscal; r < ST_SCAL_MAX; r++) a->scal[r] = a->refs[0];
    a->count = (unsigned)low.count;
    a->ilo = low.ilo; a->jlo = low.jlo; a->ni = low.ni; a->sx = low.sx;
    a->cells = dcells;
    a->mcount = st_magic((unsigned)low.count);
    a->mni = st_magic((unsigned)(low.ni > 0 ? low.ni : 1));
    a->msx = st_magic((unsigned)(low.sx > 0 ? low.sx : 1));
    a->uniform = 1;
    for (int r = 0; r < low.nrefs; r++)
        if (a->refs[r].si != a->refs[0].si || a->refs[r].sj != a->refs[0].sj || a->refs[r].plane != a->refs[0].plane) a->uniform = 0;
    a->refs_uniform = a->uniform;
    for (int r = 0; r < low.nscal; r++)
        if (a->scal[r].si != a->refs[0].si || a->scal[r].sj != a->refs[0].sj || a->scal[r].plane != a->refs[0].plane) a->uniform = 0;
}
