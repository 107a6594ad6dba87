// Stencil gather / scatter between the host's Fortran arrays and the batch-major model
// input / output, driven by tables instead of generated source.
//
// Reference: the generator driver/fortis_gather_emit.py and its checked-in output
// mom6_zb/gather.cu (gather kernel :14-49, host wrapper :50-57, scatter kernel :58-81, wrapper
// :82-91).  Index arithmetic is integer-exact; slot values go through the lifted expressions in
// explicit round-to-nearest fp32 with no contraction (the reference builds with -fmad=false).
//
// Kernel mapping on CDNA4 (differs from the reference's one-thread-per-row store pattern):
//   gather : thread = row for the loads (consecutive lanes -> consecutive i, coalesced plane
//            reads), results staged in LDS and written out as one contiguous, fully coalesced
//            block of 256 x n floats (a row-per-thread store would touch n cache lines per lane).
//   scatter: thread = cell; Y rows staged through LDS the same way in reverse; plane stores
//            are coalesced along i.
#include <vector>
#include "stencil_dev.h"

#define ST_THREADS 256
typedef float st_v4f __attribute__((ext_vector_type(4)));

// NQ: slots a thread loads and evaluates (the table's slot count rounded up to a size that is compiled; entries
// past the table's own repeat slot 0 and are not stored).
template <int NQ>
__global__ __launch_bounds__(ST_THREADS) void gather_kernel(GatherArgs args, float* __restrict__ X, unsigned rows)
{
    __shared__ GatherArgs d;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    params_to_lds(&d, ST_THREADS);
    const int n = st_u(d.nrefs);
    const int tid = threadIdx.x;
    // plain workgroup order: this kernel mostly writes, and it writes fastest as ONE contiguous stream.  Banding the
    // workgroups per XCD halves the input fetches but spreads the rows in flight over eight bands (5 % slower); two
    // bands of four vertical strips, in which the workgroup one row down runs on the same XCD a few steps later,
    // fetch each input row once and still measured 5 % slower inside the step (0.463 against 0.440 ms on
    // 1028 x 1028 x 15), no different launched back to back
    const unsigned row0 = blockIdx.x * ST_THREADS, row = row0 + tid;
    if (row < rows) {
        int i, j, kk;
        st_row(d, row, i, j, kk);
        // all slot loads are issued before any of them is consumed
        float tv[NQ];
        StCell cell;
        if (st_u(d.uniform)) {
            // every slot and scalar has the same strides: one element offset per cell, and a slot is its
            // pointer plus that offset (unused table entries repeat slot 0)
            const long off = st_off(d.refs[0], i, j, kk);
#pragma unroll
            // (the pointers straight from the kernel arguments, by literal index: scalar loads, where the copy in LDS
            // costs a vector read and two v_readfirstlane per pointer)
            for (int q = 0; q < NQ; q++) tv[q] = st_g(args.refs[q].p)[off];
#pragma unroll
            for (int sI = 0; sI < ST_SCAL_MAX; sI++) cell.S[sI] = st_g(args.scal[sI].p)[off];
            st_cell_program(d, cell);
        } else {
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                const StSlotT<const float*> sl = d.refs[q < n ? q : 0];
                tv[q] = st_g(sl.p)[st_off(sl, i, j, kk)];
            }
            st_prepare(d, i, j, kk, cell);
        }
        st_chain_apply(d, cell, tv);
#pragma unroll
        for (int q = 0; q < NQ; q++)
            if (q < n) lds[tid * n + q] = tv[q];
    }
    __syncthreads();
    const unsigned lim = (rows - row0 < ST_THREADS ? rows - row0 : ST_THREADS) * n;
    float* out = X + (size_t)row0 * n;
    // the block's rows are one contiguous run of X, which starts on a 16-byte boundary when X does (256 rows
    // of n floats each): written as 16-byte vectors, the last few floats of a ragged block one by one.  X is
    // written once and read by another kernel: the stores are marked non-temporal.
    if (((uintptr_t)X & 15) == 0) {
        const unsigned lim4 = lim / 4;
        for (unsigned idx = tid; idx < lim4; idx += ST_THREADS) __builtin_nontemporal_store(((const st_v4f*)lds)[idx], (st_v4f*)out + idx);
        for (unsigned idx = lim4 * 4 + tid; idx < lim; idx += ST_THREADS) out[idx] = lds[idx];
    } else {
        for (unsigned idx = tid; idx < lim; idx += ST_THREADS) out[idx] = lds[idx];
    }
}

// A workgroup takes SC_TILES consecutive tiles of 256 cells (the table's copy into LDS is paid once for all of them).
#define SC_TILES 4
__global__ __launch_bounds__(ST_THREADS) void scatter_kernel(ScatterArgs args, const float* __restrict__ Y, int kk)
{
    __shared__ ScatterArgs d;
    extern __shared__ __attribute__((aligned(16))) float lds[];
    params_to_lds(&d, ST_THREADS);
    const int n = st_u(d.nrefs);
    const int tid = threadIdx.x;
    kk += blockIdx.y;                                         // gridDim.y > 1: one enclosing-loop iteration per y
    for (int tile = 0; tile < SC_TILES; tile++) {
        const unsigned col0 = (blockIdx.x * SC_TILES + tile) * ST_THREADS, col = col0 + tid;
        if (col0 >= d.count) break;
        const unsigned lim = (d.count - col0 < ST_THREADS ? d.count - col0 : ST_THREADS) * n;
        const float* in = Y + ((size_t)blockIdx.y * d.count + col0) * n;
        // the cell's own reads are issued before Y is staged, so that both are in flight together (0.135 -> 0.129 ms
        // for the 1028 x 1028 x 15 scatter; staging all four tiles before one barrier instead measured 0.162 ms)
        int i = 0, j = 0;
        StCell cell;
        if (col < d.count) { st_cell(d, col, i, j); st_prepare(d, i, j, kk, cell); }
        if (tile) __syncthreads();                            // the tile before has been read out of LDS
        if (((uintptr_t)in & 15) == 0) {
            const unsigned lim4 = lim / 4;
            for (unsigned idx = tid; idx < lim4; idx += ST_THREADS) ((st_v4f*)lds)[idx] = __builtin_nontemporal_load((const st_v4f*)in + idx);   // Y is read once
            for (unsigned idx = lim4 * 4 + tid; idx < lim; idx += ST_THREADS) lds[idx] = in[idx];
        } else {
            for (unsigned idx = tid; idx < lim; idx += ST_THREADS) lds[idx] = in[idx];
        }
        __syncthreads();
        if (col >= d.count) continue;
        // outputs are few (one per model output); handled eight at a time
        for (int q0 = 0; q0 < n; q0 += 8) {
            float tv[8];
#pragma unroll
            for (int t = 0; t < 8; t++) tv[t] = q0 + t < n ? lds[tid * n + q0 + t] : 0.f;
            st_chain_apply(d, cell, tv);
#pragma unroll
            for (int t = 0; t < 8; t++)
                if (q0 + t < n) {
                    const StSlotT<float*> sl = d.refs[q0 + t];
                    __builtin_nontemporal_store(tv[t], st_g(sl.p) + st_off(sl, i, j, kk));     // written once, read by the host's next phase
                }
        }
    }
}

// All enclosing-loop iterations of a thin table (at most four outputs per cell) in one pass over the cells: a lane keeps
// its cell and walks the layers, SC_LB of them at a time with all their reads (the cell's slice of Y straight from
// global memory, its same-cell scalars) in flight before the first result is stored.  The cell list is read once
// instead of once per layer and no barrier separates the lanes.
#define SC_LB 5
template <int N>
__global__ __launch_bounds__(ST_THREADS) void scatter_layers_kernel(ScatterArgs args, const float* __restrict__ Y, int layers)
{
    __shared__ ScatterArgs d;
    params_to_lds(&d, ST_THREADS);
    const unsigned col = blockIdx.x * ST_THREADS + threadIdx.x;
    if (col >= d.count) return;
    int i, j;
    st_cell(d, col, i, j);
    for (int l0 = 0; l0 < layers; l0 += SC_LB) {
        StCell cell[SC_LB];
        float tv[SC_LB][8];
#pragma unroll
        for (int u = 0; u < SC_LB; u++) {
            const int l = l0 + u < layers ? l0 + u : layers - 1;
            const float* in = Y + ((size_t)l * d.count + col) * N;
#pragma unroll
            for (int q = 0; q < 8; q++) tv[u][q] = q < N ? __builtin_nontemporal_load(in + q) : 0.f;    // Y is read once
            st_prepare(d, i, j, l, cell[u]);
        }
#pragma unroll
        for (int u = 0; u < SC_LB; u++) {
            if (l0 + u >= layers) break;
            st_chain_apply(d, cell[u], tv[u]);
#pragma unroll
            for (int q = 0; q < N; q++) {
                const StSlotT<float*> sl = d.refs[q];
                __builtin_nontemporal_store(tv[u][q], st_g(sl.p) + st_off(sl, i, j, l0 + u));
            }
        }
    }
}

// ---- lowering: straight-line program -> per-cell code + tv chain -----------------------------
static bool g_lower_quiet = false;     // set while a table is only being tried for the fused kernels
#define LOWER_ERR(...) do { if (!g_lower_quiet) fprintf(stderr, __VA_ARGS__); } while (0)
int fortis_stencil_lower(const fortis_stencil_t* in, StencilDev* out)
{
    memset(out, 0, sizeof *out);
    if (in->narrays < 1 || in->narrays > FORTIS_MAX_ARRAYS || in->nrefs < 1 || in->nrefs > ST_KREFS ||
        in->nscal < 0 || in->nscal > ST_SCAL_MAX || in->nins < 0 || in->nins > FORTIS_MAX_INS ||
        in->nconst < 0 || in->nconst > FORTIS_MAX_CONST || in->count < 1 || in->nk < 1 ||
        in->count * in->nk >= 4294967295L / ST_KREFS) {
        LOWER_ERR("fortis: stencil table out of range\n");
        return -1;
    }
    out->narrays = in->narrays;
    for (int a = 0; a < in->narrays; a++) out->plane[a] = in->plane[a];
    out->nrefs = in->nrefs;
    out->nscal = in->nscal;
    for (int r = 0; r < in->nrefs; r++) out->refs[r] = in->refs[r];
    for (int r = 0; r < in->nscal; r++) out->scal[r] = in->scal[r];
    for (int r = 0; r < in->nrefs + in->nscal; r++) {
        const fortis_ref_t& f = r < in->nrefs ? in->refs[r] : in->scal[r - in->nrefs];
        if (f.array < 0 || f.array >= in->narrays) { LOWER_ERR("fortis: stencil ref names array %d\n", f.array); return -1; }
        if (f.si > 2147483647L || f.sj > 2147483647L || f.si < -2147483647L || f.sj < -2147483647L) { LOWER_ERR("fortis: stencil stride out of range\n"); return -1; }
    }
    for (int c = 0; c < in->nconst; c++) out->consts[c] = in->consts[c];
    out->count = in->count; out->nk = in->nk;
    out->ilo = in->ilo; out->jlo = in->jlo; out->ni = in->ni > 0 ? in->ni : 1; out->sx = in->sx > 0 ? in->sx : 1;
    out->cells = nullptr;
    // dep[n]: instruction n depends on tv; map[n]: its index in the per-cell program otherwise
    int dep[FORTIS_MAX_INS], map[FORTIS_MAX_INS], last_dep = -1;
    for (int n = 0; n < in->nins; n++) {
        const fortis_ins_t& I = in->ins[n];
        int codes[2] = { I.a, I.b }, isdep[2], lowered[2];
        for (int s = 0; s < 2; s++) {
            const int c = codes[s];
            bool ok = c == 0 || (c >= 1 && c <= in->nscal) || (c >= 16 && c < 16 + in->nconst) || (c >= 32 && c < 32 + n);
            if (!ok || I.op < 0 || I.op > 3) { LOWER_ERR("fortis: bad stencil instruction %d\n", n); return -1; }
            if (c == 0) { isdep[s] = 1; lowered[s] = 0; if (last_dep >= 0) { LOWER_ERR("fortis: stencil expression re-reads the slot value after transforming it\n"); return -1; } }
            else if (c >= 32 && dep[c - 32]) { isdep[s] = 1; lowered[s] = 0; if (c - 32 != last_dep) { LOWER_ERR("fortis: stencil expression is not a single chain on the slot value\n"); return -1; } }
            else { isdep[s] = 0; lowered[s] = c >= 32 ? 32 + map[c - 32] : c; }
        }
        if (isdep[0] && isdep[1]) { LOWER_ERR("fortis: stencil expression combines the slot value with itself\n"); return -1; }
        if (isdep[0] || isdep[1]) {
            dep[n] = 1; map[n] = -1; last_dep = n;
            CellStep st = { I.op, isdep[0] ? lowered[1] : lowered[0], isdep[0] ? 1 : 0 };
            if (out->nchain == ST_CHAIN_MAX) { LOWER_ERR("fortis: stencil expression chains more than %d operations on the slot value\n", ST_CHAIN_MAX); return -1; }
            out->chain[out->nchain++] = st;
        } else {
            dep[n] = 0; map[n] = out->ncell;
            if (out->ncell == ST_CELL_MAX) { LOWER_ERR("fortis: more than %d per-cell stencil instructions\n", ST_CELL_MAX); return -1; }
            fortis_ins_t ci = { I.op, lowered[0], lowered[1] };
            out->cell[out->ncell++] = ci;
        }
    }
    if (in->nins > 0 && last_dep != in->nins - 1 && last_dep >= 0) {
        LOWER_ERR("fortis: the last stencil instruction must produce the slot value\n");
        return -1;
    }
    if (in->nins > 0 && last_dep < 0) { LOWER_ERR("fortis: stencil expressions never use the slot value\n"); return -1; }
    return 0;
}

// ---- device copies of tables -----------------------------------------------------------------
// 0: the table runs in the fused-form kernels (lowered into *low), 1: it takes the general kernels, -1: invalid.
static int route_table(const fortis_stencil_t* t, StencilDev* low)
{
    if (fortis_stencil_validate(t) != 0) return -1;
    if (fortis_stencil_typed(t)) return 1;
    g_lower_quiet = true;
    const int rc = fortis_stencil_lower(t, low);
    g_lower_quiet = false;
    return rc == 0 ? 0 : 1;
}
static inline size_t esz_of(const fortis_stencil_t& t, int a) { return t.elt[a] == 8 ? 8 : 4; }

struct BoundStencil {
    bool ok = false;
    bool generic = false;        // the table takes the general kernels
    fortis_stencil_t host;       // as configured (cells pointer not owned)
    StencilDev low;              // lowered table
    int* dcells = nullptr;       // device copy of the cell list
    void* darr[FORTIS_MAX_ARRAYS] = {};       // planes of the host arrays: device memory (gather) or page-locked host memory (scatter)
    void* dblock = nullptr;                   // gather: the one device allocation darr[] points into
    bool host_planes = false;
    // scatter under loop distribution: all iterations computed at the first call of a step (see fortis_scatter_v)
    StencilDev low_all;                       // the table with a plane per iteration for every written array
    void* sall[FORTIS_MAX_ARRAYS] = {};       // page-locked planes for all iterations
    bool spec_ready = false;
    long spec_gen = -1;
    const void* reg[FORTIS_MAX_ARRAYS] = {};  // last host address seen per array
    bool written[FORTIS_MAX_ARRAYS] = {};
    bool init = false;
};
static BoundStencil g_gather, g_scatter;

// Device copies of cell lists, shared by content: the gather and the scatter table of one step name the same
// cells, and with ONE device copy behind both the fused kernel sees equal list pointers and decodes a row once.
struct CellList { unsigned long long hash; long count; int* d; int users; };
static CellList g_lists[32];
static unsigned long long cells_hash(const int* c, long n)
{
    unsigned long long h = 1469598103934665603ULL;
    for (long i = 0; i < n; i++) { h ^= (unsigned)c[i]; h *= 1099511628211ULL; }
    return h;
}
static int* cells_acquire(const int* host, long count)
{
    const unsigned long long h = cells_hash(host, count);
    CellList* slot = nullptr;
    std::vector<int> tmp;
    for (CellList& l : g_lists) {
        if (!l.d) { if (!slot) slot = &l; continue; }
        if (l.hash != h || l.count != count) continue;
        // same hash: compare the contents before sharing
        if (tmp.empty()) tmp.resize((size_t)count);
        if (hipMemcpy(tmp.data(), l.d, (size_t)count * sizeof(int), hipMemcpyDeviceToHost) == hipSuccess &&
            !memcmp(tmp.data(), host, (size_t)count * sizeof(int))) { l.users++; return l.d; }
        (void)hipGetLastError();
    }
    int* d = nullptr;
    if (fortis_dev_malloc((void**)&d, (size_t)count * sizeof(int), "stencil cell list") != 0) return nullptr;
    if (hipMemcpy(d, host, (size_t)count * sizeof(int), hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        fprintf(stderr, "fortis: copying the stencil cell list to the device failed\n");
        fortis_dev_free(d);
        return nullptr;
    }
    if (slot) { slot->hash = h; slot->count = count; slot->d = d; slot->users = 1; }   // no free slot: an unshared copy
    return d;
}
static void cells_release(int* d)
{
    if (!d) return;
    for (CellList& l : g_lists)
        if (l.d == d) {
            if (--l.users > 0) return;
            l.d = nullptr;
            break;
        }
    fortis_dev_free(d);
}

// Returns the table's route (see route_table) after copying its cell list to the device; -1 also when the
// list found no device memory (nothing may then be launched on the table).
static int upload_table(const fortis_stencil_t* t, StencilDev* low, int** dcells)
{
    const int route = route_table(t, low);
    if (route < 0) return -1;
    if (t->cells) {
        *dcells = cells_acquire(t->cells, t->count);
        if (!*dcells) return -1;
        if (route == 0) low->cells = *dcells;
    }
    return route;
}

static void release(BoundStencil& b)
{
    cells_release(b.dcells);
    if (b.dblock) fortis_dev_free(b.dblock);                    // the gather's planes: one allocation
    else
        for (int a = 0; a < FORTIS_MAX_ARRAYS; a++)
            if (b.darr[a]) { if (b.host_planes) HIP_OK(hipHostFree(b.darr[a])); else fortis_dev_free(b.darr[a]); }
    for (int a = 0; a < FORTIS_MAX_ARRAYS; a++) if (b.sall[a]) HIP_OK(hipHostFree(b.sall[a]));
    b = BoundStencil();
}

static int config(BoundStencil& b, const fortis_stencil_t* t, bool is_scatter)
{
    release(b);
    const int route = upload_table(t, &b.low, &b.dcells);
    if (route < 0) return -1;
    b.generic = route == 1;
    b.host = *t;
    b.host.cells = nullptr;
    if (is_scatter) for (int r = 0; r < t->nrefs; r++) b.written[t->refs[r].array] = true;
    if (is_scatter && !b.generic) {
        fortis_stencil_t all = *t;
        for (int r = 0; r < all.nrefs; r++)
            if (!all.refs[r].planar) { all.refs[r].planar = 1; all.plane[all.refs[r].array] = all.total[all.refs[r].array]; }
        if (fortis_stencil_lower(&all, &b.low_all) != 0) return -1;
        b.low_all.cells = b.low.cells;
    }
    b.ok = true;
    return 0;
}

void fortis_stencil_reset_internal()
{
    release(g_gather);
    release(g_scatter);
}

// cache of device tables for the device-resident API (keyed by table contents)
// A table with a cell list is matched by the list too: a caller may free a list and build another at the same
// address.  A host copy of the list is kept; a call with the same address and count as the entry's last match is
// checked by a fingerprint (first, last and 1022 evenly spaced entries: constant cost, a few microseconds), any other
// by a full compare (0.3 MB for the 71,040 cells of the ZB step, 63 MB for a 15.7 M-cell list).  A list rewritten in
// place that keeps its address, its count and every sampled entry is therefore taken for the old one.
struct CacheEnt { fortis_stencil_t key; std::vector<int> cells_key; const int* cells_addr; int* dcells; StencilDev low; bool generic; };
static CacheEnt g_cache[16];
static int g_ncache = 0;
static bool cells_fingerprint_equal(const int* a, const int* b, long n)
{
    if (n <= 1024) return !memcmp(a, b, (size_t)n * sizeof(int));
    for (long k = 0; k < 1023; k++) { const long i = k * (n - 1) / 1023; if (a[i] != b[i]) return false; }
    return a[n - 1] == b[n - 1];
}
static CacheEnt* cached(const fortis_stencil_t* t)
{
    for (int i = 0; i < g_ncache; i++) {
        fortis_stencil_t a = g_cache[i].key, b = *t;
        a.cells = b.cells = nullptr;
        if (memcmp(&a, &b, sizeof a) || (t->cells != nullptr) != !g_cache[i].cells_key.empty()) continue;
        if (!t->cells) return &g_cache[i];
        const int* key = g_cache[i].cells_key.data();
        if (t->cells == g_cache[i].cells_addr ? cells_fingerprint_equal(key, t->cells, t->count)
                                               : !memcmp(key, t->cells, (size_t)t->count * sizeof(int))) {
            g_cache[i].cells_addr = t->cells;
            return &g_cache[i];
        }
    }
    CacheEnt* e;
    const bool evict = g_ncache == 16;
    if (evict) {
        // full: the oldest entry is replaced in place (once nothing in flight can still read its cell list)
        static int victim = 0;
        e = &g_cache[victim];
        victim = (victim + 1) % 16;
        HIP_OK(hipStreamSynchronize(fortis_stream_get()));
        cells_release(e->dcells);
        e->key.narrays = -1;            // matches no table until it is filled again
    } else {
        e = &g_cache[g_ncache];
    }
    e->dcells = nullptr;
    const int route = upload_table(t, &e->low, &e->dcells);
    if (route < 0) return nullptr;
    e->generic = route == 1;
    e->key = *t;
    e->cells_key.clear();
    if (t->cells) e->cells_key.assign(t->cells, t->cells + t->count);
    e->cells_addr = t->cells;
    if (!evict) g_ncache++;
    return e;
}

static void launch_gather(const StencilDev& low, const float* const* dA, float* dX, hipStream_t s)
{
    GatherArgs a;
    st_make_args<const float*>(low, low.cells, dA, &a);
    const unsigned rows = (unsigned)(low.count * low.nk);
    const dim3 grid((unsigned)cdiv(rows, ST_THREADS)), block(ST_THREADS);
    const size_t shmem = (size_t)ST_THREADS * low.nrefs * sizeof(float);
    if (low.nrefs <= 8) hipLaunchKernelGGL(gather_kernel<8>, grid, block, shmem, s, a, dX, rows);
    else if (low.nrefs <= 16) hipLaunchKernelGGL(gather_kernel<16>, grid, block, shmem, s, a, dX, rows);
    else if (low.nrefs <= 24) hipLaunchKernelGGL(gather_kernel<24>, grid, block, shmem, s, a, dX, rows);
    else if (low.nrefs <= 28) hipLaunchKernelGGL(gather_kernel<28>, grid, block, shmem, s, a, dX, rows);
    else hipLaunchKernelGGL(gather_kernel<32>, grid, block, shmem, s, a, dX, rows);
    HIP_OK(hipGetLastError());
}
static void launch_scatter(const StencilDev& low, float* const* dA, const float* dY, int kk, hipStream_t s, int layers = 1)
{
    ScatterArgs a;
    st_make_args<float*>(low, low.cells, dA, &a);
    static const bool by_layers = !(getenv("FORTIS_SCATTER_LAYERS") && atoi(getenv("FORTIS_SCATTER_LAYERS")) == 0);
    if (by_layers && layers > 1 && kk == 0 && low.nrefs <= 4) {
        const dim3 grid((unsigned)cdiv(low.count, ST_THREADS)), block(ST_THREADS);
        switch (low.nrefs) {
        case 1: hipLaunchKernelGGL(scatter_layers_kernel<1>, grid, block, 0, s, a, dY, layers); break;
        case 2: hipLaunchKernelGGL(scatter_layers_kernel<2>, grid, block, 0, s, a, dY, layers); break;
        case 3: hipLaunchKernelGGL(scatter_layers_kernel<3>, grid, block, 0, s, a, dY, layers); break;
        default: hipLaunchKernelGGL(scatter_layers_kernel<4>, grid, block, 0, s, a, dY, layers); break;
        }
        HIP_OK(hipGetLastError());
        return;
    }
    hipLaunchKernelGGL(scatter_kernel, dim3((unsigned)cdiv(low.count, ST_THREADS * SC_TILES), (unsigned)layers), dim3(ST_THREADS),
                       (size_t)ST_THREADS * low.nrefs * sizeof(float), s, a, dY, kk);
    HIP_OK(hipGetLastError());
}

void fortis_launch_chain_stencil(const ChainDesc& d, const StencilDev& g, const StencilDev& sc, long rows,
                                 const float* const* dG, float* const* dS, float* dY, hipStream_t s);
// plan.hip: describes the plan as a chain if it is one
int fortis_plan_as_chain(fortis_plan* p, ChainDesc* out);

extern "C" {

int fortis_stencil_check(const fortis_stencil_t* t)
{
    StencilDev tmp;
    return t && route_table(t, &tmp) >= 0 ? 0 : -1;
}
// Test hook: 0 if the table runs in the fused-form kernels, 1 if it takes the general ones, -1 if invalid.
int fortis_stencil_route(const fortis_stencil_t* t)
{
    StencilDev tmp;
    return t ? route_table(t, &tmp) : -1;
}
int fortis_gather_config(const fortis_stencil_t* g) { return config(g_gather, g, false); }
int fortis_scatter_config(const fortis_stencil_t* s) { return config(g_scatter, s, true); }

// A host array whose address changes between calls is a temporary: forget it once and never treat
// it as program-scope again (driver/fortis_gather_emit.py:41-44).  Host memory is staged with plain
// stream-ordered copies; existing host memory is never page-locked by this library.
static void note_host(BoundStencil& b, int a, const void* H)
{
    if (b.reg[a] && b.reg[a] != H) b.reg[a] = (const void*)1;
    else if (!b.reg[a]) b.reg[a] = H;
}

void fortis_gather_v(const int* a, const void* const* H)
{
    BoundStencil& b = g_gather;
    if (!b.ok) { fprintf(stderr, "fortis_gather: no gather table configured\n"); return; }
    hipStream_t s = fortis_stream_get();
    const fortis_stencil_t& t = b.host;
    const bool kdist = t.nk > 1;
    if (!b.init) {
        // gather.cu:8-11 allocates a buffer per array; here the arrays' planes sit one behind the other in ONE
        // allocation: a set of planes that fits the memory-side cache stays in it from step to step only if its
        // lines spread evenly over the cache's sets, which consecutive addresses do.
        size_t off[FORTIS_MAX_ARRAYS + 1] = {0};
        for (int ai = 0; ai < t.narrays; ai++)
            off[ai + 1] = off[ai] + (((size_t)t.plane[ai] * t.nk * esz_of(t, ai) + 255) & ~(size_t)255);
        if (fortis_dev_malloc(&b.dblock, off[t.narrays], "gather planes") != 0) return;
        for (int ai = 0; ai < t.narrays; ai++) b.darr[ai] = (char*)b.dblock + off[ai];
        b.init = true;
    }
    const float* dptr[FORTIS_MAX_ARRAYS];
    for (int ai = 0; ai < t.narrays; ai++) {
        note_host(b, ai, H[ai]);
        // under loop distribution all nk planes starting at klo; otherwise the plane of the
        // current enclosing-loop index (gather.cu:52-55; gather_emit.py:66-68)
        long off = 0;
        const bool planar3d = t.total[ai] > t.plane[ai];
        if (planar3d) off = kdist ? (long)(t.klo - 1) * t.plane[ai] : (long)((a ? a[0] : 1) - 1) * t.plane[ai];
        const long nelem = (kdist && planar3d) ? t.plane[ai] * t.nk : t.plane[ai];
        HIP_OK(hipMemcpyAsync(b.darr[ai], (const char*)H[ai] + off * esz_of(t, ai), nelem * esz_of(t, ai), hipMemcpyHostToDevice, s));
        dptr[ai] = (const float*)b.darr[ai];
    }
    if (b.generic) {
        fortis_launch_gather_generic(t, b.dcells, (const void* const*)dptr, (float*)fortis_model_input(), s);
    } else {
        launch_gather(b.low, dptr, (float*)fortis_model_input(), s);
    }
}

void fortis_scatter_v(const int* a, void* const* H)
{
    BoundStencil& b = g_scatter;
    if (!b.ok) { fprintf(stderr, "fortis_scatter: no scatter table configured\n"); return; }
    hipStream_t s = fortis_stream_get();
    const fortis_stencil_t& t = b.host;
    // One page-locked host plane per array, which the kernel reads and writes directly over the bus: the
    // scalars' planes are copied in by the CPU, the visited cells of the written planes are copied out by
    // the CPU after the one synchronisation.  The reference issues two uploads and three pitched downloads
    // per call (gather.cu:84-90); as copy commands from and to pageable memory those cost far more than the
    // kernel here (a pitched download is handled row by row).
    if (!b.init) {
        b.host_planes = true;
        for (int ai = 0; ai < t.narrays; ai++)
            if (!b.darr[ai] && hipHostMalloc(&b.darr[ai], (size_t)t.plane[ai] * esz_of(t, ai), hipHostMallocDefault) != hipSuccess) {
                (void)hipGetLastError();
                b.darr[ai] = nullptr;
                fprintf(stderr, "fortis_scatter: no page-locked memory for the staging planes\n");
                return;
            }
        b.init = true;
    }
    const int k1 = a ? a[0] : 1;   // 1-based enclosing-loop index
    bool whole_plane[FORTIS_MAX_ARRAYS] = {};
    for (int r = 0; r < t.nrefs; r++)
        if (t.cells || t.refs[r].si != 1) whole_plane[t.refs[r].array] = true;
    for (int ai = 0; ai < t.narrays; ai++) note_host(b, ai, H[ai]);
    bool rects = true;
    for (int ai = 0; ai < t.narrays; ai++) if (whole_plane[ai]) rects = false;
    // Under loop distribution the model output of every iteration is already on the device when the first
    // scatter of a step arrives.  That call therefore scatters ALL iterations in one launch, reading the
    // scalars' planes of every iteration as the host holds them at that moment; a later call of the same step
    // compares its iteration's scalar planes with what was read then and, if they are the same bytes (the
    // normal case: they were inputs of the gather too), only copies its rows out -- no launch and no
    // synchronisation.  Any difference, or a new forward pass in between, takes the one-iteration path below.
    if (t.nk > 1 && rects && !b.generic && !getenv("FORTIS_SCATTER_PER_CALL")) {
        const int idx = k1 - t.klo;
        const long gen = fortis_step_generation();
        auto planes = [&](int ai) { return (t.total[ai] > t.plane[ai] || b.written[ai]) ? (long)t.nk : 1L; };
        auto pelems = [&](int ai) { return b.written[ai] && t.total[ai] <= t.plane[ai] ? t.total[ai] : t.plane[ai]; };
        if (idx == 0) {
            float* sp[FORTIS_MAX_ARRAYS];
            for (int ai = 0; ai < t.narrays; ai++) {
                if (!b.sall[ai] && hipHostMalloc(&b.sall[ai], (size_t)planes(ai) * pelems(ai) * sizeof(float), hipHostMallocDefault) != hipSuccess) {
                    (void)hipGetLastError();
                    b.sall[ai] = nullptr;
                    fprintf(stderr, "fortis_scatter: no page-locked memory for the staging planes\n");
                    return;
                }
                sp[ai] = (float*)b.sall[ai];
                if (!b.written[ai]) {
                    const long off = t.total[ai] > t.plane[ai] ? (long)(t.klo - 1) * t.plane[ai] : 0;
                    memcpy(b.sall[ai], (const float*)H[ai] + off, (size_t)planes(ai) * pelems(ai) * sizeof(float));
                }
            }
            launch_scatter(b.low_all, sp, (const float*)fortis_model_output(), 0, s, t.nk);
            HIP_OK(hipStreamSynchronize(s));
            b.spec_ready = true;
            b.spec_gen = gen;
        }
        if (b.spec_ready && b.spec_gen == gen && idx >= 0 && idx < t.nk) {
            bool same = true;
            for (int ai = 0; ai < t.narrays && same; ai++) {
                if (b.written[ai]) continue;
                const bool p3 = t.total[ai] > t.plane[ai];
                const float* hp = (const float*)H[ai] + (p3 ? (long)(k1 - 1) * t.plane[ai] : 0);
                const float* sp = (const float*)b.sall[ai] + (p3 ? (long)idx * t.plane[ai] : 0);
                same = memcmp(hp, sp, (size_t)t.plane[ai] * sizeof(float)) == 0;
            }
            if (same) {
                for (int r = 0; r < t.nrefs; r++) {
                    const int ai = t.refs[r].array;
                    const long off = t.total[ai] > t.plane[ai] ? (long)(k1 - 1) * t.plane[ai] : 0;
                    float* hbase = (float*)H[ai] + off;
                    const float* stage = (const float*)b.sall[ai] + (long)idx * pelems(ai);
                    const long rect = t.refs[r].base + (long)t.ilo * t.refs[r].si + (long)t.jlo * t.refs[r].sj;
                    const long pitch = t.refs[r].sj > 0 ? t.refs[r].sj : t.ni;
                    const long nrow = t.nj > 0 ? t.nj : t.count / t.ni;
                    for (long j = 0; j < nrow; j++) memcpy(hbase + rect + j * pitch, stage + rect + j * pitch, (size_t)t.ni * sizeof(float));
                }
                return;
            }
        }
    }
    float* dptr[FORTIS_MAX_ARRAYS];
    for (int ai = 0; ai < t.narrays; ai++) {
        dptr[ai] = (float*)b.darr[ai];
        // inputs always; a written array only when its whole plane goes back (unvisited cells must survive)
        if (!b.written[ai] || whole_plane[ai]) {
            const long off = t.total[ai] > t.plane[ai] ? (long)(k1 - 1) * t.plane[ai] : 0;
            memcpy(b.darr[ai], (const char*)H[ai] + off * esz_of(t, ai), t.plane[ai] * esz_of(t, ai));
        }
    }
    // the staging holds ONE plane per array, so the kernel runs with plane index 0
    const long yoff = t.nk > 1 ? (long)(k1 - t.klo) * t.count * t.nrefs : 0;   // gather.cu:86
    if (b.generic) fortis_launch_scatter_generic(t, b.dcells, (void* const*)dptr, (const float*)fortis_model_output() + yoff, 0, s);
    else launch_scatter(b.low, dptr, (const float*)fortis_model_output() + yoff, 0, s);
    HIP_OK(hipStreamSynchronize(s));
    for (int r = 0; r < t.nrefs; r++) {
        const int ai = t.refs[r].array;
        const size_t es = esz_of(t, ai);
        const long off = t.total[ai] > t.plane[ai] ? (long)(k1 - 1) * t.plane[ai] : 0;
        char* hbase = (char*)H[ai] + off * es;
        const char* stage = (const char*)b.darr[ai];
        if (whole_plane[ai]) {
            // cell list or non-unit inner stride: no rectangle to copy, return the whole plane
            memcpy(hbase, stage, t.plane[ai] * es);
        } else {
            // visited rectangle, pitch = stride of the j index (gather.cu:87-89; gather_emit.py:88-95)
            const long rect = t.refs[r].base + (long)t.ilo * t.refs[r].si + (long)t.jlo * t.refs[r].sj;
            const long pitch = t.refs[r].sj > 0 ? t.refs[r].sj : t.ni;
            const long nrow = t.nj > 0 ? t.nj : t.count / t.ni;
            for (long j = 0; j < nrow; j++) memcpy(hbase + (rect + j * pitch) * es, stage + (rect + j * pitch) * es, (size_t)t.ni * es);
        }
    }
}

void fortis_gather(const float* H0, const float* H1, const float* H2, const float* H3)
{
    const void* H[4] = { H0, H1, H2, H3 };
    fortis_gather_v(nullptr, H);
}
void fortis_scatter(int a0, float* H0, float* H1, float* H2, float* H3, float* H4)
{
    void* H[5] = { H0, H1, H2, H3, H4 };
    fortis_scatter_v(&a0, H);
}

void fortis_stencil_gather_dev(const fortis_stencil_t* g, const float* const* dA, float* dX)
{
    CacheEnt* e = cached(g);
    if (!e) return;
    if (e->generic) { fortis_launch_gather_generic(*g, e->dcells, (const void* const*)dA, dX, fortis_stream_get()); return; }
    launch_gather(e->low, dA, dX, fortis_stream_get());
}
void fortis_stencil_scatter_dev(const fortis_stencil_t* sd, float* const* dA, const float* dY, int kk)
{
    CacheEnt* e = cached(sd);
    if (!e) return;
    if (e->generic) { fortis_launch_scatter_generic(*sd, e->dcells, (void* const*)dA, dY, kk, fortis_stream_get()); return; }
    launch_scatter(e->low, dA, dY, kk, fortis_stream_get());
}

// Every enclosing-loop iteration in one launch (the entry path's scatter under loop distribution, mom6_zb/kdist.json):
// dY holds the model output of all nk iterations, and an array that is 2-D on the host, which the reference's per-
// iteration launches overwrite nk times, has nk planes on the device, as in fortis_stencil_step_fused.
int fortis_stencil_scatter_all_dev(const fortis_stencil_t* sd, float* const* dA, const float* dY)
{
    if (!sd || !dA || !dY) return -1;
    fortis_stencil_t s2 = *sd;
    for (int r = 0; r < s2.nrefs; r++)
        if (!s2.refs[r].planar) { s2.refs[r].planar = 1; s2.plane[s2.refs[r].array] = s2.total[s2.refs[r].array]; }
    CacheEnt* e = cached(&s2);
    if (!e) return -1;
    if (e->generic) {
        for (int kk = 0; kk < sd->nk; kk++)
            fortis_launch_scatter_generic(s2, e->dcells, (void* const*)dA, dY + (size_t)kk * sd->count * sd->nrefs, kk, fortis_stream_get());
        return 0;
    }
    launch_scatter(e->low, dA, dY, 0, fortis_stream_get(), (int)sd->nk);
    return 0;
}

int fortis_stencil_step_fused(const fortis_stencil_t* g, const fortis_stencil_t* sd, fortis_plan* p,
                              const float* const* dG, float* const* dS, float* dY)
{
    ChainDesc d;
    if (fortis_plan_as_chain(p, &d) != 0) {
        fprintf(stderr, "fortis_stencil_step_fused: the plan is not a narrow MLP chain\n");
        return -1;
    }
    if (d.L[0].K != g->nrefs || d.L[d.nlayers - 1].N != sd->nrefs || g->count != sd->count || g->nk != sd->nk) {
        fprintf(stderr, "fortis_stencil_step_fused: gather/scatter tables do not match the model (%d->%d vs %d->%d)\n",
                g->nrefs, sd->nrefs, d.L[0].K, d.L[d.nlayers - 1].N);
        return -1;
    }
    // Every written array gets a plane per enclosing-loop iteration on the device, also the ones
    // that are 2-D on the host (overwritten each iteration there).
    fortis_stencil_t s2 = *sd;
    for (int r = 0; r < s2.nrefs; r++)
        if (!s2.refs[r].planar) { s2.refs[r].planar = 1; s2.plane[s2.refs[r].array] = s2.total[s2.refs[r].array]; }
    CacheEnt* es = cached(&s2);
    CacheEnt* eg = cached(g);
    if (eg && es && memcmp(&es->key, &s2, offsetof(fortis_stencil_t, cells)) != 0) es = cached(&s2);   // the second lookup replaced the first
    if (!eg || !es) return -1;
    if (eg->generic || es->generic) {
        fprintf(stderr, "fortis_stencil_step_fused: the tables need the general stencil kernels (fp64 arrays, functions or a "
                        "non-chain expression); run gather, model and scatter as separate launches\n");
        return -1;
    }
    fortis_launch_chain_stencil(d, eg->low, es->low, g->count * g->nk, dG, dS, dY, fortis_stream_get());
    return 0;
}


struct FusedArgs { const fortis_stencil_t* g; const fortis_stencil_t* s; fortis_plan* p; const float* const* dG; float* const* dS; float* dY; };
static void fused_cb(void* a)
{
    FusedArgs* f = (FusedArgs*)a;
    fortis_stencil_step_fused(f->g, f->s, f->p, f->dG, f->dS, f->dY);
}
float fortis_stencil_step_fused_time_ms(const fortis_stencil_t* g, const fortis_stencil_t* sd, fortis_plan* p,
                                        const float* const* dG, float* const* dS, float* dY, int iters)
{
    FusedArgs a = { g, sd, p, dG, dS, dY };
    if (fortis_stencil_step_fused(g, sd, p, dG, dS, dY) != 0) return -1.f;   // validates, warms the table cache
    return fortis_time_ms(fused_cb, &a, iters);
}
}  // extern "C"

// Test hook: quotient and remainder of n / d through the multiply-shift the kernels use (host evaluation of
// the same arithmetic as st_divmod).
extern "C" void fortis_magic_divmod(unsigned n, unsigned d, unsigned* q, unsigned* r)
{
    const StMagic m = st_magic(d);
    if (m.one) { *q = n; *r = 0; return; }
    const unsigned long long t = (unsigned long long)n * m.mh + (unsigned)(((unsigned long long)n * m.ml) >> 32);
    *q = (unsigned)(t >> 32);
    *r = n - *q * m.d;
}
