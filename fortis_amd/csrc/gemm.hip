// Fused GEMM + bias + activation on the fp32 matrix cores:
//     C[B][N] = epi(A[B][K] . W[N][K]^T)
// One kernel replaces the reference's cuBLAS SGEMM (runtime/fortis_rt.c:45-75) AND the separate
// epilogue kernel fortis-fuse emits behind it (compiler/FortisFuse.cpp:685-692, 721-760: load C,
// add bias, activation, store), which re-reads and re-writes every activation once per layer.
//
// Tiling for CDNA4 (64-lane waves, v_mfma_f32_32x32x2f32, 4 SIMDs per CU):
//   workgroup tile 128 x 128 (halves and quarters of it at the tail of a launch), 256 threads =
//   4 waves in a 2 x 2 grid, each wave TM x TN MFMA tiles of 32 x 32; k is consumed in slabs of BK
//   staged through LDS, double buffered (global -> registers -> LDS while the previous slab is
//   multiplied).
//   Both operands are k-contiguous in memory (A row-major, W[N][K]), so both are staged the same
//   way, and a lane reads 4 consecutive k as one 16-byte LDS load that feeds 4 MFMAs: MFMA step s
//   of an 8-wide k group uses k = 4h + s for lane half h, identically for A and B.
//   LDS rows are padded by 4 floats so the 16-byte reads of consecutive rows fall in different banks.
#include "common.h"

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));   // native vector: selects and copies stay in registers

#define GM_THREADS 256

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

// Epilogue of a tile with all its rows and nothing but bias and activation: per element one add, the activation
// (MODE 0 none, 1 max(v, 0), 2 max(v, alpha v) for 0 <= alpha <= 1, 3 the general form) and a store to
// uniform row base + one of TM*TN per-lane 32-bit offsets.
template <int TM, int TN, int MODE>
__device__ __forceinline__ void gemm_store_plain(const v16f (&acc)[TM][TN], float* cb, unsigned Nu, const float* bias,
                                                 int wm, int wn, int lr, int lh, int ncols, const GemmEpi& epi)
{
    const float alpha = epi.alpha;
#pragma unroll
    for (int j = 0; j < TN; j++) {
        if (wn + j * 32 + lr >= ncols) continue;                         // column past the end of C
        const float bv = bias ? bias[wn + j * 32 + lr] : 0.f;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            const unsigned off = (unsigned)(wm + i * 32 + 4 * lh) * Nu + (unsigned)(wn + j * 32 + lr);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float v = acc[i][j][r] + bv;
                if (MODE == 1) v = fmaxf(v, 0.f);
                else if (MODE == 2) v = fmaxf(v, alpha * v);
                else if (MODE == 3) v = gemm_act(v, epi.act, alpha);
                float* rb = cb + (size_t)((unsigned)(8 * (r >> 2) + (r & 3)) * Nu);     // uniform row base
                rb[off] = v;
            }
        }
    }
}

// Workgroup barrier that orders LDS traffic only: global loads issued earlier stay in flight across it
// (__syncthreads() would also wait for every outstanding global load).
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// One output tile of (64 TM) x (64 TN) at (m0, n0), by the whole workgroup.
//
// Schedule of one k slab (NKG groups of 8 k, one group = TM*TN*4 MFMAs per wave):
//   top      global loads of the next slab -> staging registers (ra, rw)
//   group g  LDS reads of the fragments of group g+1, then the MFMAs of group g
//   before the last group: staging registers -> other LDS buffer, barrier, LDS reads of the next slab's group 0
// so every LDS read has a whole group of MFMAs to arrive, and the barrier is followed by MFMAs that
// were already fed.  The staging registers belong to the caller: when `preloaded`, they already hold
// this tile's slab 0, and when `has_next`, the last slab's "next slab" is slab 0 of tile (m0n, n0n),
// whose latency then hides behind this tile's epilogue.
template <int TM, int TN, int GM_BK>
__device__ __forceinline__ void gemm_tile(const float* __restrict__ A, const float* __restrict__ W,
                                          float* __restrict__ C, long B, long N, long K,
                                          long m0, long n0, const GemmEpi& epi, float* smem,
                                          v4f (&ra)[TM * GM_BK / 16], v4f (&rw)[TN * GM_BK / 16],
                                          bool preloaded, bool has_next, long m0n, long n0n)
{
    constexpr int BM = 64 * TM, BN = 64 * TN;
    constexpr int GM_LDK = GM_BK + 4;                   // LDS row pitch: +4 floats staggers the banks
    constexpr int F4R = GM_BK / 4;                      // v4f per staged row
    constexpr int LA = TM * GM_BK / 16;                 // v4f loads per thread per slab (A)
    constexpr int LW = TN * GM_BK / 16;
    constexpr int NKG = GM_BK / 8;
    static_assert(NKG % 2 == 0, "fragment sets alternate per k group");
    float* sA = smem;                                   // [2][BM][GM_LDK]
    float* sW = sA + 2 * BM * GM_LDK;                   // [2][BN][GM_LDK]

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

    // staging map: v4f index f = tid + t*256 -> row = f / F4R, kq = f % F4R.
    // A thread's byte offsets inside the tile's rows are fixed for the whole tile (32 bits: rows past
    // the end of A or W are clamped to the last one -- their products land in rows/columns of the tile
    // that are never stored), so a load is uniform base + k0 plus a per-thread 32-bit offset.
    auto offsets = [&](long mt, long nt, unsigned (&oa)[LA], unsigned (&ow)[LW]) __attribute__((always_inline)) {
        const int lastm = (int)(B - 1 - mt < BM - 1 ? B - 1 - mt : BM - 1);
        const int lastn = (int)(N - 1 - nt < BN - 1 ? N - 1 - nt : BN - 1);
#pragma unroll
        for (int t = 0; t < LA; t++) {
            const int f = tid + t * GM_THREADS, row = f / F4R, kq = f % F4R;
            oa[t] = ((unsigned)(row < lastm ? row : lastm) * (unsigned)K + kq * 4) * 4u;
        }
#pragma unroll
        for (int t = 0; t < LW; t++) {
            const int f = tid + t * GM_THREADS, row = f / F4R, kq = f % F4R;
            ow[t] = ((unsigned)(row < lastn ? row : lastn) * (unsigned)K + kq * 4) * 4u;
        }
    };
    // Every staged chunk of a thread sits at the same k inside the slab (GM_THREADS is a multiple of F4R).
    static_assert(GM_THREADS % F4R == 0, "a thread's chunks share their k position");
    const int kq4 = (tid % F4R) * 4;
    // ONE load site and ONE store site per slab, whatever the slab is (a full one, the one that runs past K,
    // slab 0 of the next tile): the compiler otherwise merges the register sets of the different sites with
    // copies placed right behind the loads, and every wave then waits for its loads before it multiplies.
    // A chunk at or beyond K reads the row's chunk 0 instead (a valid address) and is zeroed when stored.
    auto load_slab = [&](const float* Ab, const float* Wb, const unsigned (&oa)[LA], const unsigned (&ow)[LW], long k0) __attribute__((always_inline)) {
        const char* ab = (const char*)(Ab + k0);
        const char* wb = (const char*)(Wb + k0);
#pragma unroll
        for (int t = 0; t < LA; t++) ra[t] = *(const v4f*)(ab + oa[t]);
#pragma unroll
        for (int t = 0; t < LW; t++) rw[t] = *(const v4f*)(wb + ow[t]);
    };
    // Before the load of a slab that runs past K (the last one of a tile, after which these offsets are not
    // used again): chunks at or beyond K are pointed at their row's chunk 0.
    auto clamp_offsets = [&](long k0, unsigned (&oa)[LA], unsigned (&ow)[LW]) __attribute__((always_inline)) {
        if (k0 + GM_BK > K) {
            asm volatile("" ::: "memory");               // stays a branch
            const unsigned adj = k0 + kq4 < K ? 0u : (unsigned)kq4 * 4u;
#pragma unroll
            for (int t = 0; t < LA; t++) oa[t] -= adj;
#pragma unroll
            for (int t = 0; t < LW; t++) ow[t] -= adj;
        }
    };
    // k0: the slab the staging registers hold
    auto store_slab = [&](int buf, long k0) __attribute__((always_inline)) {
        float* a = sA + buf * BM * GM_LDK;
        float* w = sW + buf * BN * GM_LDK;
        if (k0 + GM_BK > K) {
            // only the slab that runs past K comes here; the empty asm keeps this a branch (as a select it
            // would cost every slab one instruction per staged register)
            asm volatile("" ::: "memory");
            if (k0 + kq4 >= K) {
                const v4f zero = (v4f)(0.f);
#pragma unroll
                for (int t = 0; t < LA; t++) ra[t] = zero;
#pragma unroll
                for (int t = 0; t < LW; t++) rw[t] = zero;
            }
        }
#pragma unroll
        for (int t = 0; t < LA; t++) {
            const int f = tid + t * GM_THREADS, row = f / F4R, kq = f % F4R;
            *(v4f*)(a + row * GM_LDK + kq * 4) = ra[t];
        }
#pragma unroll
        for (int t = 0; t < LW; t++) {
            const int f = tid + t * GM_THREADS, row = f / F4R, kq = f % F4R;
            *(v4f*)(w + row * GM_LDK + kq * 4) = rw[t];
        }
    };
    v4f fa[2][TM], fw[2][TN];
    auto read_frag = [&](int set, int buf, int kg) __attribute__((always_inline)) {
        const float* a = sA + buf * BM * GM_LDK + (wm + lr) * GM_LDK + 4 * lh + kg * 8;
        const float* w = sW + buf * BN * GM_LDK + (wn + lr) * GM_LDK + 4 * lh + kg * 8;
#pragma unroll
        for (int i = 0; i < TM; i++) fa[set][i] = *(const v4f*)(a + i * 32 * GM_LDK);
#pragma unroll
        for (int j = 0; j < TN; j++) fw[set][j] = *(const v4f*)(w + j * 32 * GM_LDK);
    };
    auto multiply = [&](int set) __attribute__((always_inline)) {
#pragma unroll
        for (int c = 0; c < 4; c++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[set][i][c], fw[set][j][c], acc[i][j], 0, 0, 0);
    };

    const int nslab = (int)((K + GM_BK - 1) / GM_BK);
    unsigned oa[LA], ow[LW];
    offsets(m0, n0, oa, ow);
    const float* Ab = A + m0 * K;
    const float* Wb = W + n0 * K;
    if (!preloaded) {
        clamp_offsets(0, oa, ow);
        load_slab(Ab, Wb, oa, ow, 0);
    }
    store_slab(0, 0);
    lds_barrier();
    read_frag(0, 0, 0);
    // one k slab out of LDS buffer `buf` (a literal at both call sites, so every LDS address below is a
    // constant offset from the thread's base and no address arithmetic is left in the loop)
    auto slab = [&](int sl, int buf) __attribute__((always_inline)) {
        const bool more = sl + 1 < nslab;
        long knext = (long)(sl + 1) * GM_BK;
        if (!more && has_next) {
            // the staging registers now fetch slab 0 of the next tile: its offsets replace this tile's
            offsets(m0n, n0n, oa, ow);
            Ab = A + m0n * K;
            Wb = W + n0n * K;
            knext = 0;
        }
        if (more || has_next) {
            clamp_offsets(knext, oa, ow);
            load_slab(Ab, Wb, oa, ow, knext);
        }
#pragma unroll
        for (int kg = 0; kg + 1 < NKG; kg++) {
            read_frag((kg + 1) & 1, buf, kg + 1);
            multiply(kg & 1);
        }
        // the staged slab goes to LDS as late as possible: its loads have had NKG - 1 groups of MFMAs to arrive
        if (more) store_slab(buf ^ 1, knext);
        lds_barrier();
        if (more) read_frag(0, buf ^ 1, 0);
        multiply((NKG - 1) & 1);
    };
    for (int sl = 0; sl < nslab; sl += 2) {
        slab(sl, 0);
        if (sl + 1 < nslab) slab(sl + 1, 1);
    }

    // epilogue: lane holds column n = lr of 16 rows per MFMA tile.
    // Tiles with all their rows and a plain bias + activation epilogue (every hidden layer) take a path
    // with one add and the activation per element; everything else takes the guarded one.
    const bool plain = !epi.out_scale && epi.mask_from >= N && m0 + BM <= B;
    const int ncols = (int)(N - n0 < BN ? N - n0 : BN);                 // columns of this tile that exist
    if (plain) {
        float* cb = C + m0 * N + n0;                                    // uniform
        const float* bias = epi.bias ? epi.bias + n0 : nullptr;
        if (epi.act == FORTIS_ACT_RELU) gemm_store_plain<TM, TN, 1>(acc, cb, (unsigned)N, bias, wm, wn, lr, lh, ncols, epi);
        else if (epi.act == FORTIS_ACT_LEAKY && epi.alpha >= 0.f && epi.alpha <= 1.f) gemm_store_plain<TM, TN, 2>(acc, cb, (unsigned)N, bias, wm, wn, lr, lh, ncols, epi);
        else if (epi.act == FORTIS_ACT_NONE) gemm_store_plain<TM, TN, 0>(acc, cb, (unsigned)N, bias, wm, wn, lr, lh, ncols, epi);
        else gemm_store_plain<TM, TN, 3>(acc, cb, (unsigned)N, bias, wm, wn, lr, lh, ncols, epi);
        return;
    }
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

// Work list of one launch.  Tiles are numbered row-major over 128 x 128 blocks of C; a phase hands
// out items of 1 (level 0), 1/2 (level 1: 128 x 64) or 1/4 (level 2: 64 x 64) of such a block.
struct GemmPhase { int level, pad; long base, count; };
struct GemmSched { int nphase, tiles_n; long slots; GemmPhase ph[4]; };

// Persistent kernel: the grid is exactly the number of workgroups the chip holds at once (slots), and
// every workgroup walks the phases taking item (round * slots + its place).  Whole rounds of full
// blocks come first; what is left over is cut into halves and quarters so that the last rounds still
// give every workgroup (hence every CU) the same amount of work -- with plain one-tile-per-workgroup
// launches a 1.5-round problem costs 2 rounds.
// Within a round the places are numbered so that each XCD (workgroup id mod 8) gets a contiguous band
// of items: the band's A rows and all of W stay in that XCD's L2.
template <int GM_BK>
__global__ __launch_bounds__(GM_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                          float* __restrict__ C, long B, long N, long K,
                                                          GemmSched sc, GemmEpi epi)
{
    extern __shared__ float4 smem4[];
    float* smem = (float*)smem4;
    const long w = blockIdx.x;
    for (int p = 0; p < sc.nphase; p++) {
        const int level = sc.ph[p].level;
        const long base = sc.ph[p].base, count = sc.ph[p].count;
        if (level == 0) {
            // whole rounds: count is a multiple of slots, this workgroup's place is the same in each
            const long place = (w & 7) * (sc.slots / 8) + (w >> 3);
            const long rounds = count / sc.slots;
            v4f ra[2 * GM_BK / 16], rw[2 * GM_BK / 16];
            for (long r = 0; r < rounds; r++) {
                const long tile = base + r * sc.slots + place, next = tile + sc.slots;
                const long tm = tile / sc.tiles_n, tn = tile - tm * sc.tiles_n;
                const long tmn = next / sc.tiles_n, tnn = next - tmn * sc.tiles_n;
                gemm_tile<2, 2, GM_BK>(A, W, C, B, N, K, tm * 128, tn * 128, epi, smem, ra, rw,
                                       r > 0, r + 1 < rounds, tmn * 128, tnn * 128);
            }
            continue;
        }
        // a partial round of halves or quarters
        const long per_xcd = (count + 7) / 8;
        if ((w >> 3) >= per_xcd) continue;
        const long item = (w & 7) * per_xcd + (w >> 3);
        if (item >= count) continue;
        const long tile = base + (level == 1 ? (item >> 1) : (item >> 2));
        const long tm = tile / sc.tiles_n, tn = tile - tm * sc.tiles_n;
        if (level == 1) {
            const long m0 = tm * 128, n0 = tn * 128 + (item & 1) * 64;
            if (m0 >= B || n0 >= N) continue;
            v4f ra[2 * GM_BK / 16], rw[GM_BK / 16];
            gemm_tile<2, 1, GM_BK>(A, W, C, B, N, K, m0, n0, epi, smem, ra, rw, false, false, 0, 0);
        } else {
            const long m0 = tm * 128 + ((item >> 1) & 1) * 64, n0 = tn * 128 + (item & 1) * 64;
            if (m0 >= B || n0 >= N) continue;
            v4f ra[GM_BK / 16], rw[GM_BK / 16];
            gemm_tile<1, 1, GM_BK>(A, W, C, B, N, K, m0, n0, epi, smem, ra, rw, false, false, 0, 0);
        }
    }
}

// Small batches (B <= 16; the reference's generated warp-per-output kernel for batch < 32,
// compiler/FortisFuse.cpp:667-719): one wave per output column n.  The lanes stride over k with 16-byte
// loads of W[n][:] (1 KiB per wave per step, fully coalesced) and of the few A rows (the same for every
// wave: served by the caches), then the 64 partial sums are folded with a shuffle tree.  Memory-bound on
// reading W once; a 128 x 128 MFMA tile would be 1 % useful.
template <int BR>
__global__ __launch_bounds__(256) void gemm_small_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                         float* __restrict__ C, int B, long N, long K, GemmEpi epi)
{
    const int lane = threadIdx.x & 63;
    const long n = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    float acc[BR];
#pragma unroll
    for (int r = 0; r < BR; r++) acc[r] = 0.f;
    const float* wrow = W + n * K;
    for (long k0 = lane * 4; k0 < K; k0 += 256) {
        const v4f w = *(const v4f*)(wrow + k0);
#pragma unroll
        for (int r = 0; r < BR; r++) {
            const v4f a = *(const v4f*)(A + (long)(r < B ? r : 0) * K + k0);
            acc[r] = fmaf(w.w, a.w, fmaf(w.z, a.z, fmaf(w.y, a.y, fmaf(w.x, a.x, acc[r]))));
        }
    }
#pragma unroll
    for (int r = 0; r < BR; r++)
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) acc[r] += __shfl_xor(acc[r], off, 64);
    if (lane == 0) {
        const float bv = epi.bias ? epi.bias[n] : 0.f;
#pragma unroll
        for (int r = 0; r < BR; r++) {
            if (r >= B) break;
            float v = gemm_act(acc[r] + bv, epi.act, epi.alpha);
            if (epi.out_scale) v = v * epi.out_scale[n];
            if (n >= epi.mask_from) v = v > 0.f ? v : 0.f;
            C[(long)r * N + n] = v;
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

// Work list for C[B][N] on `slots` resident workgroups (a multiple of 8): whole rounds of 128 x 128 tiles,
// then one round of halves if at least half a round is left, one round of quarters if at least a quarter
// round is left, and the rest as quarters.
static void gemm_make_sched(long B, long N, long slots, GemmSched* out)
{
    GemmSched sc = {};
    sc.tiles_n = (int)cdiv(N, 128);
    sc.slots = slots;
    const long total = cdiv(B, 128) * sc.tiles_n;
    long base = total / slots * slots, rem = total - base;
    auto phase = [&](int level, long b, long count) { GemmPhase ph = { level, 0, b, count }; sc.ph[sc.nphase++] = ph; };
    if (base) phase(0, 0, base);
    if (2 * rem >= slots) { phase(1, base, slots); base += slots / 2; rem -= slots / 2; }
    if (4 * rem >= slots) { phase(2, base, slots); base += slots / 4; rem -= slots / 4; }
    if (rem) phase(2, base, 4 * rem);
    *out = sc;
}

// Test hook: the schedule as (level, first tile, items) triples; returns the number of phases.
extern "C" int fortis_gemm_schedule(long B, long N, long slots, long* triples)
{
    if (B <= 0 || N <= 0 || slots < 8 || slots % 8) return -1;
    GemmSched sc;
    gemm_make_sched(B, N, slots, &sc);
    for (int p = 0; p < sc.nphase; p++) { triples[3 * p] = sc.ph[p].level; triples[3 * p + 1] = sc.ph[p].base; triples[3 * p + 2] = sc.ph[p].count; }
    return sc.nphase;
}

// slots = workgroups resident at once (occupancy x CUs), a multiple of 8
template <int BK>
static void launch_tiled(const float* A, const float* W, float* C, long B, long N, long K, const GemmEpi& epi, hipStream_t s)
{
    const size_t shmem = (size_t)2 * (128 + 128) * (BK + 4) * sizeof(float);
    static long slots = 0;
    if (!slots) {
        HIP_OK(hipFuncSetAttribute((const void*)gemm_kernel<BK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem));
        int occ = 0, dev = 0;
        hipDeviceProp_t prop;
        HIP_OK(hipGetDevice(&dev));
        HIP_OK(hipGetDeviceProperties(&prop, dev));
        HIP_OK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void*)gemm_kernel<BK>, GM_THREADS, shmem));
        if (occ < 1) occ = 1;
        slots = (long)occ * prop.multiProcessorCount / 8 * 8;
        if (slots < 8) slots = 8;
    }
    GemmSched sc;
    gemm_make_sched(B, N, slots, &sc);
    long items = 0;
    for (int p = 0; p < sc.nphase; p++) items = sc.ph[p].count > items ? sc.ph[p].count : items;
    const long grid = items < slots ? cdiv(items, 8) * 8 : slots;
    hipLaunchKernelGGL((gemm_kernel<BK>), dim3((unsigned)grid), dim3(GM_THREADS), shmem, s, A, W, C, B, N, K, sc, epi);
    HIP_OK(hipGetLastError());
}

int fortis_launch_gemm(const float* A, const float* W, const float* bias, float* C, long B, long N, long K,
                       int act, float alpha, const float* out_scale, long mask_tail, hipStream_t s)
{
    if (B <= 0 || N <= 0 || K <= 0) return -1;
    GemmEpi epi = { bias, out_scale, act, alpha, mask_tail > 0 ? N - mask_tail : N };
    const bool vec_ok = (K % 4 == 0) && K < (1L << 22) && N < (1L << 24) && (((uintptr_t)A | (uintptr_t)W) % 16 == 0);
    if (!vec_ok) {
        hipLaunchKernelGGL(gemm_naive_kernel, dim3((unsigned)cdiv(B * N, 256)), dim3(256), 0, s, A, W, C, B, N, K, epi);
        HIP_OK(hipGetLastError());
        return 0;
    }
    if (B <= 16) {
        const dim3 grid((unsigned)cdiv(N, 4)), block(256);
        if (B == 1) hipLaunchKernelGGL(gemm_small_kernel<1>, grid, block, 0, s, A, W, C, (int)B, N, K, epi);
        else if (B <= 4) hipLaunchKernelGGL(gemm_small_kernel<4>, grid, block, 0, s, A, W, C, (int)B, N, K, epi);
        else hipLaunchKernelGGL(gemm_small_kernel<16>, grid, block, 0, s, A, W, C, (int)B, N, K, epi);
        HIP_OK(hipGetLastError());
        return 0;
    }
    static int bk = 0;
    if (!bk) { const char* e = getenv("FORTIS_GEMM_BK"); bk = (e && atoi(e) == 16) ? 16 : 32; }
    if (bk == 16) launch_tiled<16>(A, W, C, B, N, K, epi, s);
    else launch_tiled<32>(A, W, C, B, N, K, epi, s);
    return 0;
}
