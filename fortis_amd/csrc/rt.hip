// Runtime tier: persistent stream, device buffer pool and the memref-expanded GEMM / conv entry
// points of include/fortis_rt.h.  Replaces runtime/fortis_rt.c of the reference one for one; the
// vendor-library calls behind those entries are replaced by the hand-written kernels of this
// library.
#include "common.h"

// ---- stream (runtime/fortis_rt.c:5-12) ---------------------------------------------------
static hipStream_t g_stream = nullptr;

// ---- fixed scratch of the entry that allocates nothing (fortis_conv3d_noalloc) -----------------------------
// The array's name is a host-side handle, not a device address: host code uses the address that
// hipGetSymbolAddress returns for the current device, looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[FORTIS_NOALLOC_SCRATCH_BYTES];
#define FORTIS_MAX_DEVICES 64
static void* g_scratch_ptr[FORTIS_MAX_DEVICES];
static void* noalloc_scratch()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= FORTIS_MAX_DEVICES) { (void)hipGetLastError(); return nullptr; }
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            fprintf(stderr, "fortis: the fixed scratch array has no address on device %d: %s\n", dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}

extern "C" {
int fortis_capturing = 0;

void* mgpuStreamCreate(void)
{
    if (!g_stream) {
        int ndev = 0;
        if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
            fprintf(stderr, "fortis: no HIP device available; this library has no CPU path\n");
            abort();
        }
        HIP_OK(hipStreamCreate(&g_stream));   // default priority, blocking flag like cudaStreamCreate
        (void)noalloc_scratch();              // set-up: the fixed scratch's address on this device
    }
    return (void*)g_stream;
}
void mgpuStreamDestroy(void*) {}
void mgpuStreamSynchronize(void*) {}
}

// ---- pool (runtime/fortis_rt.c:14-40) ------------------------------------------------------
// Same policy as the reference: 256 slots, best fit among released buffers, allocate otherwise,
// release-all-unused-and-retry once when the device is out of memory.  The allocator behind it is
// switchable so the policy can be exercised on a machine with no GPU (tests set a host allocator).
#define FORTIS_POOL 256
typedef int (*fortis_raw_alloc_fn)(void** p, size_t n);
typedef void (*fortis_raw_free_fn)(void* p);
static long g_raw_allocs = 0;   // raw allocations asked of the device allocator since the library was loaded
static int dev_alloc(void** p, size_t n) { g_raw_allocs++; return hipMalloc(p, n) == hipSuccess ? 0 : -1; }
static void dev_free(void* p) { HIP_OK(hipFree(p)); }
static fortis_raw_alloc_fn g_alloc = dev_alloc;
static fortis_raw_free_fn g_free = dev_free;
static struct { long n; void* p; int used; } g_pool[FORTIS_POOL];

int fortis_dev_malloc(void** p, size_t nbytes, const char* what)
{
    *p = nullptr;
    if (g_alloc(p, nbytes ? nbytes : 4) == 0 && *p) return 0;
    if (g_alloc == dev_alloc) (void)hipGetLastError();
    *p = nullptr;
    fprintf(stderr, "fortis: device allocation of %zu bytes failed (%s)\n", nbytes, what);
    return -1;
}
void fortis_dev_free(void* p) { if (p) g_free(p); }
bool fortis_pool_on_device() { return g_alloc == dev_alloc; }
long fortis_pool_best_fit(long n)
{
    long best = -1;
    for (int i = 0; i < FORTIS_POOL; i++)
        if (g_pool[i].p && !g_pool[i].used && g_pool[i].n >= n && (best < 0 || g_pool[i].n < best)) best = g_pool[i].n;
    return best;
}

extern "C" {
// Test hook: replaces the raw allocator (null restores hipMalloc/hipFree) and empties the pool table.
void fortis_pool_set_allocator(fortis_raw_alloc_fn a, fortis_raw_free_fn f)
{
    g_alloc = a ? a : dev_alloc;
    g_free = f ? f : dev_free;
    memset(g_pool, 0, sizeof g_pool);
    fortis_conv_forget_buffers();
}
// Test hook: how many times the library has asked the device for memory (every hipMalloc of the library goes
// through one function): a call that must allocate nothing leaves the count unchanged.
long fortis_dev_alloc_calls(void) { return g_raw_allocs; }
// Runtime calls that have failed since the library was loaded (each was also printed).
static long g_errors = 0;
void fortis_note_error(void) { __atomic_add_fetch(&g_errors, 1, __ATOMIC_RELAXED); }
long fortis_error_count(void) { return __atomic_load_n(&g_errors, __ATOMIC_RELAXED); }
// Test hook: number of slots holding a buffer, and how many of them are in use.
void fortis_pool_stats(int* held, int* used)
{
    int h = 0, u = 0;
    for (int i = 0; i < FORTIS_POOL; i++) if (g_pool[i].p) { h++; u += g_pool[i].used; }
    if (held) *held = h;
    if (used) *used = u;
}

// Gives the buffers the pool holds unused back to the device (a host between two phases of different sizes; the
// benchmark between workloads, so that each starts on fresh memory).  Returns how many were freed.
int fortis_pool_trim(void)
{
    int freed = 0;
    for (int i = 0; i < FORTIS_POOL; i++)
        if (g_pool[i].p && !g_pool[i].used) { g_free(g_pool[i].p); g_pool[i].p = nullptr; g_pool[i].n = 0; freed++; }
    return freed;
}

void* fortis_alloc(long n)
{
    int best = -1;
    for (int i = 0; i < FORTIS_POOL; i++)
        if (g_pool[i].p && !g_pool[i].used && g_pool[i].n >= n && (best < 0 || g_pool[i].n < g_pool[best].n)) best = i;
    if (best >= 0) { g_pool[best].used = 1; return g_pool[best].p; }
    for (int attempt = 0; attempt < 2; attempt++) {
        for (int i = 0; i < FORTIS_POOL; i++)
            if (!g_pool[i].p) {
                if (g_alloc(&g_pool[i].p, (size_t)n) == 0) { g_pool[i].n = n; g_pool[i].used = 1; return g_pool[i].p; }
                g_pool[i].p = nullptr;
                break;
            }
        if (g_alloc == dev_alloc) (void)hipGetLastError();
        for (int i = 0; i < FORTIS_POOL; i++)
            if (g_pool[i].p && !g_pool[i].used) { g_free(g_pool[i].p); g_pool[i].p = nullptr; g_pool[i].n = 0; }
    }
    fprintf(stderr, "fortis_alloc: device allocation of %ld bytes failed\n", n);
    return nullptr;
}
void fortis_free(void* p)
{
    if (!p) return;
    for (int i = 0; i < FORTIS_POOL; i++) if (g_pool[i].p == p) { g_pool[i].used = 0; return; }
    g_free(p);
}

// ---- GEMM entry (runtime/fortis_rt.c:45-75) ------------------------------------------------
// The reference pre-transposes each weight once so cuBLAS can run N,N.  The MFMA kernel reads
// W[N][K] rows directly as its B operand (k is the contiguous axis of both operands), so no
// transpose cache exists here and FORTIS_NO_PRETRANS has nothing to switch.
void fortis_gemm(float* Aa, float* A, long Ao, long As0, long As1, long At0, long At1,
                 float* Wa, float* W, long Wo, long Ws0, long Ws1, long Wt0, long Wt1,
                 float* Ca, float* C, long Co, long Cs0, long Cs1, long Ct0, long Ct1,
                 long B, long N, long K)
{
    (void)Aa; (void)As0; (void)As1; (void)At0; (void)At1; (void)Wa; (void)Ws0; (void)Ws1; (void)Wt0; (void)Wt1;
    (void)Ca; (void)Cs0; (void)Cs1; (void)Ct0; (void)Ct1;
    // Empty problems as the reference's SGEMM call treats them (runtime/fortis_rt.c:69-74, beta = 0): no rows or no
    // columns, nothing happens; no k, the sum is empty and C becomes zero.
    if (B <= 0 || N <= 0 || K < 0) return;
    if (K == 0) { fortis_launch_zero(C + Co, B * N, fortis_stream_get()); return; }
    if (fortis_launch_gemm(A + Ao, W + Wo, nullptr, C + Co, B, N, K, FORTIS_ACT_NONE, 0.f, nullptr, 0, fortis_stream_get()) != 0)
        fprintf(stderr, "fortis_gemm: unsupported shape B%ld N%ld K%ld\n", B, N, K);
}

// ---- conv entries (runtime/fortis_rt.c:108-156, runtime/fortis_fft.cu:66-79, 131-146) -------
// Shapes the matrix-core kernel takes (stride 1, K = 1 or 3 with same padding, enough output channels to fill a
// 32-channel group) go to it: the raw weights are packed on the device with every call (the reference reads the
// weights it is given on every call, so nothing is cached by pointer).  FORTIS_CONV_DIRECT=1 keeps the direct
// kernels.  Returns -1 when the shape is not taken.
static int conv_entry_mfma(const float* x, const float* w, float* y, long C, long D, long H, long Wd, long F, long KD, long KS)
{
    static int direct_only = -1;
    if (direct_only < 0) direct_only = getenv("FORTIS_CONV_DIRECT") != nullptr;
    if (direct_only || !(F >= 16 || (KD == 1 && KS == 1))) return -1;
    hipStream_t s = fortis_stream_get();
    const float* wp = fortis_conv_mfma_pack_dev(w, F, C, (int)(KD * KS * KS), s, fortis_conv_mfma_kgroups(C, D, H, Wd, F, (int)KD, (int)KS));
    if (!wp) return -1;
    ConvEpi e = { nullptr, nullptr, FORTIS_ACT_NONE, 0.f, nullptr };
    return fortis_launch_conv_mfma(x, wp, y, C, D, H, Wd, F, (int)KD, (int)KS, 0, e, s);
}

void fortis_conv2d(float* xa, float* x, long xo, long x0, long x1, long x2, long x3, long xt0, long xt1, long xt2, long xt3,
                   float* wa, float* w, long wo, long w0, long w1, long w2, long w3, long wt0, long wt1, long wt2, long wt3,
                   float* ya, float* y, long yo, long y0, long y1, long y2, long y3, long yt0, long yt1, long yt2, long yt3,
                   long N, long C, long Hin, long Win, long F, long KH, long KW, long Hout, long Wout,
                   long sh, long sw, long ph, long pw)
{
    (void)xa; (void)x0; (void)x1; (void)x2; (void)x3; (void)xt0; (void)xt1; (void)xt2; (void)xt3;
    (void)wa; (void)w0; (void)w1; (void)w2; (void)w3; (void)wt0; (void)wt1; (void)wt2; (void)wt3;
    (void)ya; (void)y0; (void)y1; (void)y2; (void)y3; (void)yt0; (void)yt1; (void)yt2; (void)yt3;
    ConvEpi e = { nullptr, nullptr, FORTIS_ACT_NONE, 0.f, nullptr };
    const bool same = sh == 1 && sw == 1 && KH == KW && (KH == 1 || KH == 3) && ph == KH / 2 && pw == KW / 2 && Hout == Hin && Wout == Win;
    for (long n = 0; n < N; n++) {
        if (same && conv_entry_mfma(x + xo + n * C * Hin * Win, w + wo, y + yo + n * F * Hout * Wout, C, 1, Hin, Win, F, 1, KH) == 0) continue;
        int rc = fortis_launch_conv2d(x + xo + n * C * Hin * Win, w + wo, y + yo + n * F * Hout * Wout, C, Hin, Win, F,
                                      KH, KW, Hout, Wout, sh, sw, ph, pw, e, 0, F, fortis_stream_get());
        if (rc != 0) {
            fprintf(stderr, "fortis_conv2d: unsupported shape  N%ld C%ld in%ldx%ld F%ld K%ldx%ld out%ldx%ld s%ld,%ld p%ld,%ld\n",
                    N, C, Hin, Win, F, KH, KW, Hout, Wout, sh, sw, ph, pw);
            return;
        }
    }
}

// fortis_conv3d takes what the reference's library path takes (runtime/fortis_rt.c:128-156): any batch, any
// stride.  The direct and large-kernel entries keep the reference's own limits (N = 1, stride 1;
// runtime/fortis_fft.cu:70, 135).
static int conv3d_any(const char* who, bool general, float* x, long xo, float* w, long wo, float* y, long yo, long N, long C,
                      long Din, long Hin, long Win, long F, long KD, long KH, long KW, long Dout, long Hout,
                      long Wout, long sd, long sh, long sw, long pd, long ph, long pw)
{
    const bool unit = sd == 1 && sh == 1 && sw == 1;
    if (!general && (N != 1 || !unit)) { fprintf(stderr, "%s: unsupported shape\n", who); return -1; }
    const long xn = C * Din * Hin * Win, yn = F * Dout * Hout * Wout;
    for (long n = 0; n < N; n++) {
        float* xb = x + xo + n * xn;
        float* yb = y + yo + n * yn;
        if (unit && KD == 3 && KH == 3 && KW == 3 && pd == 1 && ph == 1 && pw == 1 && Dout == Din && Hout == Hin && Wout == Win &&
            conv_entry_mfma(xb, w + wo, yb, C, Din, Hin, Win, F, 3, 3) == 0)
            continue;
        ConvEpi e = { nullptr, nullptr, FORTIS_ACT_NONE, 0.f, nullptr };
        int rc = -1;
        // a caller's fixed workspace that was too small is an error of its own: the shape is not handed on to
        // a slower kernel behind the caller's back
        if (!fortis_conv_workspace_overflowed())
            rc = fortis_launch_conv3d(xb, w + wo, yb, C, Din, Hin, Win, F, KD, KH, KW, Dout, Hout, Wout, pd, ph, pw, e,
                                      fortis_stream_get(), sd, sh, sw);
        if (fortis_conv_workspace_overflowed()) {
            fprintf(stderr, "%s: this shape needs %zu bytes of scratch, more than the fixed %ld; nothing computed\n", who,
                    fortis_conv_workspace_overflowed(), (long)FORTIS_NOALLOC_SCRATCH_BYTES);
            return -1;
        }
        if (rc != 0) { fprintf(stderr, "%s: unsupported shape\n", who); return -1; }
    }
    return 0;
}
#define CONV3D_UNUSED                                                                                               \
    (void)xa; (void)x0; (void)x1; (void)x2; (void)x3; (void)x4; (void)xt0; (void)xt1; (void)xt2; (void)xt3; (void)xt4; \
    (void)wa; (void)w0; (void)w1; (void)w2; (void)w3; (void)w4; (void)wt0; (void)wt1; (void)wt2; (void)wt3; (void)wt4; \
    (void)ya; (void)y0; (void)y1; (void)y2; (void)y3; (void)y4; (void)yt0; (void)yt1; (void)yt2; (void)yt3; (void)yt4
#define CONV3D_FWD(who, general)                                                                                    \
    conv3d_any(who, general, x, xo, w, wo, y, yo, N, C, Din, Hin, Win, F, KD, KH, KW, Dout, Hout, Wout, sd, sh, sw, pd, ph, pw)

void fortis_conv3d(FORTIS_CONV3D_ARGS) { CONV3D_UNUSED; (void)CONV3D_FWD("fortis_conv3d", true); }
// The same call for callers that cannot allocate device memory: the packed weights and the partial sums of
// channel-split launches live in the fixed scratch array instead of buffers grown with hipMalloc.  Every call
// on a GPU uses that GPU's one array (both regions are written in full before they are read, so nothing needs
// clearing): calls that overlap in time on one GPU race.
int fortis_conv3d_noalloc(FORTIS_CONV3D_ARGS)
{
    CONV3D_UNUSED;
    (void)fortis_stream_get();
    void* ws = noalloc_scratch();
    if (!ws) return -1;
    fortis_conv_workspace(ws, FORTIS_NOALLOC_SCRATCH_BYTES);
    const int rc = CONV3D_FWD("fortis_conv3d_noalloc", true);
    fortis_conv_workspace(nullptr, 0);
    return rc;
}
void fortis_conv3d_direct(FORTIS_CONV3D_ARGS) { CONV3D_UNUSED; (void)CONV3D_FWD("fortis_conv3d_direct", false); }
void fortis_conv3d_fft(FORTIS_CONV3D_ARGS)
{
    CONV3D_UNUSED;
    if (pd || ph || pw) { fprintf(stderr, "fortis_conv3d_fft: unsupported shape\n"); return; }
    (void)CONV3D_FWD("fortis_conv3d_fft", false);
}

// ---- host utilities ----------------------------------------------------------------------------
void fortis_h2d(void* dst, const void* src, long n)
{
    hipStream_t s = fortis_stream_get();
    HIP_OK(hipMemcpyAsync(dst, src, (size_t)n, hipMemcpyHostToDevice, s));
    HIP_OK(hipStreamSynchronize(s));
}
void fortis_d2h(void* dst, const void* src, long n)
{
    hipStream_t s = fortis_stream_get();
    HIP_OK(hipMemcpyAsync(dst, src, (size_t)n, hipMemcpyDeviceToHost, s));
    HIP_OK(hipStreamSynchronize(s));
}
void fortis_d2d(void* dst, const void* src, long n)
{
    HIP_OK(hipMemcpyAsync(dst, src, (size_t)n, hipMemcpyDeviceToDevice, fortis_stream_get()));
}
void fortis_sync(void) { HIP_OK(hipStreamSynchronize(fortis_stream_get())); }
int fortis_device_info(char* name, int len, long* total_mem)
{
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) { (void)hipGetLastError(); return -1; }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return -1;
    if (name && len > 0) { strncpy(name, prop.gcnArchName, (size_t)len - 1); name[len - 1] = 0; }
    if (total_mem) *total_mem = (long)prop.totalGlobalMem;
    return 0;
}
}  // extern "C"
