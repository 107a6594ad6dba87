/*
 * fortis_rt.h -- runtime tier of the MI355X backend: the C ABI that the compiled model object
 * (model.o) and the generated glue call.  Every symbol keeps the name, argument order and
 * behaviour of the reference runtime it replaces; the citation after each declaration is the
 * reference definition (paths relative to the reference tree).
 *
 * Memrefs are passed expanded, exactly as MLIR's default C convention does and as the
 * reference shim builds them (driver/fortis_shim.py:49-53):
 *     T* allocated, T* aligned, long offset, long size[rank], long stride[rank]
 * Like the reference, only `aligned + offset` is used; the data is assumed dense row-major.
 *
 * All device work is issued on one persistent HIP stream.  Nothing here returns an error code:
 * diagnostics go to stderr and the call returns without computing, as in the reference.
 */
#ifndef FORTIS_RT_H
#define FORTIS_RT_H

#ifdef __cplusplus
extern "C" {
#endif

/* ---- stream ---------------------------------------------------------------------------- */
/* The one persistent stream, created on first use.  Destroy and synchronize are deliberate
 * no-ops so that generated code never blocks.                       runtime/fortis_rt.c:5-12 */
void* mgpuStreamCreate(void);
void  mgpuStreamDestroy(void* stream);
void  mgpuStreamSynchronize(void* stream);
/* Set to 1 by the step driver while a graph capture is in progress.   runtime/fortis_rt.c:6 */
extern int fortis_capturing;

/* ---- device buffer pool ---------------------------------------------------------------- */
/* Best fit among released buffers (smallest with size >= nbytes), else a new allocation; on
 * allocation failure every unused buffer is released and the allocation retried once; on a
 * second failure prints and returns NULL.  256 slots.               runtime/fortis_rt.c:14-36 */
void* fortis_alloc(long nbytes);
/* Marks a pooled buffer unused (it stays allocated); a pointer the pool does not know is
 * freed for real.                                                   runtime/fortis_rt.c:37-40 */
void  fortis_free(void* p);

/* Test hooks, no reference counterpart: swap the raw allocator under the pool (NULL, NULL restores
 * the device allocator) and empty the pool table; count held / in-use slots.  They let the pool
 * policy be exercised on a machine without a GPU. */
void  fortis_pool_set_allocator(int (*raw_alloc)(void** p, unsigned long nbytes), void (*raw_free)(void* p));
void  fortis_pool_stats(int* held, int* used);
/* Frees every buffer the pool holds unused (fortis_free only marks a buffer as reusable, runtime/fortis_rt.c:36-40) and
 * returns their number.  No reference counterpart: there the pool only shrinks when an allocation fails. */
int   fortis_pool_trim(void);
/* Grows the library's buffer for the partial sums of channel-split convolutions ahead of time (it otherwise grows on
 * the first call that needs it): 0, or -1 with a message when the device has no memory.  No reference counterpart. */
int   fortis_conv_scratch_reserve(long bytes);
long  fortis_dev_alloc_calls(void);   /* test hook: raw device allocations the library has made since it was loaded */
/* Runtime (HIP) calls that have failed since the library was loaded.  Like the reference runtime
 * (runtime/fortis_rt.c:30-34, 124, 153: print and return) the library reports a failed call on stderr and goes on; a
 * host that would rather stop reads this count after a step.  fortis_note_error adds one (the library's own use). */
long  fortis_error_count(void);
void  fortis_note_error(void);

/* ---- GEMM -------------------------------------------------------------------------------- */
/* C[B][N] = A[B][K] . W[N][K]^T, fp32, beta = 0.                     runtime/fortis_rt.c:45-75
 * Empty problems as the reference's SGEMM call leaves them: B = 0 or N = 0 does nothing, K = 0 sets C to zero. */
void fortis_gemm(float* Aa, float* A, long Ao, long As0, long As1, long At0, long At1,
                 float* Wa, float* W, long Wo, long Ws0, long Ws1, long Wt0, long Wt1,
                 float* Ca, float* C, long Co, long Cs0, long Cs1, long Ct0, long Ct1,
                 long B, long N, long K);

/* ---- convolutions ------------------------------------------------------------------------ */
/* NCHW cross-correlation, weights [F][C][KH][KW], explicit symmetric padding, stride (sh,sw),
 * dilation 1, beta = 0; bias/BN/activation are applied by the caller's epilogue.
 *                                                                   runtime/fortis_rt.c:108-127 */
void fortis_conv2d(float* xa, float* x, long xo, long x0, long x1, long x2, long x3, long xt0, long xt1, long xt2, long xt3,
                   float* wa, float* w, long wo, long w0, long w1, long w2, long w3, long wt0, long wt1, long wt2, long wt3,
                   float* ya, float* y, long yo, long y0, long y1, long y2, long y3, long yt0, long yt1, long yt2, long yt3,
                   long N, long C, long Hin, long Win, long F, long KH, long KW, long Hout, long Wout,
                   long sh, long sw, long ph, long pw);

#define FORTIS_CONV3D_ARGS                                                                                      \
    float* xa, float* x, long xo, long x0, long x1, long x2, long x3, long x4, long xt0, long xt1, long xt2,   \
    long xt3, long xt4, float* wa, float* w, long wo, long w0, long w1, long w2, long w3, long w4, long wt0,   \
    long wt1, long wt2, long wt3, long wt4, float* ya, float* y, long yo, long y0, long y1, long y2, long y3,  \
    long y4, long yt0, long yt1, long yt2, long yt3, long yt4, long N, long C, long Din, long Hin, long Win,   \
    long F, long KD, long KH, long KW, long Dout, long Hout, long Wout, long sd, long sh, long sw, long pd,    \
    long ph, long pw

/* NCDHW cross-correlation.  The reference chooses between a vendor library and its direct
 * kernel with FORTIS_DIRECT; here every shape runs the library-free direct path.
 *                                                                   runtime/fortis_rt.c:128-156 */
void fortis_conv3d(FORTIS_CONV3D_ARGS);
/* No counterpart in the reference.  fortis_conv3d for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): same arguments and result, but the
 * packed weights and the partial sums of channel-split launches live in a fixed device array of
 * FORTIS_NOALLOC_SCRATCH_BYTES that the library holds on every GPU it runs on, and the call makes no hipMalloc,
 * hipFree or other allocating call.  Returns 0, or -1 with a message on stderr when the shape is unsupported or
 * needs more scratch than that (nothing is computed then).  All calls on one GPU share the array: calls that
 * overlap in time on one GPU race.  The library must have been used once before (any entry; mgpuStreamCreate
 * does) when the caller is capturing. */
#define FORTIS_NOALLOC_SCRATCH_BYTES (32L << 20)
int  fortis_conv3d_noalloc(FORTIS_CONV3D_ARGS);
/* Direct tiled conv3d; N = 1 and stride 1 only, otherwise prints "unsupported shape" and
 * returns without computing.                                        runtime/fortis_fft.cu:131-146 */
void fortis_conv3d_direct(FORTIS_CONV3D_ARGS);
/* Large-kernel entry (kernel volume >= 125, pad 0, N = 1).  Same result as the direct path,
 * which is what runs; shapes it rejected in the reference (N != 1, stride != 1, pad != 0) are
 * rejected here with the same message.                              runtime/fortis_fft.cu:66-79 */
void fortis_conv3d_fft(FORTIS_CONV3D_ARGS);

/* ---- host utilities ------------------------------------------------------------------------ */
/* No reference counterpart: the reference's generated glue calls cudaMemcpy / cudaStreamSynchronize
 * directly.  These give a caller without a HIP binding (the Python host layer, tests, a Fortran
 * host) stream-ordered copies to and from buffers obtained from fortis_alloc. */
void fortis_h2d(void* dst_device, const void* src_host, long nbytes);   /* returns when src may be reused */
void fortis_d2h(void* dst_host, const void* src_device, long nbytes);   /* returns with dst filled */
void fortis_d2d(void* dst_device, const void* src_device, long nbytes); /* asynchronous */
void fortis_sync(void);                                                 /* waits for the persistent stream */
/* Device name into `name` (at most len bytes), total device memory in bytes; 0 on success, -1
 * when no GPU is present. */
int  fortis_device_info(char* name, int len, long* total_mem);

#ifdef __cplusplus
}
#endif
#endif
