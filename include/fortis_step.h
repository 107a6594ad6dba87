/*
 * fortis_step.h -- host-facing tier of the MI355X backend: the entry points a Fortran/C host
 * calls by bind(c) name, and the tables that parameterise them.
 *
 * In the reference these entries are C/CUDA text generated per build with every size baked in
 * (driver/fortis_shim.py -> shim.c, driver/fortis_gather_emit.py -> gather.cu) and the model is
 * MLIR-generated host code (`mlp_kernel` in model.o).  Here the same entry names live in the
 * library and read their sizes from tables bound once at start-up:
 *     fortis_plan_*     the model: the op list fortis-fuse would have emitted, with its weights
 *     fortis_step_bind  the facts of the `fortis.host` attribute (driver/fortis_hostattr.py:11-28)
 *     fortis_gather_config / fortis_scatter_config   gather.json / scatter.json / loop.json / kdist.json
 * The per-build generated file shrinks to a table plus one bind call.
 *
 * Conventions kept from the reference (driver/fortis_shim.py, mom6_zb/gather.cu): host arrays
 * belong to the host; device buffers belong to the library for the life of the process; no return
 * codes on the bind(c) entries, diagnostics on stderr; one host thread, one stream, file-scope
 * state.  mlp_forward, mlp_download and fortis_scatter return with results visible on the host;
 * fortis_gather, mlp_forward_dev and the argument-less mlp_forward_batched are asynchronous.
 * Table-building calls (fortis_plan_*, *_config, fortis_step_bind) return 0 or -1.
 */
#ifndef FORTIS_STEP_H
#define FORTIS_STEP_H

#ifdef __cplusplus
extern "C" {
#endif

/* ================================ model plan ============================================ */
/* ReLU is v > 0 ? v : 0 and LeakyReLU v > 0 ? v : alpha * v on finite values and infinities.  A NaN pre-activation is
 * outside the parity contract: ReLU turns it into 0 in most kernels, while the straight-line kernels of narrow
 * networks (all widths <= 64) take the maximum on the bit pattern and keep a NaN whose sign bit is clear. */
enum { FORTIS_ACT_NONE = 0, FORTIS_ACT_RELU = 1, FORTIS_ACT_LEAKY = 2 };

typedef struct fortis_plan fortis_plan;

fortis_plan* fortis_plan_create(void);
void         fortis_plan_destroy(fortis_plan* p);
/* Declares an activation tensor of `nbytes` bytes; returns its id (>= 0).  Tensors are device
 * buffers taken from fortis_alloc at finalize. */
int  fortis_plan_tensor(fortis_plan* p, long nbytes);
/* Declares a window [byte_offset, byte_offset + nbytes) of tensor `base` as a tensor of its own
 * (16-byte aligned).  A channel concatenation is then two producers writing the two windows of
 * one buffer (what the reference does with memref.copy into a subview,
 * compiler/FortisFuse.cpp:547-551, 122-133) and costs no copy. */
int  fortis_plan_view(fortis_plan* p, int base, long byte_offset, long nbytes);

/* dst[B][N] = act(src[B][K] . W[N][K]^T + bias[N]).  W, bias are host pointers, copied to the
 * device at finalize (the role of setup() uploading w<i>, driver/fortis_shim.py:67-72).  bias may
 * be NULL.  Replaces a fortis_gemm call plus its epilogue kernel (runtime/fortis_rt.c:45-75,
 * compiler/FortisFuse.cpp:685-692, 721-760) with one fused kernel. */
int  fortis_plan_linear(fortis_plan* p, int src, int dst, const float* W, const float* bias,
                        long B, long K, long N, int act, float alpha);
/* dst[r][c] = divide ? src[r][c] / vec[c] : src[r][c] * vec[c]; the lifted input/output
 * normalisation chain (mom6_zb/export_zb.py:14; compiler/FortisFuse.cpp:526-573). */
int  fortis_plan_scale(fortis_plan* p, int src, int dst, const float* vec, long rows, long n, int divide);
/* dst = src with ReLU applied to the last `tail` of n features of every row: the
 * `y + mask*(relu(y) - y)` head (benchmarks/climsim/export_wide.py:27-28). */
int  fortis_plan_mask_relu(fortis_plan* p, int src, int dst, long rows, long n, long tail);
/* Boundary verdict, pre side: src is the host's own column-major (NI, NK) array of element size
 * host_esz (4 or 8); dst[i][k] = (float)((src[i + NI*k] - mean[k]) / (vmax[k] - vmin[k])) computed
 * in the host type.  mean/vmax/vmin are host vectors of that type (any may be NULL: mean 0,
 * range 1).  trt_backend/e3sm_boundary.cu:9-14; driver/fortis_emit2d.py:20-36. */
int  fortis_plan_boundary_pre(fortis_plan* p, int src, int dst, long NI, long NK, const void* mean,
                              const void* vmax, const void* vmin, int host_esz);
/* Post side: dst[i + NI*k] = (H)src[i][k] / scale[k].  trt_backend/e3sm_boundary.cu:15-20. */
int  fortis_plan_boundary_post(fortis_plan* p, int src, int dst, long NI, long NK, const void* scale,
                               int host_esz);

/* conv2d NCHW (N = 1): dst[coff .. coff+F) of a tensor holding ctot channels (so that a skip
 * concatenation is a channel-offset write, compiler/FortisFuse.cpp:547-551) =
 * act(bn(conv(src, W) + bias)).  W [F][C][KH][KW]; bias, and the four BatchNorm-eval vectors
 * (gamma, beta, mean, var; all or none) are host pointers of length F or NULL.  Replaces
 * fortis_conv2d + epilogue kernel (runtime/fortis_rt.c:108-127; FortisFuse.cpp:688-692). */
int  fortis_plan_conv2d(fortis_plan* p, int src, int dst, const float* W, const float* bias,
                        const float* bn_gamma, const float* bn_beta, const float* bn_mean,
                        const float* bn_var, float bn_eps, long C, long H, long Wd, long F, long KH,
                        long KW, long stride, long pad, int act, float alpha, long coff, long ctot);
/* Transposed conv2d, weights [C][F][KH][KW] (PyTorch layout), output size
 * (H-1)*stride - 2*pad + KH + output_padding.  Same epilogue and concat arguments. */
int  fortis_plan_convt2d(fortis_plan* p, int src, int dst, const float* W, const float* bias,
                         long C, long H, long Wd, long F, long KH, long KW, long stride, long pad,
                         long output_padding, int act, float alpha, long coff, long ctot);
/* k x k max pooling, stride k (compiler/FortisFuse.cpp:667-672: non-additive reduction). */
int  fortis_plan_maxpool2d(fortis_plan* p, int src, int dst, long C, long H, long Wd, long k);
/* Nearest-neighbour upsample by s over the trailing nd (2 or 3) spatial dims; D = 1 for nd = 2. */
int  fortis_plan_upsample(fortis_plan* p, int src, int dst, long C, long D, long H, long Wd, long s, int nd);
/* Copy C channels of S elements into dst at channel offset coff of ctot (concat by copy). */
int  fortis_plan_concat_copy(fortis_plan* p, int src, int dst, long C, long S, long coff, long ctot);
/* conv3d NCDHW, N = 1, stride 1: dst = act(conv(src, W) + bias) [+ res].  res is a tensor id
 * added after the activation (residual skip), or -1.  W [F][C][KD][KH][KW].  Replaces
 * fortis_conv3d(_direct) + epilogue (runtime/fortis_fft.cu:131-201). */
int  fortis_plan_conv3d(fortis_plan* p, int src, int dst, int res, const float* W, const float* bias,
                        long C, long D, long H, long Wd, long F, long K, long pad, int act, float alpha);
/* Layout permutes around a channels-last host tensor: to_channels_first != 0: [S][C] -> [C][S];
 * otherwise [C][S] -> [S][C].  S = product of the spatial dims. */
int  fortis_plan_permute(fortis_plan* p, int src, int dst, long C, long S, int to_channels_first);

/* Fixes the plan: allocates tensors, uploads weights, folds BatchNorm, fuses neighbouring ops
 * into single kernels.  in_tensor / out_tensor are what fortis_model_input/output return. */
int   fortis_plan_finalize(fortis_plan* p, int in_tensor, int out_tensor);
/* Enqueues one forward pass on the persistent stream (the role of the generated
 * mlp_kernel(...) host function, driver/fortis_shim.py:62-63, 86). */
void  fortis_plan_run(fortis_plan* p);
void* fortis_plan_tensor_ptr(fortis_plan* p, int tensor);
int   fortis_plan_num_kernels(fortis_plan* p);   /* launches per forward pass after fusion */

/* ================================ step binding ========================================== */
enum { FORTIS_VERDICT_WHOLE = 0, FORTIS_VERDICT_BATCHED = 1, FORTIS_VERDICT_BOUNDARY = 2 };

/* The facts the reference bakes into shim.c from the `fortis.host` attribute
 * (driver/fortis_shim.py:9-38, 94-133). */
typedef struct {
    long n_in, n_out;     /* elements of the whole model input / output */
    int  in_esz, out_esz; /* host element size: 4, or 8 under a boundary verdict on f64 arrays */
    int  verdict;         /* FORTIS_VERDICT_* */
    int  expanded;        /* batched: call temporaries expanded across the batch (pack/unpack form) */
    long count;           /* batched: rows per batched call */
    long lo, step, minc;  /* batched: loop start, stride, smallest visited column (1-based) */
    int  graph;           /* the fortis.graph attribute; FORTIS_GRAPH in the environment also enables it */
    int  gather, scatter; /* the build-time FORTIS_GATHER / FORTIS_SCATTER switches */
} fortis_host_t;

int  fortis_step_bind(fortis_plan* p, const fortis_host_t* host);
/* Registers a function that builds and binds the step; it runs once, at the first use of any entry point
 * below while no step is bound: the role of `if (!din) setup();` in the generated shim
 * (driver/fortis_shim.py:64-73), which copies weights and host globals at the first call, not at load time. */
void fortis_step_on_first_use(void (*bind)(void));
/* Forgets the bound step, the stencil tables and the graph (tests; a host never calls it). */
void fortis_step_reset(void);
int  fortis_step_graph_active(void);    /* 1 once a captured graph is being replayed */

/* ---- entry points, names and behaviour of the generated shim --------------------------- */
void  mlp_upload(void* in);                       /* driver/fortis_shim.py:93 */
void  mlp_forward_dev(void);                      /* :82-90  capture on call #2, replay after, eager fallback */
void  mlp_download(void* out);                    /* :92 */
void  mlp_forward(void* in, void* out);           /* :122 (single row, batched build) / :132-133 (whole array) */
/* One symbol, two reference forms: the expanded form takes no arguments (:113-115) and ignores
 * what it is passed; the slice form takes the host's whole in/out arrays (:117-121). */
void  mlp_forward_batched(void* in, void* out);
void  fortis_pack(void* row, int col);            /* :105  col is 0-based */
void  fortis_unpack(void* row, int col);          /* :106 */
void* fortis_model_input(void);                   /* :109 */
void* fortis_model_output(void);                  /* :110 */
/* Run-time extents: re-specialises the bound step for `count` rows per call; no JIT, the
 * kernels take the row count at run time.                  driver/fortis_stub.c:12-31 */
void  fortis_begin(int count);

/* ================================ stencil gather / scatter ============================== */
/* One element of one host array relative to cell (i, j) (1-based Fortran indices) and the
 * enclosing-loop plane kk (0-based): elem = base + i*si + j*sj + (planar ? kk*plane[array] : 0).
 * For A(i+di, j+dj, k) on a column-major (sx, sy, nk) array: si = 1, sj = sx,
 * base = (di-1) + (dj-1)*sx.  This is what driver/fortis_gather_emit.py:27-33 (elem, plane_off)
 * prints into the generated kernel. */
typedef struct { int array; int planar; long base, si, sj; } fortis_ref_t;

/* Lifted expressions as straight-line code: r[n] = operand(a) op operand(b).
 * operand: 0 = tv (the slot value), 1..8 = scalar S0..S7, 16+n = constant n, 32+n = r[n].
 * op (low byte): 0 add, 1 sub, 2 mul, 3 div, 4 fmaxf, 5 fminf, and on operand a alone 6 negate,
 * 7 sqrtf, 8 expf, 9 logf, 10 tanhf (the operator set of the reference's lifter,
 * driver/fortis_gather.py:89-121) and 11 conversion to float.  The last result replaces tv.  Each op is one IEEE operation,
 * never fused (the reference compiles gather.cu with -fmad=false).
 * Types follow the C the reference's generator prints (driver/fortis_gather_emit.py:57-61, 76-81):
 * tv is float, a scalar has its array's element type, a literal is float with an f suffix and
 * double without; + - * / and negate have a double result when an operand is double, which the
 * table builder marks with FORTIS_INS_F64 in op; the assignment back to tv at the end of an
 * expression is an explicit conversion (op 11) where the expression's type is double; the
 * f-suffixed functions convert their operands to float first.
 * Tables of at most 32 slots whose expressions are one chain of + - * / on the slot value over fp32 arrays
 * (tv op c, c op tv; at most 6 chained and 6 per-cell operations) run in the fused kernels; anything else takes
 * the general kernels, which take a table's slots 32 at a time. */
typedef struct { int op, a, b; } fortis_ins_t;
#define FORTIS_INS_F64 0x100
enum { FORTIS_OP_ADD = 0, FORTIS_OP_SUB, FORTIS_OP_MUL, FORTIS_OP_DIV, FORTIS_OP_MAX, FORTIS_OP_MIN,
       FORTIS_OP_NEG, FORTIS_OP_SQRT, FORTIS_OP_EXP, FORTIS_OP_LOG, FORTIS_OP_TANH, FORTIS_OP_F32 };

#define FORTIS_MAX_ARRAYS 8
#define FORTIS_MAX_REFS 128   /* e.g. a 5 x 5 neighbourhood of five arrays */
#define FORTIS_MAX_SCAL 8
#define FORTIS_MAX_INS 32
#define FORTIS_MAX_CONST 16

typedef struct {
    int  narrays;
    long total[FORTIS_MAX_ARRAYS];     /* elements of each host array */
    long plane[FORTIS_MAX_ARRAYS];     /* elements per enclosing-loop iteration (== total for 2-D arrays) */
    int  nrefs;                        /* gather: feature slots in order; scatter: one store per output slot */
    fortis_ref_t refs[FORTIS_MAX_REFS];
    int  nscal;
    fortis_ref_t scal[FORTIS_MAX_SCAL];
    int  nins;
    fortis_ins_t ins[FORTIS_MAX_INS];
    int  nconst;
    float consts[FORTIS_MAX_CONST];
    long count;                        /* cells per enclosing-loop iteration */
    int  nk, klo;                      /* enclosing-loop distribution: trip count and first index (nk = 1: none) */
    int  nargs;                        /* leading int arguments of the generated entry (enclosing-loop variables) */
    int  ilo, jlo, ni, nj;             /* visited rectangle (1-based lower bounds) */
    int  sx;                           /* leading dimension of the cell plane, for the cell list */
    const int* cells;                  /* optional host list of `count` 0-based cell indices (i-1)+(j-1)*sx;
                                          NULL = the rectangle.  Copied to the device at config; the
                                          device-resident calls (fortis_stencil_*_dev, _step_fused) copy it the
                                          first time they see a table with these contents and this list (compared
                                          by value on every call), and equal lists share one device copy. */
    int  elt[FORTIS_MAX_ARRAYS];       /* bytes per element of each host array: 4 (or 0) fp32, 8 fp64
                                          (the descriptor's "elt", driver/fortis_gather_emit.py:13) */
    int  cdouble[FORTIS_MAX_CONST];    /* constant n is a C double literal: its value is dconsts[n], not consts[n] */
    double dconsts[FORTIS_MAX_CONST];
} fortis_stencil_t;

/* Validates a table without touching the GPU (ranges, and that the expressions form one chain on
 * the slot value); what *_config and the device-resident forms check first. */
int  fortis_stencil_check(const fortis_stencil_t* t);
int  fortis_gather_config(const fortis_stencil_t* g);
int  fortis_scatter_config(const fortis_stencil_t* s);
/* Generic forms of the generated entries.  a: the enclosing-loop index arguments (1-based
 * Fortran values; none for the gather under loop distribution); H: the host arrays in
 * descriptor order.  fortis_gather_v: async H2D of the planes it needs, then the gather kernel
 * writing the model input (mom6_zb/gather.cu:50-57).  fortis_scatter_v: H2D of the arrays it
 * only reads, scatter kernel on the model output of iteration a[0], device->host copy of the
 * visited rectangle of every written array, stream sync (mom6_zb/gather.cu:82-91). */
void fortis_gather_v(const int* a, const void* const* H);
void fortis_scatter_v(const int* a, void* const* H);
/* The checked-in ZB instance's exact signatures (mom6_zb/gather.cu:50, :82). */
void fortis_gather(const float* H0, const float* H1, const float* H2, const float* H3);
void fortis_scatter(int a0, float* H0, float* H1, float* H2, float* H3, float* H4);

/* Device-resident forms (arrays already in HBM; nothing is copied).  dA: device pointers in
 * descriptor order.  Asynchronous on the persistent stream. */
/* (With fp64 arrays in the table the matching entries of dA point to doubles.) */
/* Host cost per call: the table is looked up in a small cache by its contents; a cell list at the address and with the
 * count of the entry's last match is compared by 1024 sampled entries (microseconds), at a new address in full
 * (4 bytes per cell).  A list rewritten in place must change its address, its count or a sampled entry to be seen. */
void fortis_stencil_gather_dev(const fortis_stencil_t* g, const float* const* dA, float* dX);
void fortis_stencil_scatter_dev(const fortis_stencil_t* s, float* const* dA, const float* dY, int kk);
/* All nk iterations in one launch: dY is the model output of every iteration, [nk][count][n]; an array that is 2-D on
 * the host (rewritten by every iteration there, like Txy_h) has nk planes of `total` elements on the device.  What
 * fortis_scatter does under loop distribution (mom6_zb/kdist.json, mom6_zb/gather.cu:82-91 run nk times).  -1: bad table. */
int  fortis_stencil_scatter_all_dev(const fortis_stencil_t* s, float* const* dA, const float* dY);
/* The whole lifted step in ONE kernel: gather (g) -> MLP chain (plan p, every op a linear or a
 * feature scale) -> scatter (s) for all nk iterations at once.  Arrays the scatter writes need a
 * plane per iteration on the device: an array that is 2-D on the host (written once per
 * iteration, like Txy_h) is given nk planes of `plane` elements.  dY (optional) also receives the
 * raw model output.  Returns -1 if the plan is not such a chain or is too wide for the kernel. */
int  fortis_stencil_step_fused(const fortis_stencil_t* g, const fortis_stencil_t* s, fortis_plan* p,
                               const float* const* dG, float* const* dS, float* dY);

/* ================================ timing helper ========================================= */
/* Runs fn(arg) `iters` times on the persistent stream between two HIP events on that stream and
 * returns the elapsed milliseconds (the benchmark's per-kernel clock). */
float fortis_time_ms(void (*fn)(void*), void* arg, int iters);
/* A step made of `nparts` (at most 16) enqueues fns[k](args[k]), run `iters` (at most 4096) times with a
 * HIP event between the parts and no host wait inside: ms_out[k] receives the elapsed milliseconds of
 * part k summed over the iterations.  Returns -1 on bad arguments. */
int   fortis_time_parts_ms(int nparts, void (*const* fns)(void*), void* const* args, int iters, float* ms_out);
/* Same clock around `iters` enqueues of a plan (use_graph: captured once, then replayed) and of
 * the fused stencil step. */
float fortis_plan_time_ms(fortis_plan* p, int iters, int use_graph);
float fortis_stencil_step_fused_time_ms(const fortis_stencil_t* g, const fortis_stencil_t* s, fortis_plan* p,
                                        const float* const* dG, float* const* dS, float* dY, int iters);
/* Per-kernel clock: while enabled, every fortis_plan_run records a HIP event on the persistent
 * stream before its first and after each of its kernels.  fortis_plan_profile_read adds up the
 * elapsed milliseconds per kernel over the passes recorded since the last read, returns the
 * number of passes and starts over.  fortis_plan_kernel_name names kernel idx of the pass. */
void  fortis_plan_profile(fortis_plan* p, int enable);
int   fortis_plan_profile_read(fortis_plan* p, float* ms_per_kernel);
const char* fortis_plan_kernel_name(fortis_plan* p, int idx);

/* ================================ test hooks ============================================ */
/* No reference counterpart; host-only, usable without a GPU.
 * fortis_gemm_schedule: the persistent GEMM's work list for C[B][N] on `slots` resident workgroups, as
 *   (level, first 128 x 128 tile, items) triples, level 0 whole tiles, 1 halves (128 x 64), 2 quarters
 *   (64 x 64); returns the number of phases (at most 4), -1 on bad arguments.
 * fortis_magic_divmod: n / d and n % d by the exact multiply-shift the stencil kernels decode cells with.
 * fortis_stencil_route: which kernels a stencil table takes: 0 the fused-form ones (fp32 arrays, one chain
 *   of + - * / on the slot value), 1 the general ones, -1 the table is invalid. */
int  fortis_gemm_schedule(long B, long N, long slots, long* triples);
int  fortis_stencil_route(const fortis_stencil_t* t);
void fortis_magic_divmod(unsigned n, unsigned d, unsigned* q, unsigned* r);

#ifdef __cplusplus
}
#endif
#endif
