/*
 * fortis_oracle.c -- CPU restatement of the FORTIS fused-inference-step algorithms.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product library links, loads or calls this file.
 * It is the checker for the HIP kernels (tests/, the smoke check) and the scalar/OpenMP CPU
 * baseline that the benchmark times beside the GPU.  Every function cites the reference file
 * and lines whose arithmetic it restates (paths relative to the reference tree).
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off; contraction off so fp32 gather/scatter
 * expressions round exactly like the reference's `-fmad=false` CUDA and its Fortran host).
 *
 * How each function is pinned (the tests that do it live in tests/test_oracle_*.py):
 *   orc_zb_fields / orc_zb_prep / orc_zb_step_native
 *        bit-compared against the output of the reference's own Fortran host + native forward
 *        (mom6_zb/zb_host.f90 + fwd_native_zb.f90, built by oracle/build_ref.sh with flang),
 *        via tests/golden/zb_native_golden.npz.
 *   orc_mlp_native / orc_mlp_native_t / orc_mlp_f64
 *        reference-held known answer x_test -> y_test in mom6_zb/zb_nn.npz (copied as a data
 *        fixture to tests/golden/zb_nn.npz); README stamp 7.775037 for the toy MLP.
 *   orc_stencil_gather / orc_stencil_scatter
 *        brute-force comparison with the Fortran host's RESHAPE order through orc_zb_step_native
 *        (which does not call them) and with the closed-form index expressions of mom6_zb/gather.cu.
 *   orc_conv3d / orc_conv2d / orc_convt2d / orc_maxpool2d / orc_upsample_nearest / orc_bn_eval
 *        README stamp 9617.28 (conv probe) and torch.nn.functional on CPU for the op micro-suite models.
 *   orc_boundary_pre / orc_boundary_post
 *        closed form; post(pre(A)) with unit scale is the identity on A (transpose round trip).
 *   orc_gemm      numpy float64 matmul.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define IDX2(i, j, sx) ((size_t)((i) - 1) + (size_t)((j) - 1) * (size_t)(sx))
#define IDX3(i, j, k, sx, sy) (IDX2(i, j, sx) + (size_t)((k) - 1) * (size_t)(sx) * (size_t)(sy))

/* ------------------------------------------------------------------------------------------
 * ZB host: field synthesis.  mom6_zb/zb_host.f90:37-40 (three make_field calls sharing one
 * LCG seed), :124-135 (make_field).  Values are computed in fp64 and cast to fp32.
 * ---------------------------------------------------------------------------------------- */
static void make_field(int64_t* seed, int sx, int sy, int nz, double a, double b, double c, float* out)
{
    for (int k = 1; k <= nz; k++)
        for (int j = 1; j <= sy; j++)
            for (int i = 1; i <= sx; i++) {
                *seed = (*seed * 1103515245LL + 12345LL) % 2147483648LL;
                double r = (double)(*seed) / 2147483648.0 - 0.5;
                double f = 1e-5 * (0.6 * sin(a * i + b * j + c * k) * cos(b * i - a * j) + 0.4 * r);
                out[IDX3(i, j, k, sx, sy)] = (float)f;
            }
}

void orc_zb_fields(int sx, int sy, int nz, float* sh_xy, float* sh_xx, float* vort_xy,
                   float* mask2dT, float* mask2dBu, float* kappa_h)
{
    int64_t seed = 12345;
    make_field(&seed, sx, sy, nz, 0.31, 0.23, 0.17, sh_xy);
    make_field(&seed, sx, sy, nz, 0.27, 0.19, 0.13, sh_xx);
    make_field(&seed, sx, sy, nz, 0.29, 0.21, 0.11, vort_xy);
    /* zb_host.f90:41-46: unit masks with a zero one-cell border; kappa_h = -amplitude*areaT*mask */
    const float amplitude = 1.0f, areaT = 6.25e8f;
    for (int j = 1; j <= sy; j++)
        for (int i = 1; i <= sx; i++) {
            float m = (i == 1 || i == sx || j == 1 || j == sy) ? 0.0f : 1.0f;
            mask2dT[IDX2(i, j, sx)] = m;
            mask2dBu[IDX2(i, j, sx)] = m;
            kappa_h[IDX2(i, j, sx)] = -amplitude * areaT * m;
        }
}

/* ------------------------------------------------------------------------------------------
 * ZB host: per-step feature interpolation and stencil norm.  mom6_zb/zb_host.f90:52-75.
 * halo is the halo width (4 in the reference); is=halo+1, ie=sx-halo, js=halo+1, je=sy-halo.
 * ---------------------------------------------------------------------------------------- */
void orc_zb_prep(int sx, int sy, int nz, int halo, const float* sh_xy, const float* sh_xx,
                 const float* vort_xy, const float* mask2dT, float* sh_xy_h, float* vort_xy_h,
                 float* norm_h)
{
    const int is = halo + 1, ie = sx - halo, js = halo + 1, je = sy - halo;
    size_t n3 = (size_t)sx * sy * nz;
    memset(sh_xy_h, 0, n3 * sizeof(float));
    memset(vort_xy_h, 0, n3 * sizeof(float));
    memset(norm_h, 0, n3 * sizeof(float));
    float* sqr_h = (float*)calloc((size_t)sx * sy, sizeof(float));
    for (int k = 1; k <= nz; k++) {
        for (int j = js - 3; j <= je + 3; j++)
            for (int i = is - 3; i <= ie + 3; i++) {
                float a = 0.25f * ((sh_xy[IDX3(i - 1, j - 1, k, sx, sy)] + sh_xy[IDX3(i, j, k, sx, sy)]) +
                                   (sh_xy[IDX3(i - 1, j, k, sx, sy)] + sh_xy[IDX3(i, j - 1, k, sx, sy)]));
                float v = 0.25f * ((vort_xy[IDX3(i - 1, j - 1, k, sx, sy)] + vort_xy[IDX3(i, j, k, sx, sy)]) +
                                   (vort_xy[IDX3(i - 1, j, k, sx, sy)] + vort_xy[IDX3(i, j - 1, k, sx, sy)]));
                sh_xy_h[IDX3(i, j, k, sx, sy)] = a;
                vort_xy_h[IDX3(i, j, k, sx, sy)] = v;
                float xx = sh_xx[IDX3(i, j, k, sx, sy)];
                float s = xx * xx + a * a;
                s = s + v * v;
                sqr_h[IDX2(i, j, sx)] = s * mask2dT[IDX2(i, j, sx)];
            }
        for (int j = js - 2; j <= je + 2; j++)
            for (int i = is - 2; i <= ie + 2; i++) {
                float tmp = 0.0f;
                for (int jj = j - 1; jj <= j + 1; jj++)
                    for (int ii = i - 1; ii <= i + 1; ii++) tmp = tmp + sqr_h[IDX2(ii, jj, sx)];
                norm_h[IDX3(i, j, k, sx, sy)] = sqrtf(tmp);
            }
    }
    free(sqr_h);
}

/* ------------------------------------------------------------------------------------------
 * Native per-column MLP, the shipped ANN_apply: divide by input_norms, Layer_apply loops
 * (input index outer, output index inner, y(j) += x(i)*A(j,i)), bias, ReLU on hidden layers,
 * multiply by output_norms.  mom6_zb/fwd_native_zb.f90:30-48 (Layer_apply), :51-77 (ANN_apply).
 * Generalised to L layers; W[l] is [n_out][n_in] row-major (== Fortran A(j,i) read as A0[j][i],
 * the npz orientation, mom6_zb/make_zb_weights.py:12-17).  All arithmetic fp32, no FMA.
 * in_norms / out_norms may be NULL.
 * ---------------------------------------------------------------------------------------- */
void orc_mlp_native(int nlayers, const int* widths, const float* const* W, const float* const* b,
                    const float* in_norms, const float* out_norms, long rows, const float* X, float* Y)
{
    int maxw = 0;
    for (int l = 0; l <= nlayers; l++) if (widths[l] > maxw) maxw = widths[l];
#pragma omp parallel if (rows > 256)
    {
        float* x1 = (float*)malloc(sizeof(float) * maxw);
        float* x2 = (float*)malloc(sizeof(float) * maxw);
#pragma omp for schedule(static)
        for (long r = 0; r < rows; r++) {
            const float* x = X + (size_t)r * widths[0];
            for (int i = 0; i < widths[0]; i++) x1[i] = in_norms ? x[i] / in_norms[i] : x[i];
            for (int l = 0; l < nlayers; l++) {
                const int ni = widths[l], no = widths[l + 1];
                for (int j = 0; j < no; j++) x2[j] = 0.0f;
                for (int i = 0; i < ni; i++)
                    for (int j = 0; j < no; j++) x2[j] = x2[j] + (x1[i] * W[l][(size_t)j * ni + i]);
                for (int j = 0; j < no; j++) {
                    x2[j] = x2[j] + b[l][j];
                    if (l < nlayers - 1) x2[j] = x2[j] > 0.0f ? x2[j] : 0.0f;
                }
                float* t = x1; x1 = x2; x2 = t;
            }
            float* y = Y + (size_t)r * widths[nlayers];
            for (int j = 0; j < widths[nlayers]; j++) y[j] = out_norms ? x1[j] * out_norms[j] : x1[j];
        }
        free(x1); free(x2);
    }
}

/* The same native loop nest with the weights held as the Fortran code holds them, A(out, in)
 * column-major, i.e. Wt[l] is [n_in][n_out] with the output index contiguous, so the inner j loop
 * is unit stride exactly as in Layer_apply (mom6_zb/fwd_native_zb.f90:37-41).  Same arithmetic and
 * order as orc_mlp_native (bit-identical for ReLU networks; the test suite checks that), plus
 * LeakyReLU for the ClimSim-shaped network.  This is the CPU baseline the benchmark times:
 * columns in parallel over OpenMP threads, one column through all layers at a time. */
void orc_mlp_native_t(int nlayers, const int* widths, const float* const* Wt, const float* const* b,
                      const int* act, const float* alpha, const float* in_norms, const float* out_norms,
                      long rows, const float* X, float* Y)
{
    int maxw = 0;
    for (int l = 0; l <= nlayers; l++) if (widths[l] > maxw) maxw = widths[l];
#pragma omp parallel if (rows > 64)
    {
        float* x1 = (float*)malloc(sizeof(float) * maxw);
        float* x2 = (float*)malloc(sizeof(float) * maxw);
#pragma omp for schedule(static)
        for (long r = 0; r < rows; r++) {
            const float* x = X + (size_t)r * widths[0];
            for (int i = 0; i < widths[0]; i++) x1[i] = in_norms ? x[i] / in_norms[i] : x[i];
            for (int l = 0; l < nlayers; l++) {
                const int ni = widths[l], no = widths[l + 1];
                for (int j = 0; j < no; j++) x2[j] = 0.0f;
                for (int i = 0; i < ni; i++) {
                    const float xi = x1[i];
                    const float* w = Wt[l] + (size_t)i * no;
                    for (int j = 0; j < no; j++) x2[j] = x2[j] + (xi * w[j]);
                }
                for (int j = 0; j < no; j++) {
                    float v = x2[j] + b[l][j];
                    if (act[l] == 1) v = v > 0.0f ? v : 0.0f;
                    else if (act[l] == 2) v = v > 0.0f ? v : alpha[l] * v;
                    x2[j] = v;
                }
                float* t = x1; x1 = x2; x2 = t;
            }
            float* y = Y + (size_t)r * widths[nlayers];
            for (int j = 0; j < widths[nlayers]; j++) y[j] = out_norms ? x1[j] * out_norms[j] : x1[j];
        }
        free(x1); free(x2);
    }
}

/* ------------------------------------------------------------------------------------------
 * Ground-truth MLP with fp64 accumulation: the chain fortis-fuse lowers to
 * (fortis_gemm -> epilogue kernel)*L.  C[b][n] = sum_k A[b][k]*W[n][k]  (runtime/fortis_rt.c:45-75),
 * epilogue = bias add then activation in program order (compiler/FortisFuse.cpp:685-692, 721-760).
 * Layer outputs are rounded to fp32 between layers (each layer's result is an fp32 buffer in the
 * reference).  act[l]: 0 none, 1 ReLU max(x,0), 2 LeakyReLU x>0?x:alpha*x.
 * Optional input scale x/in_norms (mom6_zb/export_zb.py:14) and output scale *out_norms, and the
 * ClimSim mask head y + mask*(relu(y)-y) on the last mask_tail outputs (benchmarks/climsim/export_wide.py:28).
 * ---------------------------------------------------------------------------------------- */
void orc_mlp_f64(int nlayers, const int* widths, const float* const* W, const float* const* b,
                 const int* act, const float* alpha, const float* in_norms, const float* out_norms,
                 int mask_tail, long rows, const float* X, float* Y)
{
    int maxw = 0;
    for (int l = 0; l <= nlayers; l++) if (widths[l] > maxw) maxw = widths[l];
#pragma omp parallel if (rows > 256)
    {
        float* x1 = (float*)malloc(sizeof(float) * maxw);
        float* x2 = (float*)malloc(sizeof(float) * maxw);
#pragma omp for schedule(static)
        for (long r = 0; r < rows; r++) {
            const float* x = X + (size_t)r * widths[0];
            for (int i = 0; i < widths[0]; i++) x1[i] = in_norms ? x[i] / in_norms[i] : x[i];
            for (int l = 0; l < nlayers; l++) {
                const int ni = widths[l], no = widths[l + 1];
                for (int j = 0; j < no; j++) {
                    double acc = 0.0;
                    const float* w = W[l] + (size_t)j * ni;
                    for (int i = 0; i < ni; i++) acc += (double)x1[i] * (double)w[i];
                    float v = (float)acc;
                    if (b && b[l]) v = v + b[l][j];
                    if (act[l] == 1) v = v > 0.0f ? v : 0.0f;
                    else if (act[l] == 2) v = v > 0.0f ? v : alpha[l] * v;
                    x2[j] = v;
                }
                float* t = x1; x1 = x2; x2 = t;
            }
            const int no = widths[nlayers];
            float* y = Y + (size_t)r * no;
            for (int j = 0; j < no; j++) {
                float v = out_norms ? x1[j] * out_norms[j] : x1[j];
                if (j >= no - mask_tail) v = v > 0.0f ? v : 0.0f;
                y[j] = v;
            }
        }
        free(x1); free(x2);
    }
}

/* C[B][N] = A[B][K] . W[N][K]^T, beta = 0.  runtime/fortis_rt.c:45-75.  fp64 accumulate. */
void orc_gemm(long B, long N, long K, const float* A, const float* W, float* C)
{
#pragma omp parallel for schedule(static)
    for (long bi = 0; bi < B; bi++)
        for (long n = 0; n < N; n++) {
            double acc = 0.0;
            for (long k = 0; k < K; k++) acc += (double)A[bi * K + k] * (double)W[n * K + k];
            C[bi * N + n] = (float)acc;
        }
}

/* ------------------------------------------------------------------------------------------
 * Stencil gather / scatter, descriptor driven.
 * Generic form: driver/fortis_gather_emit.py:49-97; checked-in instance: mom6_zb/gather.cu:14-49
 * (gather kernel) and :58-81 (scatter kernel).
 *
 * A "ref" addresses one element of one host array relative to the cell (i, j) (1-based Fortran
 * indices) and the enclosing-loop plane kk (0-based):
 *      elem = base + i*si + j*sj + (planar ? kk*plane : 0)
 * where base already holds the (offset-1)*stride terms.  For A(i+di, j+dj, k) on a column-major
 * (sx, sy, nk) array: si = 1, sj = sx, base = (di-1) + (dj-1)*sx, plane = sx*sy.
 *
 * Expressions are straight-line programs over fp32 values: each instruction is
 *      {op, a, b}:  r[next] = operand(a) op operand(b)
 * operand code: 0 = tv (the slot value as loaded), 1..8 = scalar S0..S7, 16+n = constant n,
 * 32+n = result of instruction n.  op: 0 add, 1 sub, 2 mul, 3 div.  The value of the last
 * instruction replaces tv.  Each op is one IEEE fp32 operation, never contracted.
 *
 * Cells: row = kk*count + col.  If cells == NULL the visited set is the rectangle
 * i = ilo + col % ni, j = jlo + col / ni (gather.cu:15-16); otherwise cells[col] is the
 * 0-based linear index (i-1) + (j-1)*sx of an active cell on the (sx, *) plane.
 * ---------------------------------------------------------------------------------------- */
typedef struct { int array; int planar; long base, si, sj, plane; } orc_ref_t;
typedef struct { int op, a, b; } orc_ins_t;

static float eval_prog(int nins, const orc_ins_t* ins, const float* consts, float tv, const float* S)
{
    float r[32];
    float v = tv;
    for (int n = 0; n < nins; n++) {
        float o[2];
        int code[2] = { ins[n].a, ins[n].b };
        for (int s = 0; s < 2; s++) {
            int c = code[s];
            o[s] = c == 0 ? tv : c < 16 ? S[c - 1] : c < 32 ? consts[c - 16] : r[c - 32];
        }
        switch (ins[n].op) {
            case 0: v = o[0] + o[1]; break;
            case 1: v = o[0] - o[1]; break;
            case 2: v = o[0] * o[1]; break;
            default: v = o[0] / o[1]; break;
        }
        r[n] = v;
    }
    return v;
}

static void cell_ij(long col, const int* cells, int sx, int ilo, int jlo, int ni, int* i, int* j)
{
    if (cells) { *i = 1 + cells[col] % sx; *j = 1 + cells[col] / sx; }
    else { *i = ilo + (int)(col % ni); *j = jlo + (int)(col / ni); }
}

void orc_stencil_gather(int nslots, const orc_ref_t* slots, int nscal, const orc_ref_t* scal,
                        int nins, const orc_ins_t* ins, const float* consts,
                        const float* const* arrays, long count, int nk, const int* cells, int sx,
                        int ilo, int jlo, int ni, float* X)
{
    for (long row = 0; row < count * nk; row++) {
        long col = row % count; int kk = (int)(row / count);
        int i, j; cell_ij(col, cells, sx, ilo, jlo, ni, &i, &j);
        float S[8];
        for (int s = 0; s < nscal; s++)
            S[s] = arrays[scal[s].array][scal[s].base + i * scal[s].si + j * scal[s].sj + (scal[s].planar ? kk * scal[s].plane : 0)];
        for (int q = 0; q < nslots; q++) {
            float tv = arrays[slots[q].array][slots[q].base + i * slots[q].si + j * slots[q].sj + (slots[q].planar ? kk * slots[q].plane : 0)];
            X[(size_t)row * nslots + q] = nins ? eval_prog(nins, ins, consts, tv, S) : tv;
        }
    }
}

/* One enclosing-loop iteration kk (0-based) of the scatter: Y is the model output of that layer,
 * [count][nout]; stores[q] says where slot q goes.  gather.cu:67-81. */
void orc_stencil_scatter(int nout, const orc_ref_t* stores, int nscal, const orc_ref_t* scal,
                         int nins, const orc_ins_t* ins, const float* consts,
                         float* const* arrays, long count, int kk, const int* cells, int sx,
                         int ilo, int jlo, int ni, const float* Y)
{
    for (long col = 0; col < count; col++) {
        int i, j; cell_ij(col, cells, sx, ilo, jlo, ni, &i, &j);
        float S[8];
        for (int s = 0; s < nscal; s++)
            S[s] = arrays[scal[s].array][scal[s].base + i * scal[s].si + j * scal[s].sj + (scal[s].planar ? kk * scal[s].plane : 0)];
        for (int q = 0; q < nout; q++) {
            float tv = Y[(size_t)col * nout + q];
            if (nins) tv = eval_prog(nins, ins, consts, tv, S);
            arrays[stores[q].array][stores[q].base + i * stores[q].si + j * stores[q].sj + (stores[q].planar ? kk * stores[q].plane : 0)] = tv;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Whole ZB step exactly as the Fortran host does it, cell by cell: RESHAPE stencil packing,
 * x/(norm+1e-30), native MLP, y*norm*norm*kappa, stores, corner interpolation of Txy_h.
 * mom6_zb/zb_host.f90:77-107.  Written from the Fortran, NOT through orc_stencil_* (so that
 * those are checked against this).  Txx/Tyy/Txy are (sx,sy,nz), Txy_h is (sx,sy); callers
 * zero them first (zb_host.f90:47).
 * ---------------------------------------------------------------------------------------- */
void orc_zb_step_native(int sx, int sy, int nz, int halo, const float* sh_xy_h, const float* sh_xx,
                        const float* vort_xy_h, const float* norm_h, const float* kappa_h,
                        const float* mask2dBu, int nlayers, const int* widths,
                        const float* const* W, const float* const* b, const float* in_norms,
                        const float* out_norms, float* Txx, float* Tyy, float* Txy, float* Txy_h)
{
    const int is = halo + 1, ie = sx - halo, js = halo + 1, je = sy - halo;
    const int Isq = is - 1, Ieq = ie, Jsq = js - 1, Jeq = je;
    const float subroundoff_shear = 1.0e-30f;
    float x[27], y[8];
    for (int k = 1; k <= nz; k++) {
        for (int j = js - 2; j <= je + 2; j++)
            for (int i = is - 2; i <= ie + 2; i++) {
                int q = 0;
                const float* F[3] = { sh_xy_h, sh_xx, vort_xy_h };
                for (int f = 0; f < 3; f++)
                    for (int jj = j - 1; jj <= j + 1; jj++)       /* RESHAPE: column-major, i fastest */
                        for (int ii = i - 1; ii <= i + 1; ii++) x[q++] = F[f][IDX3(ii, jj, k, sx, sy)];
                float input_norm = norm_h[IDX3(i, j, k, sx, sy)];
                float d = input_norm + subroundoff_shear;
                for (q = 0; q < 27; q++) x[q] = x[q] / d;
                orc_mlp_native(nlayers, widths, W, b, in_norms, out_norms, 1, x, y);
                for (q = 0; q < 3; q++) y[q] = ((y[q] * input_norm) * input_norm) * kappa_h[IDX2(i, j, sx)];
                Txy_h[IDX2(i, j, sx)] = y[0];
                Txx[IDX3(i, j, k, sx, sy)] = y[1];
                Tyy[IDX3(i, j, k, sx, sy)] = y[2];
            }
        for (int j = Jsq - 1; j <= Jeq + 1; j++)
            for (int i = Isq - 1; i <= Ieq + 1; i++)
                Txy[IDX3(i, j, k, sx, sy)] =
                    0.25f * ((Txy_h[IDX2(i + 1, j + 1, sx)] + Txy_h[IDX2(i, j, sx)]) +
                             (Txy_h[IDX2(i + 1, j, sx)] + Txy_h[IDX2(i, j + 1, sx)])) * mask2dBu[IDX2(i, j, sx)];
    }
}

/* ------------------------------------------------------------------------------------------
 * Boundary pre/post (column-major host arrays <-> batch-major fp32 activations).
 * trt_backend/e3sm_boundary.cu:9-14 (pre), :15-20 (post); MLIR form driver/fortis_emit2d.py:20-52.
 * Arithmetic is done in the host element type, then cast.
 * ---------------------------------------------------------------------------------------- */
void orc_boundary_pre_f64(long NI, long NK, const double* A, const double* mean, const double* vmax,
                          const double* vmin, float* X)
{
    for (long i = 0; i < NI; i++)
        for (long k = 0; k < NK; k++) {
            double a = A[i + NI * k];
            a = ((a - mean[k]) / (vmax[k] - vmin[k]));
            X[i * NK + k] = (float)a;
        }
}
void orc_boundary_post_f64(long NI, long NK, const float* Y, const double* scale, double* B)
{
    for (long i = 0; i < NI; i++)
        for (long k = 0; k < NK; k++) {
            double v = (double)Y[i * NK + k];
            v = (v / scale[k]);
            B[i + NI * k] = v;
        }
}
void orc_boundary_pre_f32(long NI, long NK, const float* A, const float* mean, const float* vmax,
                          const float* vmin, float* X)
{
    for (long i = 0; i < NI; i++)
        for (long k = 0; k < NK; k++) {
            float a = A[i + NI * k];
            a = ((a - mean[k]) / (vmax[k] - vmin[k]));
            X[i * NK + k] = a;
        }
}
void orc_boundary_post_f32(long NI, long NK, const float* Y, const float* scale, float* B)
{
    for (long i = 0; i < NI; i++)
        for (long k = 0; k < NK; k++) B[i + NI * k] = Y[i * NK + k] / scale[k];
}

/* ------------------------------------------------------------------------------------------
 * Convolutions: cross-correlation, NCHW / NCDHW, weights [F][C][K..], zero padding by bounds
 * check, fp64 accumulation (ground truth).  Semantics: runtime/fortis_rt.c:108-127 (conv2d
 * contract), runtime/fortis_fft.cu:149-201 (direct conv3d: y[f][z][y][x] = sum_c sum_k
 * x[c][z+kd-pd][y+kh-ph][x+kw-pw] * w[f][c][kd][kh][kw]).
 * ---------------------------------------------------------------------------------------- */
void orc_conv3d(long N, long C, long D, long H, long Wd, long F, long KD, long KH, long KW,
                long Do, long Ho, long Wo, long sd, long sh, long sw, long pd, long ph, long pw,
                const float* x, const float* w, float* y)
{
#pragma omp parallel for collapse(2) schedule(static)
    for (long n = 0; n < N; n++)
        for (long f = 0; f < F; f++)
            for (long oz = 0; oz < Do; oz++)
                for (long oy = 0; oy < Ho; oy++)
                    for (long ox = 0; ox < Wo; ox++) {
                        double acc = 0.0;
                        for (long c = 0; c < C; c++)
                            for (long kd = 0; kd < KD; kd++) {
                                long iz = oz * sd + kd - pd; if (iz < 0 || iz >= D) continue;
                                for (long kh = 0; kh < KH; kh++) {
                                    long iy = oy * sh + kh - ph; if (iy < 0 || iy >= H) continue;
                                    for (long kw = 0; kw < KW; kw++) {
                                        long ix = ox * sw + kw - pw; if (ix < 0 || ix >= Wd) continue;
                                        acc += (double)x[(((n * C + c) * D + iz) * H + iy) * Wd + ix] *
                                               (double)w[((((f * C + c) * KD + kd) * KH + kh) * KW) + kw];
                                    }
                                }
                            }
                        y[(((n * F + f) * Do + oz) * Ho + oy) * Wo + ox] = (float)acc;
                    }
}

void orc_conv2d(long N, long C, long H, long Wd, long F, long KH, long KW, long Ho, long Wo,
                long sh, long sw, long ph, long pw, const float* x, const float* w, float* y)
{
    orc_conv3d(N, C, 1, H, Wd, F, 1, KH, KW, 1, Ho, Wo, 1, sh, sw, 0, ph, pw, x, w, y);
}

/* Transposed conv2d, PyTorch weight layout [C][F][KH][KW]; scatter form:
 * y[f][iy*s - p + kh][ix*s - p + kw] += x[c][iy][ix] * w[c][f][kh][kw].  Reaches the reference's
 * fuser as zero-insertion + flipped-kernel conv (tests/optest.py:9-12 are its op tests). */
void orc_convt2d(long C, long H, long Wd, long F, long KH, long KW, long Ho, long Wo, long s, long p,
                 const float* x, const float* w, float* y)
{
    double* acc = (double*)calloc((size_t)F * Ho * Wo, sizeof(double));
    for (long c = 0; c < C; c++)
        for (long iy = 0; iy < H; iy++)
            for (long ix = 0; ix < Wd; ix++) {
                double xv = x[(c * H + iy) * Wd + ix];
                for (long f = 0; f < F; f++)
                    for (long kh = 0; kh < KH; kh++) {
                        long oy = iy * s - p + kh; if (oy < 0 || oy >= Ho) continue;
                        for (long kw = 0; kw < KW; kw++) {
                            long ox = ix * s - p + kw; if (ox < 0 || ox >= Wo) continue;
                            acc[(f * Ho + oy) * Wo + ox] += xv * (double)w[((c * F + f) * KH + kh) * KW + kw];
                        }
                    }
            }
    for (long t = 0; t < F * Ho * Wo; t++) y[t] = (float)acc[t];
    free(acc);
}

/* maxpool k x k stride k (non-additive reduction, init -inf: compiler/FortisFuse.cpp:667-672) */
void orc_maxpool2d(long C, long H, long Wd, long k, const float* x, float* y)
{
    long Ho = H / k, Wo = Wd / k;
    for (long c = 0; c < C; c++)
        for (long oy = 0; oy < Ho; oy++)
            for (long ox = 0; ox < Wo; ox++) {
                float m = -INFINITY;
                for (long a = 0; a < k; a++)
                    for (long bb = 0; bb < k; bb++) {
                        float v = x[(c * H + oy * k + a) * Wd + ox * k + bb];
                        m = v > m ? v : m;
                    }
                y[(c * Ho + oy) * Wo + ox] = m;
            }
}

/* nearest upsample by integer factor s over the trailing nd (2 or 3) spatial dims; index gather */
void orc_upsample_nearest(long C, long D, long H, long Wd, long s, int nd, const float* x, float* y)
{
    long sd = nd == 3 ? s : 1;
    long Do = D * sd, Ho = H * s, Wo = Wd * s;
    for (long c = 0; c < C; c++)
        for (long z = 0; z < Do; z++)
            for (long yy = 0; yy < Ho; yy++)
                for (long xx = 0; xx < Wo; xx++)
                    y[((c * Do + z) * Ho + yy) * Wo + xx] = x[((c * D + z / sd) * H + yy / s) * Wd + xx / s];
}

/* BatchNorm eval affine, per channel: (x - mean) / sqrt(var + eps) * gamma + beta, fp32 in
 * PyTorch's operation order. */
void orc_bn_eval(long C, long S, const float* mean, const float* var, const float* gamma,
                 const float* beta, float eps, const float* x, float* y)
{
    for (long c = 0; c < C; c++) {
        double inv = 1.0 / sqrt((double)var[c] + (double)eps);
        for (long s = 0; s < S; s++)
            y[c * S + s] = (float)(((double)x[c * S + s] - (double)mean[c]) * inv * (double)gamma[c] + (double)beta[c]);
    }
}
