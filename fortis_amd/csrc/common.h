// Internal declarations shared by the HIP sources of libfortis_rt.
#pragma once
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "../../include/fortis_rt.h"
#include "../../include/fortis_step.h"

// A failed runtime call is reported and counted and the library goes on, as the runtime it stands in for does
// (runtime/fortis_rt.c:30-34, 124, 153 print and return); fortis_error_count() lets a caller that wants to stop on
// the first failure see it.
extern "C" void fortis_note_error(void);
#define HIP_OK(call)                                                                              \
    do {                                                                                          \
        hipError_t e_ = (call);                                                                   \
        if (e_ != hipSuccess) {                                                                   \
            fprintf(stderr, "fortis: %s failed: %s (%s:%d)\n", #call, hipGetErrorString(e_), __FILE__, __LINE__); \
            fortis_note_error();                                                                  \
        }                                                                                         \
    } while (0)

// Raw device memory for what the library keeps itself (weights, tables, staging planes): hipMalloc / hipFree
// behind the same switchable allocator as the pool (fortis_pool_set_allocator), so that a test can make any of
// these allocations fail.  fortis_dev_malloc returns 0, or -1 after printing what could not be allocated; a
// caller that gets -1 must not launch anything on the pointer.
int  fortis_dev_malloc(void** p, size_t nbytes, const char* what);
void fortis_dev_free(void* p);
long fortis_pool_best_fit(long nbytes);   // size of the released pool buffer fortis_alloc(nbytes) would hand out, or -1
bool fortis_pool_on_device();   // false while a test has replaced the raw allocator (fortis_pool_set_allocator)

extern "C" long fortis_step_generation(void);   // plan.hip: count of forward passes of the bound step
static inline hipStream_t fortis_stream_get() { return (hipStream_t)mgpuStreamCreate(); }
static inline long cdiv(long a, long b) { return (a + b - 1) / b; }

// ---- fused GEMM + bias + activation (gemm.hip) -------------------------------------------
// C[B][N] = epi(A[B][K] . W[N][K]^T): + bias[n], activation, * out_scale[n], ReLU on the last
// mask_tail columns.  bias/out_scale may be null.  Returns 0, or -1 on an unsupported shape.
int fortis_launch_gemm(const float* A, const float* W, const float* bias, float* C, long B, long N,
                       long K, int act, float alpha, const float* out_scale, long mask_tail,
                       hipStream_t s);

// ---- fused MLP chain (chain.hip) ----------------------------------------------------------
#define FORTIS_CHAIN_MAX_LAYERS 8
#define FORTIS_CHAIN_MAX_WIDTH 256
struct ChainLayer {
    int K, N, Kp, Np;   // real and padded (to 16) widths
    int woff, boff;     // float offsets of the packed weights / bias inside the blob
    int act;
    float alpha;
};
struct ChainDesc {
    int nlayers;
    ChainLayer L[FORTIS_CHAIN_MAX_LAYERS];
    const float* wall;     // device blob: every layer's packed weights and zero-padded bias
    int wfloats;           // its length in floats (multiple of 4)
    const float* in_div;   // x / in_div[c] before layer 0, or null
    const float* in_rcp;   // refined reciprocals of in_div (fortis_chain_fill_rcp) when every in_div[c] lies in [2^-40, 2^40], else null
    const float* out_mul;  // y * out_mul[c] after the last layer, or null
    int mask_tail;         // ReLU on the last mask_tail outputs
    int ld;                // LDS row pitch in floats
    int x4off;             // last layer with at most 4 outputs: offset of its weights in 4x4x1 order [q][n][Kp/16][4], or -1
};
// Packs the layers (W[l] is [N][K] row-major, b[l] may be null) into one device blob and fills the
// descriptor's shape fields; act/alpha/in_div/out_mul/mask_tail are left to the caller.
int fortis_chain_build(ChainDesc* d, int nlayers, const float* const* W, const float* const* b, const int* K,
                       const int* N, float** blob_out);
void fortis_launch_chain(const ChainDesc& d, const float* X, float* Y, long rows, hipStream_t s, long form_rows = 0);
// rcp[c] = the refined reciprocal of div[c] exactly as the IEEE division sequence forms it (v_rcp_f32 and one Newton
// step), computed on the device so that a kernel dividing many numerators by div[c] can take it from memory.
void fortis_chain_fill_rcp(const float* div, float* rcp, int n, hipStream_t s);
// ---- stencil tables as the kernels see them (stencil.hip) --------------------------------
#define ST_KREFS 32     // slots a kernel launch handles: the fused-form kernels take tables up to this, the general ones chunk
struct CellStep { int op, code, tv_left; };
struct StencilDev {
    int narrays;
    long plane[FORTIS_MAX_ARRAYS];
    int nrefs;
    fortis_ref_t refs[FORTIS_MAX_REFS];
    int nscal;
    fortis_ref_t scal[FORTIS_MAX_SCAL];
    int ncell;                         // per-cell instructions (no tv operand)
    fortis_ins_t cell[FORTIS_MAX_INS];
    int nchain;                        // tv chain: tv = tv op x  or  x op tv
    CellStep chain[FORTIS_MAX_INS];
    float consts[FORTIS_MAX_CONST];
    long count;
    int nk;
    int ilo, jlo, ni, sx;
    const int* cells;                  // device copy of the cell list, or null
};
// Splits the straight-line program into per-cell code and a tv chain.  Returns -1 if tv is used
// in a way that is not a single chain.
int fortis_stencil_lower(const fortis_stencil_t* in, StencilDev* out);
// General kernels for everything else (stencil_generic.hip): fp64 arrays, double literals, the lifter's
// functions, expressions that are not one chain.  dA: device array bases in descriptor order.
int fortis_stencil_validate(const fortis_stencil_t* t);
bool fortis_stencil_typed(const fortis_stencil_t* t);
void fortis_launch_gather_generic(const fortis_stencil_t& t, const int* dcells, const void* const* dA, float* dX, hipStream_t s);
void fortis_launch_scatter_generic(const fortis_stencil_t& t, const int* dcells, void* const* dA, const float* dY, int kk, hipStream_t s);

// ---- elementwise / layout kernels (elementwise.hip) --------------------------------------
void fortis_launch_scale(const float* src, float* dst, const float* vec, long rows, long n, int divide, hipStream_t s);
void fortis_launch_mask_relu(const float* src, float* dst, long rows, long n, long tail, hipStream_t s);
void fortis_launch_zero(float* dst, long n, hipStream_t s);
void fortis_launch_boundary_pre(const void* A, float* X, long NI, long NK, const void* mean, const void* vmax,
                                const void* vmin, int host_esz, hipStream_t s);
void fortis_launch_boundary_post(const float* Y, void* B, long NI, long NK, const void* scale, int host_esz, hipStream_t s);
void fortis_launch_permute(const float* src, float* dst, long C, long S, int to_channels_first, hipStream_t s);

// ---- convolution family (conv.hip) ---------------------------------------------------------
// Workgroups are dealt to the chip's eight XCDs round-robin (workgroup b of a row of the grid runs on XCD
// (b + constant) % 8), each XCD with its own L2.  Kernels whose neighbouring workgroups read overlapping input
// (stencil rows, conv halos and z-planes) number their work through this map, which gives each XCD a contiguous
// band of the nb items instead of every eighth one (the last nb % 8 items keep their index).
#ifdef __HIPCC__
__device__ __forceinline__ unsigned fortis_xcd_band(unsigned b, unsigned nb)
{
    const unsigned per = nb / 8;
    return b < per * 8 ? (b % 8) * per + b / 8 : b;
}
#endif

struct ConvEpi {
    const float* scale;  // per output channel multiplier (folded BatchNorm), or null
    const float* shift;  // per output channel additive term (bias, folded BatchNorm), or null
    int act;
    float alpha;
    const float* res;    // residual tensor added after the activation (same shape as output), or null
    float* pool;         // conv2d only: also receives the 2 x 2 stride-2 max pool of the output (H, W even), or null
    // conv2d only: a following 1 x 1 convolution to head_n <= 4 channels (weights [head_n][F], bias or null) written to
    // head_y INSTEAD of this conv's own output, which then is not stored (fortis_conv_mfma_head_ok says when)
    const float* head_w;
    const float* head_b;
    float* head_y;
    int head_n;
};
bool fortis_conv_mfma_head_ok(long C, long H, long Wd, long F, int KD, int KS, int nh);
int fortis_launch_conv2d(const float* x, const float* w, float* y, long C, long H, long Wd, long F, long KH,
                         long KW, long Ho, long Wo, long sh, long sw, long ph, long pw, const ConvEpi& e,
                         long coff, long ctot, hipStream_t s);
int fortis_launch_convt2d(const float* x, const float* w, float* y, long C, long H, long Wd, long F, long KH,
                          long KW, long Ho, long Wo, long stride, long pad, const ConvEpi& e, long coff,
                          long ctot, hipStream_t s);
int fortis_launch_conv3d(const float* x, const float* w, float* y, long C, long D, long H, long Wd, long F,
                         long KD, long KH, long KW, long Do, long Ho, long Wo, long pd, long ph, long pw,
                         const ConvEpi& e, hipStream_t s, long sd = 1, long sh = 1, long sw = 1);
// MFMA implicit-GEMM path (conv_mfma.hip).  kind 0: KD x KS x KS conv, pad KS/2, stride 1; kind 1: 2x2
// stride-2 transposed conv.  wp: weights packed by fortis_conv_mfma_pack.  -1: shape not taken.
// kg: fortis_conv_mfma_kgroups of the shape the weights will be used on (channel groups inside a workgroup).
int fortis_conv_mfma_kgroups(long C, long D, long H, long Wd, long Fg, int KD, int KS, bool pooled = false);   // pooled: a 2 x 2 max pool of the output is asked for with the launch
float* fortis_conv_mfma_pack(const float* W, long F, long C, int T, int transposed, long* nfloats, int kg = 1);
const float* fortis_conv_mfma_pack_dev(const float* dW, long F, long C, int T, hipStream_t s, int kg = 1);   // device weights, packed into a library buffer; null: no memory
int fortis_launch_conv_mfma(const float* x, const float* wp, float* y, long C, long D, long H, long Wd, long F, int KD,
                            int KS, int kind, const ConvEpi& e, hipStream_t s);
// Partial sums of a conv whose input channels are split over workgroups: the library's one buffer for them
// (grown on demand, null when the device has no memory left) and the kernel that adds ksplit slices of
// osize floats and applies the epilogue.
float* fortis_conv_split_scratch(size_t bytes);
void fortis_conv_forget_buffers();
// While a workspace is set (base non-null) the packed weights of fortis_conv_mfma_pack_dev and the partial sums come
// out of it and nothing in the convolution path allocates; fortis_conv_workspace_overflowed() is the size a
// refused request would have needed (0: every request fitted).
void fortis_conv_workspace(void* base, size_t bytes);
size_t fortis_conv_workspace_overflowed();
int fortis_launch_conv_split_reduce(const float* part, float* y, long osize, long ospatial, int ksplit, const ConvEpi& e,
                                    hipStream_t s);
void fortis_launch_maxpool2d(const float* x, float* y, long C, long H, long Wd, long k, hipStream_t s);
void fortis_launch_upsample(const float* x, float* y, long C, long D, long H, long Wd, long sfac, int nd, hipStream_t s);
void fortis_launch_concat_copy(const float* x, float* y, long C, long S, long coff, hipStream_t s);
