// Model plan (what the MLIR-generated `mlp_kernel` host function is in the reference), the step
// binding, and the host-facing entry points of the generated shim (driver/fortis_shim.py:54-135):
// buffer ownership, upload/download choreography, pack/unpack staging, graph capture on the
// second call and replay afterwards, with an eager fallback.
#include <atomic>
#include <condition_variable>
#include <mutex>
#include <functional>
#include <thread>
#include <vector>
#include "common.h"

enum OpKind { OP_LINEAR, OP_SCALE, OP_MASK_RELU, OP_PRE, OP_POST, OP_CONV2D, OP_CONVT2D, OP_MAXPOOL, OP_UPSAMPLE,
              OP_CONCAT, OP_CONV3D, OP_PERMUTE };

struct Op {
    OpKind kind;
    int src = -1, dst = -1, res = -1;
    long B = 0, K = 0, N = 0;                 // linear; rows/n for scale & mask
    int act = 0; float alpha = 0.f;
    int flag = 0;                             // scale: divide; permute: to_channels_first; boundary: host_esz
    long tail = 0;
    long C = 0, D = 1, H = 0, W = 0, F = 0, KD = 1, KH = 1, KW = 1, stride = 1, pad = 0, opad = 0, coff = 0, ctot = 0, sfac = 1;
    int nd = 2;
    std::vector<float> w, b, v0, v1, v2, v3;  // host copies: weights, bias, vectors (bn / boundary)
    std::vector<double> d0, d1, d2;           // f64 boundary vectors
    float eps = 1e-5f;
    bool has_bias = false, has_bn = false, has_v[3] = { false, false, false };
};

enum ExecKind { EX_CHAIN, EX_GEMM, EX_SCALE, EX_MASK, EX_PRE, EX_POST, EX_CONV2D, EX_CONVT2D, EX_MAXPOOL, EX_UPSAMPLE,
                EX_CONCAT, EX_CONV3D, EX_PERMUTE };
struct Exec {
    ExecKind kind;
    int src = -1, dst = -1, res = -1;
    long rows = 0, rows_cap = 0;
    ChainDesc chain;
    // gemm
    const float *W = nullptr, *bias = nullptr, *out_scale = nullptr, *vec = nullptr;
    long K = 0, N = 0, mask_tail = 0;
    int act = 0; float alpha = 0.f;
    int flag = 0;
    const void *p0 = nullptr, *p1 = nullptr, *p2 = nullptr;
    const Op* op = nullptr;
    ConvEpi epi = { nullptr, nullptr, 0, 0.f, nullptr };
    const float* Wmfma = nullptr;   // weights packed for the MFMA implicit-GEMM kernel, when the shape qualifies
    int pool_dst = -1;              // conv2d: tensor that receives the 2 x 2 max pool folded into this conv
    int head_dst = -1;              // conv2d: tensor that receives the thin 1 x 1 convolution folded into this conv (which then stores nothing itself)
    const float *head_w = nullptr, *head_b = nullptr;
    int head_n = 0;
};

struct fortis_plan {
    std::vector<long> tbytes;
    std::vector<int> view_of;   // -1: owns a buffer; otherwise the tensor this one is a window of
    std::vector<long> view_off; // byte offset of the window
    std::vector<void*> tptr;
    std::vector<Op> ops;
    std::vector<Exec> exec;
    std::vector<void*> owned;   // device allocations owned by the plan (weights, vectors)
    std::vector<void*> bufs;    // distinct pool buffers behind the tensors (several tensors may share one)
    bool finalized = false;
    bool upload_failed = false; // a weight / vector upload found no device memory
    int in_t = -1, out_t = -1;
    long rows0 = 0;             // rows at finalize (row-wise plans), for run-time extents
    long band_rows = 0;         // rows when every kernel works row by row, boundary transposes included (row bands can then run on their own)
    int exec_skip = 0;          // ops folded into a neighbour at finalize
    bool prof = false;          // per-kernel event timing (fortis_plan_profile)
    std::vector<hipEvent_t> ev; // events of the recorded passes: (nexec + 1) per pass
    size_t ev_used = 0;
};

// Host data -> a device allocation owned by the plan.  On failure (no memory, copy refused) returns null and
// marks the plan: fortis_plan_finalize then fails, and a plan that is not finalized never launches.
static void* upload(fortis_plan* p, const void* h, size_t nbytes)
{
    void* d = nullptr;
    if (fortis_dev_malloc(&d, nbytes, "plan weights") != 0) { p->upload_failed = true; return nullptr; }
    p->owned.push_back(d);
    if (nbytes && hipMemcpy(d, h, nbytes, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        fprintf(stderr, "fortis_plan: copying %zu bytes of weights to the device failed\n", nbytes);
        p->upload_failed = true;
        return nullptr;
    }
    return d;
}

static int bad(const char* what) { fprintf(stderr, "fortis_plan: %s\n", what); return -1; }
static bool tensor_ok(fortis_plan* p, int t, long need_bytes)
{
    return t >= 0 && t < (int)p->tbytes.size() && p->tbytes[t] >= need_bytes;
}

extern "C" {

fortis_plan* fortis_plan_create(void) { return new fortis_plan(); }
void fortis_plan_destroy(fortis_plan* p)
{
    if (!p) return;
    for (void* d : p->owned) fortis_dev_free(d);
    for (void* b : p->bufs) fortis_free(b);
    delete p;
}
int fortis_plan_tensor(fortis_plan* p, long nbytes)
{
    if (!p || p->finalized || nbytes <= 0) return -1;
    p->tbytes.push_back(nbytes);
    p->view_of.push_back(-1);
    p->view_off.push_back(0);
    return (int)p->tbytes.size() - 1;
}
int fortis_plan_view(fortis_plan* p, int base, long byte_offset, long nbytes)
{
    if (!p || p->finalized || base < 0 || base >= (int)p->tbytes.size() || byte_offset < 0 || nbytes <= 0 ||
        byte_offset % 16 || byte_offset + nbytes > p->tbytes[base]) {
        fprintf(stderr, "fortis_plan_view: window outside tensor %d or not 16-byte aligned\n", base);
        return -1;
    }
    p->tbytes.push_back(nbytes);
    p->view_of.push_back(p->view_of[base] >= 0 ? p->view_of[base] : base);
    p->view_off.push_back(p->view_off[base] + byte_offset);
    return (int)p->tbytes.size() - 1;
}

int fortis_plan_linear(fortis_plan* p, int src, int dst, const float* W, const float* bias, long B, long K, long N,
                       int act, float alpha)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (B <= 0 || K <= 0 || N <= 0 || !W || act < 0 || act > 2) return bad("linear: bad shape or arguments");
    if (!tensor_ok(p, src, B * K * 4) || !tensor_ok(p, dst, B * N * 4) || src == dst) return bad("linear: tensors too small or aliased");
    Op o; o.kind = OP_LINEAR; o.src = src; o.dst = dst; o.B = B; o.K = K; o.N = N; o.act = act; o.alpha = alpha;
    o.w.assign(W, W + N * K);
    if (bias) { o.b.assign(bias, bias + N); o.has_bias = true; }
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_scale(fortis_plan* p, int src, int dst, const float* vec, long rows, long n, int divide)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (rows <= 0 || n <= 0 || !vec) return bad("scale: bad shape");
    if (!tensor_ok(p, src, rows * n * 4) || !tensor_ok(p, dst, rows * n * 4)) return bad("scale: tensors too small");
    Op o; o.kind = OP_SCALE; o.src = src; o.dst = dst; o.B = rows; o.N = n; o.K = n; o.flag = divide ? 1 : 0;
    o.v0.assign(vec, vec + n);
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_mask_relu(fortis_plan* p, int src, int dst, long rows, long n, long tail)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (rows <= 0 || n <= 0 || tail < 0 || tail > n) return bad("mask_relu: bad shape");
    if (!tensor_ok(p, src, rows * n * 4) || !tensor_ok(p, dst, rows * n * 4)) return bad("mask_relu: tensors too small");
    Op o; o.kind = OP_MASK_RELU; o.src = src; o.dst = dst; o.B = rows; o.N = n; o.K = n; o.tail = tail;
    p->ops.push_back(std::move(o));
    return 0;
}
static void take_vec(Op& o, int which, const void* v, long n, int esz)
{
    if (!v) return;
    o.has_v[which] = true;
    if (esz == 8) { std::vector<double>& d = which == 0 ? o.d0 : which == 1 ? o.d1 : o.d2; d.assign((const double*)v, (const double*)v + n); }
    else { std::vector<float>& f = which == 0 ? o.v0 : which == 1 ? o.v1 : o.v2; f.assign((const float*)v, (const float*)v + n); }
}
int fortis_plan_boundary_pre(fortis_plan* p, int src, int dst, long NI, long NK, const void* mean, const void* vmax,
                             const void* vmin, int host_esz)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (NI <= 0 || NK <= 0 || (host_esz != 4 && host_esz != 8)) return bad("boundary_pre: bad shape or element size");
    if (!tensor_ok(p, src, NI * NK * host_esz) || !tensor_ok(p, dst, NI * NK * 4) || src == dst) return bad("boundary_pre: tensors too small or aliased");
    Op o; o.kind = OP_PRE; o.src = src; o.dst = dst; o.B = NI; o.N = NK; o.flag = host_esz;
    take_vec(o, 0, mean, NK, host_esz); take_vec(o, 1, vmax, NK, host_esz); take_vec(o, 2, vmin, NK, host_esz);
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_boundary_post(fortis_plan* p, int src, int dst, long NI, long NK, const void* scale, int host_esz)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (NI <= 0 || NK <= 0 || (host_esz != 4 && host_esz != 8)) return bad("boundary_post: bad shape or element size");
    if (!tensor_ok(p, src, NI * NK * 4) || !tensor_ok(p, dst, NI * NK * host_esz) || src == dst) return bad("boundary_post: tensors too small or aliased");
    Op o; o.kind = OP_POST; o.src = src; o.dst = dst; o.B = NI; o.N = NK; o.flag = host_esz;
    take_vec(o, 0, scale, NK, host_esz);
    p->ops.push_back(std::move(o));
    return 0;
}

int fortis_plan_conv2d(fortis_plan* p, int src, int dst, const float* W, const float* bias, const float* bn_gamma,
                       const float* bn_beta, const float* bn_mean, const float* bn_var, float bn_eps, long C, long H,
                       long Wd, long F, long KH, long KW, long stride, long pad, int act, float alpha, long coff, long ctot)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (C <= 0 || H <= 0 || Wd <= 0 || F <= 0 || KH <= 0 || KW <= 0 || stride <= 0 || pad < 0 || !W) return bad("conv2d: bad shape");
    const long Ho = (H + 2 * pad - KH) / stride + 1, Wo = (Wd + 2 * pad - KW) / stride + 1;
    if (ctot <= 0) { ctot = F; coff = 0; }
    if (Ho <= 0 || Wo <= 0 || coff < 0 || coff + F > ctot) return bad("conv2d: bad output shape or channel offset");
    if (!tensor_ok(p, src, C * H * Wd * 4) || !tensor_ok(p, dst, ctot * Ho * Wo * 4) || src == dst) return bad("conv2d: tensors too small or aliased");
    const int nbn = (bn_gamma != 0) + (bn_beta != 0) + (bn_mean != 0) + (bn_var != 0);
    if (nbn != 0 && nbn != 4) return bad("conv2d: give all four BatchNorm vectors or none");
    Op o; o.kind = OP_CONV2D; o.src = src; o.dst = dst; o.C = C; o.H = H; o.W = Wd; o.F = F; o.KH = KH; o.KW = KW;
    o.stride = stride; o.pad = pad; o.act = act; o.alpha = alpha; o.coff = coff; o.ctot = ctot; o.eps = bn_eps;
    o.w.assign(W, W + F * C * KH * KW);
    if (bias) { o.b.assign(bias, bias + F); o.has_bias = true; }
    if (nbn) { o.has_bn = true; o.v0.assign(bn_gamma, bn_gamma + F); o.v1.assign(bn_beta, bn_beta + F); o.v2.assign(bn_mean, bn_mean + F); o.v3.assign(bn_var, bn_var + F); }
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_convt2d(fortis_plan* p, int src, int dst, const float* W, const float* bias, long C, long H, long Wd,
                        long F, long KH, long KW, long stride, long pad, long output_padding, int act, float alpha,
                        long coff, long ctot)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (C <= 0 || H <= 0 || Wd <= 0 || F <= 0 || KH <= 0 || KW <= 0 || stride <= 0 || pad < 0 || !W) return bad("convt2d: bad shape");
    const long Ho = (H - 1) * stride - 2 * pad + KH + output_padding, Wo = (Wd - 1) * stride - 2 * pad + KW + output_padding;
    if (ctot <= 0) { ctot = F; coff = 0; }
    if (Ho <= 0 || Wo <= 0 || coff < 0 || coff + F > ctot) return bad("convt2d: bad output shape or channel offset");
    if (!tensor_ok(p, src, C * H * Wd * 4) || !tensor_ok(p, dst, ctot * Ho * Wo * 4) || src == dst) return bad("convt2d: tensors too small or aliased");
    Op o; o.kind = OP_CONVT2D; o.src = src; o.dst = dst; o.C = C; o.H = H; o.W = Wd; o.F = F; o.KH = KH; o.KW = KW;
    o.stride = stride; o.pad = pad; o.opad = output_padding; o.act = act; o.alpha = alpha; o.coff = coff; o.ctot = ctot;
    o.w.assign(W, W + C * F * KH * KW);
    if (bias) { o.b.assign(bias, bias + F); o.has_bias = true; }
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_maxpool2d(fortis_plan* p, int src, int dst, long C, long H, long Wd, long k)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (C <= 0 || H <= 0 || Wd <= 0 || k <= 0 || H % k || Wd % k) return bad("maxpool2d: bad shape");
    if (!tensor_ok(p, src, C * H * Wd * 4) || !tensor_ok(p, dst, C * (H / k) * (Wd / k) * 4) || src == dst) return bad("maxpool2d: tensors too small or aliased");
    Op o; o.kind = OP_MAXPOOL; o.src = src; o.dst = dst; o.C = C; o.H = H; o.W = Wd; o.KH = k;
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_upsample(fortis_plan* p, int src, int dst, long C, long D, long H, long Wd, long s, int nd)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (C <= 0 || D <= 0 || H <= 0 || Wd <= 0 || s <= 0 || (nd != 2 && nd != 3)) return bad("upsample: bad shape");
    const long out = C * (nd == 3 ? D * s : D) * H * s * Wd * s;
    if (!tensor_ok(p, src, C * D * H * Wd * 4) || !tensor_ok(p, dst, out * 4) || src == dst) return bad("upsample: tensors too small or aliased");
    Op o; o.kind = OP_UPSAMPLE; o.src = src; o.dst = dst; o.C = C; o.D = D; o.H = H; o.W = Wd; o.sfac = s; o.nd = nd;
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_concat_copy(fortis_plan* p, int src, int dst, long C, long S, long coff, long ctot)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (C <= 0 || S <= 0 || coff < 0 || coff + C > ctot) return bad("concat_copy: bad shape");
    if (!tensor_ok(p, src, C * S * 4) || !tensor_ok(p, dst, ctot * S * 4) || src == dst) return bad("concat_copy: tensors too small or aliased");
    Op o; o.kind = OP_CONCAT; o.src = src; o.dst = dst; o.C = C; o.H = S; o.coff = coff; o.ctot = ctot;
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_conv3d(fortis_plan* p, int src, int dst, int res, const float* W, const float* bias, long C, long D,
                       long H, long Wd, long F, long K, long pad, int act, float alpha)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (C <= 0 || D <= 0 || H <= 0 || Wd <= 0 || F <= 0 || K <= 0 || pad < 0 || !W) return bad("conv3d: bad shape");
    const long Do = D + 2 * pad - K + 1, Ho = H + 2 * pad - K + 1, Wo = Wd + 2 * pad - K + 1;
    if (Do <= 0 || Ho <= 0 || Wo <= 0) return bad("conv3d: empty output");
    if (!tensor_ok(p, src, C * D * H * Wd * 4) || !tensor_ok(p, dst, F * Do * Ho * Wo * 4) || src == dst) return bad("conv3d: tensors too small or aliased");
    if (res >= 0 && (!tensor_ok(p, res, F * Do * Ho * Wo * 4) || res == dst)) return bad("conv3d: residual tensor too small or aliased");
    Op o; o.kind = OP_CONV3D; o.src = src; o.dst = dst; o.res = res; o.C = C; o.D = D; o.H = H; o.W = Wd; o.F = F;
    o.KD = o.KH = o.KW = K; o.pad = pad; o.act = act; o.alpha = alpha;
    o.w.assign(W, W + F * C * K * K * K);
    if (bias) { o.b.assign(bias, bias + F); o.has_bias = true; }
    p->ops.push_back(std::move(o));
    return 0;
}
int fortis_plan_permute(fortis_plan* p, int src, int dst, long C, long S, int to_channels_first)
{
    if (!p || p->finalized) return bad("plan is null or already finalized");
    if (C <= 0 || S <= 0) return bad("permute: bad shape");
    if (!tensor_ok(p, src, C * S * 4) || !tensor_ok(p, dst, C * S * 4) || src == dst) return bad("permute: tensors too small or aliased");
    Op o; o.kind = OP_PERMUTE; o.src = src; o.dst = dst; o.C = C; o.H = S; o.flag = to_channels_first ? 1 : 0;
    p->ops.push_back(std::move(o));
    return 0;
}

}  // extern "C"

// ---- finalize: fusion + uploads -----------------------------------------------------------------
static int uses_of(const fortis_plan* p, int t)
{
    int n = (t == p->out_t) ? 1 : 0;
    for (const Op& o : p->ops) n += (o.src == t) + (o.res == t);
    return n;
}

// Tries to turn ops[i..] into one LDS-resident chain.  Returns the number of ops consumed (0 if none).
static size_t try_chain(fortis_plan* p, size_t i, Exec* ex)
{
    const std::vector<Op>& ops = p->ops;
    size_t j = i;
    const Op* in_div = nullptr;
    if (ops[j].kind == OP_SCALE && ops[j].flag == 1 && j + 1 < ops.size() && ops[j + 1].kind == OP_LINEAR &&
        ops[j + 1].src == ops[j].dst && uses_of(p, ops[j].dst) == 1 && ops[j].B == ops[j + 1].B && ops[j].N == ops[j + 1].K) {
        in_div = &ops[j];
        j++;
    }
    if (ops[j].kind != OP_LINEAR) return 0;
    std::vector<const Op*> lin;
    const long rows = ops[j].B;
    while (j < ops.size() && ops[j].kind == OP_LINEAR && ops[j].B == rows && ops[j].K <= FORTIS_CHAIN_MAX_WIDTH &&
           ops[j].N <= FORTIS_CHAIN_MAX_WIDTH && (int)lin.size() < FORTIS_CHAIN_MAX_LAYERS &&
           (lin.empty() || (ops[j].src == lin.back()->dst && uses_of(p, lin.back()->dst) == 1))) {
        lin.push_back(&ops[j]);
        j++;
    }
    if (lin.empty()) return 0;
    if (in_div && lin[0]->src != in_div->dst) return 0;
    const Op* out_mul = nullptr;
    const Op* mask = nullptr;
    int last_dst = lin.back()->dst;
    if (j < ops.size() && ops[j].kind == OP_SCALE && ops[j].flag == 0 && ops[j].src == last_dst && uses_of(p, last_dst) == 1 &&
        ops[j].B == rows && ops[j].N == lin.back()->N) { out_mul = &ops[j]; last_dst = ops[j].dst; j++; }
    if (!out_mul && j < ops.size() && ops[j].kind == OP_MASK_RELU && ops[j].src == last_dst && uses_of(p, last_dst) == 1 &&
        ops[j].B == rows && ops[j].N == lin.back()->N) { mask = &ops[j]; last_dst = ops[j].dst; j++; }
    memset(&ex->chain, 0, sizeof ex->chain);
    ex->kind = EX_CHAIN;
    ex->src = in_div ? in_div->src : lin[0]->src;
    ex->dst = last_dst;
    ex->rows = ex->rows_cap = rows;
    ChainDesc& d = ex->chain;
    {
        const float* Wh[FORTIS_CHAIN_MAX_LAYERS];
        const float* bh[FORTIS_CHAIN_MAX_LAYERS];
        int Ks[FORTIS_CHAIN_MAX_LAYERS], Ns[FORTIS_CHAIN_MAX_LAYERS];
        for (size_t l = 0; l < lin.size(); l++) {
            Wh[l] = lin[l]->w.data();
            bh[l] = lin[l]->has_bias ? lin[l]->b.data() : nullptr;
            Ks[l] = (int)lin[l]->K; Ns[l] = (int)lin[l]->N;
        }
        float* blob = nullptr;
        if (fortis_chain_build(&d, (int)lin.size(), Wh, bh, Ks, Ns, &blob) != 0) return 0;
        p->owned.push_back(blob);
        for (size_t l = 0; l < lin.size(); l++) { d.L[l].act = lin[l]->act; d.L[l].alpha = lin[l]->alpha; }
    }
    if (in_div) d.in_div = (const float*)upload(p, in_div->v0.data(), in_div->v0.size() * 4);
    if (in_div && d.in_div) {
        // divisors all in [2^-40, 2^40]: their refined reciprocals go beside them, for the kernels' short division
        bool ok = true;
        for (float v : in_div->v0) { const float m = fabsf(v); ok = ok && m >= 0x1p-40f && m <= 0x1p40f; }
        if (ok) {
            std::vector<float> z(in_div->v0.size(), 0.f);
            float* r = (float*)upload(p, z.data(), z.size() * 4);
            if (r) { fortis_chain_fill_rcp(d.in_div, r, (int)z.size(), fortis_stream_get()); d.in_rcp = r; }
        }
    }
    if (out_mul) d.out_mul = (const float*)upload(p, out_mul->v0.data(), out_mul->v0.size() * 4);
    d.mask_tail = mask ? (int)mask->tail : 0;
    return j - i;
}

// Gives every tensor its device buffer by walking the kernels in launch order the way the reference's generated
// host code does at run time (compiler/FortisFuse.cpp:512-516: a temporary is taken from the pool in front of
// the group that first writes it and handed back behind the group that last reads it), so that temporaries
// whose lifetimes do not overlap share a pool buffer and a deep stack holds two or three activations instead of
// all of them.  The walk happens once, here: the pointers are then fixed for the life of the plan (a captured
// graph names them) and every buffer the walk touched stays marked in use in the pool until the plan is
// destroyed.  The model's input and output, and tensors no kernel writes (filled by the caller), keep their
// buffer throughout; a tensor no kernel touches (folded into a neighbour at fusion) gets none.
static int assign_buffers(fortis_plan* p)
{
    const int nt = (int)p->tbytes.size(), ne = (int)p->exec.size();
    const int never = ne + 1;
    std::vector<int> first(nt, never), last(nt, -2);
    auto base = [&](int t) { return p->view_of[t] >= 0 ? p->view_of[t] : t; };
    auto reads = [&](int t, int i) { if (t < 0) return; t = base(t); if (first[t] == never) first[t] = -1; if (last[t] < i) last[t] = i; };
    auto writes = [&](int t, int i) { if (t < 0) return; t = base(t); if (first[t] > i) first[t] = i; if (last[t] < i) last[t] = i; };
    for (int i = 0; i < ne; i++) {
        const Exec& e = p->exec[i];
        reads(e.src, i); reads(e.res, i);
        if (e.head_dst < 0) writes(e.dst, i);
        writes(e.pool_dst, i); writes(e.head_dst, i);
    }
    for (int t = 0; t < nt; t++) if (first[t] == -1) last[t] = ne;          // filled by the caller: never handed back
    first[base(p->in_t)] = -1; last[base(p->in_t)] = ne;
    if (first[base(p->out_t)] == never) first[base(p->out_t)] = -1;
    last[base(p->out_t)] = ne;
    for (void* b : p->bufs) fortis_free(b);
    p->bufs.clear();
    p->tptr.assign(nt, nullptr);
    // The sharing is done on a list of the plan's own: a buffer the walk has handed back stays marked in use in the
    // pool, so the pool's release-everything-unused-and-retry (when a later raw allocation fails) can never free a
    // buffer an earlier tensor of this walk already points to.  Best fit among the walk's released buffers, like
    // the pool's own choice; a tensor that finds none takes a new buffer from the pool.
    std::vector<long> bsize;
    std::vector<char> bfree;
    int rc = 0;
    auto take = [&](int t) {
        const long n = p->tbytes[t];
        int best = -1;
        for (size_t b = 0; b < p->bufs.size(); b++)
            if (bfree[b] && bsize[b] >= n && (best < 0 || bsize[b] < bsize[best])) best = (int)b;
        // a buffer the pool holds unused (left by a plan destroyed earlier) that fits more tightly is taken instead,
        // as the pool's own best fit over all released buffers would
        const long pool_fit = fortis_pool_best_fit(n);
        if (best >= 0 && pool_fit >= 0 && pool_fit < bsize[best]) best = -1;
        if (best < 0) {
            void* d = fortis_alloc(n);
            if (!d) { rc = -1; return; }
            p->bufs.push_back(d); bsize.push_back(pool_fit >= 0 ? pool_fit : n); bfree.push_back(0);   // a released pool buffer keeps its own size
            best = (int)p->bufs.size() - 1;
        }
        bfree[best] = 0;
        p->tptr[t] = p->bufs[best];
    };
    auto give = [&](void* d) { for (size_t b = 0; b < p->bufs.size(); b++) if (p->bufs[b] == d) bfree[b] = 1; };
    for (int t = 0; t < nt && rc == 0; t++) if (p->view_of[t] < 0 && first[t] == -1) take(t);
    for (int i = 0; i < ne && rc == 0; i++) {
        for (int t = 0; t < nt && rc == 0; t++) if (p->view_of[t] < 0 && first[t] == i) take(t);
        for (int t = 0; t < nt; t++) if (p->view_of[t] < 0 && last[t] == i && p->tptr[t]) give(p->tptr[t]);
    }
    if (rc != 0) { p->tptr.assign(nt, nullptr); return -1; }
    for (int t = 0; t < nt; t++)
        if (p->view_of[t] >= 0 && p->tptr[p->view_of[t]]) p->tptr[t] = (char*)p->tptr[p->view_of[t]] + p->view_off[t];
    return 0;
}

extern "C" {

int fortis_plan_finalize(fortis_plan* p, int in_t, int out_t)
{
    if (!p || p->finalized) return bad("finalize: plan is null or already finalized");
    if (in_t < 0 || in_t >= (int)p->tbytes.size() || out_t < 0 || out_t >= (int)p->tbytes.size()) return bad("finalize: bad input/output tensor");
    if (p->ops.empty()) return bad("finalize: empty plan");
    p->in_t = in_t; p->out_t = out_t;
    const std::vector<Op>& ops = p->ops;
    int fuse_ups_src = -1;      // source tensor of an upsample folded into the convolution that follows
    for (size_t i = 0; i < ops.size();) {
        Exec ex;
        size_t took = try_chain(p, i, &ex);
        if (took) { p->exec.push_back(ex); i += took; continue; }
        const Op& o = ops[i];
        ex.src = o.src; ex.dst = o.dst; ex.res = o.res; ex.op = &ops[i];
        size_t adv = 1;
        switch (o.kind) {
            case OP_LINEAR: {
                ex.kind = EX_GEMM; ex.rows = ex.rows_cap = o.B; ex.K = o.K; ex.N = o.N; ex.act = o.act; ex.alpha = o.alpha;
                ex.W = (const float*)upload(p, o.w.data(), o.w.size() * 4);
                ex.bias = o.has_bias ? (const float*)upload(p, o.b.data(), o.b.size() * 4) : nullptr;
                // fold a directly following output scale or masked-ReLU head into the epilogue
                if (i + 1 < ops.size() && ops[i + 1].src == o.dst && uses_of(p, o.dst) == 1 && ops[i + 1].B == o.B && ops[i + 1].N == o.N) {
                    if (ops[i + 1].kind == OP_SCALE && ops[i + 1].flag == 0) {
                        ex.out_scale = (const float*)upload(p, ops[i + 1].v0.data(), ops[i + 1].v0.size() * 4);
                        ex.dst = ops[i + 1].dst; adv = 2;
                    } else if (ops[i + 1].kind == OP_MASK_RELU) {
                        ex.mask_tail = ops[i + 1].tail; ex.dst = ops[i + 1].dst; adv = 2;
                    }
                }
                break;
            }
            case OP_SCALE:
                ex.kind = EX_SCALE; ex.rows = ex.rows_cap = o.B; ex.N = o.N; ex.flag = o.flag;
                ex.vec = (const float*)upload(p, o.v0.data(), o.v0.size() * 4);
                break;
            case OP_MASK_RELU:
                ex.kind = EX_MASK; ex.rows = ex.rows_cap = o.B; ex.N = o.N; ex.mask_tail = o.tail;
                break;
            case OP_PRE:
            case OP_POST: {
                ex.kind = o.kind == OP_PRE ? EX_PRE : EX_POST; ex.rows = ex.rows_cap = o.B; ex.N = o.N; ex.flag = o.flag;
                const void* hv[3]; size_t nb = (size_t)o.N * o.flag;
                hv[0] = o.flag == 8 ? (const void*)o.d0.data() : (const void*)o.v0.data();
                hv[1] = o.flag == 8 ? (const void*)o.d1.data() : (const void*)o.v1.data();
                hv[2] = o.flag == 8 ? (const void*)o.d2.data() : (const void*)o.v2.data();
                ex.p0 = o.has_v[0] ? upload(p, hv[0], nb) : nullptr;
                ex.p1 = o.has_v[1] ? upload(p, hv[1], nb) : nullptr;
                ex.p2 = o.has_v[2] ? upload(p, hv[2], nb) : nullptr;
                break;
            }
            case OP_CONV2D:
            case OP_CONVT2D:
            case OP_CONV3D: {
                ex.kind = o.kind == OP_CONV2D ? EX_CONV2D : o.kind == OP_CONVT2D ? EX_CONVT2D : EX_CONV3D;
                if (o.kind == OP_CONV3D && fuse_ups_src >= 0) { ex.src = fuse_ups_src; ex.flag = 1; }
                fuse_ups_src = -1;
                ex.W = (const float*)upload(p, o.w.data(), o.w.size() * 4);
                // y = act(scale * conv + shift): bias and BatchNorm-eval folded into two vectors.
                // scale = gamma / sqrt(var + eps); shift = beta + (bias - mean) * scale.
                std::vector<float> scale, shift;
                if (o.has_bn) {
                    scale.resize(o.F); shift.resize(o.F);
                    for (long f = 0; f < o.F; f++) {
                        const double sc = (double)o.v0[f] / sqrt((double)o.v3[f] + (double)o.eps);
                        scale[f] = (float)sc;
                        shift[f] = (float)((double)o.v1[f] + ((o.has_bias ? (double)o.b[f] : 0.0) - (double)o.v2[f]) * sc);
                    }
                } else if (o.has_bias) shift = o.b;
                ex.epi.scale = scale.empty() ? nullptr : (const float*)upload(p, scale.data(), scale.size() * 4);
                ex.epi.shift = shift.empty() ? nullptr : (const float*)upload(p, shift.data(), shift.size() * 4);
                ex.epi.act = o.act; ex.epi.alpha = o.alpha;
                // matrix-core path for the shapes it takes; narrow outputs stay on the direct kernel
                static int direct_only = -1;
                if (direct_only < 0) direct_only = getenv("FORTIS_CONV_DIRECT") != 0;
                // enough output channels to fill a 32-channel MFMA group; a 1 x 1 conv always (it is a plain GEMM over
                // the pixels whose cost is reading the input once, which the staged kernel does and the direct one does not)
                const bool wide = o.F >= 16 || (o.kind == OP_CONV2D && o.KH == 1 && o.KW == 1);
                bool ok = false;
                int T = 0, tr = 0;
                if (o.kind == OP_CONV2D) { ok = o.stride == 1 && o.KH == o.KW && (o.KH == 1 || o.KH == 3) && o.pad == o.KH / 2; T = (int)(o.KH * o.KW); }
                else if (o.kind == OP_CONV3D) { ok = o.KD == 3 && o.pad == 1; T = 27; }
                else { ok = o.KH == 2 && o.KW == 2 && o.stride == 2 && o.pad == 0 && o.opad == 0; T = 1; tr = 1; }
                // (a 2 x 2 max pool that will be folded into this conv, see below, is part of the choice of the kernel form)
                const bool will_pool = o.kind == OP_CONV2D && i + 1 < ops.size() && ops[i + 1].kind == OP_MAXPOOL && ops[i + 1].src == o.dst &&
                    ops[i + 1].KH == 2 && ops[i + 1].C == o.F && ops[i + 1].H == o.H && ops[i + 1].W == o.W && o.coff == 0 &&
                    (o.ctot == 0 || o.ctot == o.F) && !(o.H & 1) && !(o.W & 1) && ops[i + 1].dst != o.dst;
                if (ok && wide && !direct_only) {
                    const int kg = o.kind == OP_CONV3D ? 1 : fortis_conv_mfma_kgroups(o.C, 1, o.H, o.W, tr ? 4 * o.F : o.F, 1, tr ? 1 : (int)o.KH, will_pool);
                    float* wp = fortis_conv_mfma_pack(o.w.data(), o.F, o.C, T, tr, nullptr, kg);
                    if (!wp) p->upload_failed = true; else p->owned.push_back(wp);
                    ex.Wmfma = wp;
                }
                // A 2 x 2 max pool that directly follows and reads this conv's whole output is written by the conv's
                // own last stage (the reduce of a channel-split launch, else a pool launch from the conv launcher).
                if (ex.Wmfma && will_pool) {
                    ex.pool_dst = ops[i + 1].dst;
                    p->exec.push_back(ex);
                    p->exec_skip++;
                    i += adv + 1;
                    continue;
                }
                // A 1 x 1 convolution to at most four channels (no BatchNorm, no activation) that is the only reader of
                // this conv's output is computed by this conv's kernel from its finished tiles where the launcher has
                // that form; the intermediate tensor is then never stored.
                if (o.kind == OP_CONV2D && ex.Wmfma && i + 1 < ops.size() && o.coff == 0 && (o.ctot == 0 || o.ctot == o.F)) {
                    const Op& h = ops[i + 1];
                    if (h.kind == OP_CONV2D && h.src == o.dst && uses_of(p, o.dst) == 1 && h.KH == 1 && h.KW == 1 && h.stride == 1 && h.pad == 0 &&
                        h.C == o.F && h.H == o.H && h.W == o.W && h.F <= 4 && !h.has_bn && h.act == FORTIS_ACT_NONE && h.coff == 0 &&
                        (h.ctot == 0 || h.ctot == h.F) && h.dst != o.dst && o.dst != p->out_t && getenv("FORTIS_NO_HEAD_FOLD") == nullptr &&
                        fortis_conv_mfma_head_ok(o.C, o.H, o.W, o.F, 1, (int)o.KH, (int)h.F)) {
                        ex.head_dst = h.dst;
                        ex.head_n = (int)h.F;
                        ex.head_w = (const float*)upload(p, h.w.data(), h.w.size() * 4);
                        ex.head_b = h.has_bias ? (const float*)upload(p, h.b.data(), h.b.size() * 4) : nullptr;
                        p->exec.push_back(ex);
                        p->exec_skip++;
                        i += adv + 1;
                        continue;
                    }
                }
                break;
            }
            case OP_MAXPOOL: ex.kind = EX_MAXPOOL; break;
            case OP_UPSAMPLE: {
                ex.kind = EX_UPSAMPLE;
                // A 3-D nearest x2 upsample whose only reader is the next 3x3x3 convolution is not run:
                // the convolution reads the half-resolution tensor through the upsample's index map.
                static int direct_only = -1;
                if (direct_only < 0) direct_only = getenv("FORTIS_CONV_DIRECT") != 0;
                if (!direct_only && o.nd == 3 && o.sfac == 2 && i + 1 < ops.size() && ops[i + 1].kind == OP_CONV3D &&
                    ops[i + 1].src == o.dst && ops[i + 1].KD == 3 && ops[i + 1].pad == 1 && ops[i + 1].F >= 16 && out_t != o.dst) {
                    bool other = false;
                    for (size_t j = 0; j < ops.size(); j++)
                        if (j != i + 1 && (ops[j].src == o.dst || ops[j].res == o.dst)) other = true;
                    if (ops[i + 1].res == o.dst) other = true;
                    if (!other) { fuse_ups_src = o.src; p->exec_skip++; i += 1; continue; }
                }
                break;
            }
            case OP_CONCAT: ex.kind = EX_CONCAT; break;
            case OP_PERMUTE: ex.kind = EX_PERMUTE; break;
        }
        p->exec.push_back(ex);
        i += adv;
    }
    bool rowwise = true;
    long rows = -1;
    for (const Exec& e : p->exec) {
        if (e.kind > EX_MASK) { rowwise = false; break; }
        if (rows < 0) rows = e.rows; else if (rows != e.rows) rowwise = false;
    }
    p->rows0 = rowwise ? rows : 0;
    {
        bool bandable = true;
        long br = -1;
        for (const Exec& e : p->exec) {
            if (e.kind > EX_POST) { bandable = false; break; }
            if (br < 0) br = e.rows; else if (br != e.rows) bandable = false;
        }
        for (int v : p->view_of) if (v >= 0) bandable = false;
        p->band_rows = bandable ? br : 0;
    }
    if (p->upload_failed) return bad("finalize: out of device memory for the weights");
    if (assign_buffers(p) != 0) return bad("finalize: out of device memory for the activations");
    p->finalized = true;
    // (with a test's host allocator in place of the device's there is no device to wait for, and no launch may follow)
    if (fortis_pool_on_device()) { (void)fortis_stream_get(); HIP_OK(hipDeviceSynchronize()); }
    return 0;
}

void fortis_plan_run(fortis_plan* p)
{
    if (!p || !p->finalized) { fprintf(stderr, "fortis_plan_run: plan not finalized\n"); return; }
    hipStream_t s = fortis_stream_get();
    auto mark = [&]() {
        if (!p->prof || fortis_capturing) return;
        if (p->ev_used == p->ev.size()) { hipEvent_t e; HIP_OK(hipEventCreate(&e)); p->ev.push_back(e); }
        HIP_OK(hipEventRecord(p->ev[p->ev_used++], s));
    };
    mark();
    for (const Exec& e : p->exec) {
        const float* src = (const float*)p->tptr[e.src];
        float* dst = (float*)p->tptr[e.dst];
        const Op* o = e.op;
        int rc = 0;
        switch (e.kind) {
            case EX_CHAIN: fortis_launch_chain(e.chain, src, dst, e.rows, s); break;
            case EX_GEMM: rc = fortis_launch_gemm(src, e.W, e.bias, dst, e.rows, e.N, e.K, e.act, e.alpha, e.out_scale, e.mask_tail, s); break;
            case EX_SCALE: fortis_launch_scale(src, dst, e.vec, e.rows, e.N, e.flag, s); break;
            case EX_MASK: fortis_launch_mask_relu(src, dst, e.rows, e.N, e.mask_tail, s); break;
            case EX_PRE: fortis_launch_boundary_pre(p->tptr[e.src], dst, e.rows, e.N, e.p0, e.p1, e.p2, e.flag, s); break;
            case EX_POST: fortis_launch_boundary_post(src, p->tptr[e.dst], e.rows, e.N, e.p0, e.flag, s); break;
            case EX_CONV2D: {
                const long Ho = (o->H + 2 * o->pad - o->KH) / o->stride + 1, Wo = (o->W + 2 * o->pad - o->KW) / o->stride + 1;
                ConvEpi epi = e.epi;
                epi.pool = e.pool_dst >= 0 ? (float*)p->tptr[e.pool_dst] : nullptr;
                if (e.head_dst >= 0) { epi.head_w = e.head_w; epi.head_b = e.head_b; epi.head_n = e.head_n; epi.head_y = (float*)p->tptr[e.head_dst]; }
                rc = e.Wmfma ? fortis_launch_conv_mfma(src, e.Wmfma, dst + o->coff * Ho * Wo, o->C, 1, o->H, o->W, o->F, 1, (int)o->KH, 0, epi, s) : -1;
                if (rc != 0 && e.head_dst >= 0) { fprintf(stderr, "fortis_plan_run: conv2d with a folded 1 x 1 head not taken by the kernel\n"); break; }
                if (rc != 0) {
                    rc = fortis_launch_conv2d(src, e.W, dst, o->C, o->H, o->W, o->F, o->KH, o->KW, Ho, Wo, o->stride, o->stride,
                                              o->pad, o->pad, e.epi, o->coff, o->ctot, s);
                    if (rc == 0 && epi.pool) fortis_launch_maxpool2d(dst, epi.pool, o->F, Ho, Wo, 2, s);
                }
                break;
            }
            case EX_CONVT2D: {
                const long Ho = (o->H - 1) * o->stride - 2 * o->pad + o->KH + o->opad, Wo = (o->W - 1) * o->stride - 2 * o->pad + o->KW + o->opad;
                rc = e.Wmfma ? fortis_launch_conv_mfma(src, e.Wmfma, dst + o->coff * Ho * Wo, o->C, 1, o->H, o->W, o->F, 1, 1, 1, e.epi, s) : -1;
                if (rc != 0)
                    rc = fortis_launch_convt2d(src, e.W, dst, o->C, o->H, o->W, o->F, o->KH, o->KW, Ho, Wo, o->stride, o->pad, e.epi,
                                               o->coff, o->ctot, s);
                break;
            }
            case EX_CONV3D: {
                ConvEpi epi = e.epi;
                epi.res = e.res >= 0 ? (const float*)p->tptr[e.res] : nullptr;
                const long Do = o->D + 2 * o->pad - o->KD + 1, Ho = o->H + 2 * o->pad - o->KH + 1, Wo = o->W + 2 * o->pad - o->KW + 1;
                rc = e.Wmfma ? fortis_launch_conv_mfma(src, e.Wmfma, dst, o->C, o->D, o->H, o->W, o->F, 3, 3, e.flag ? 2 : 0, epi, s) : -1;
                if (rc != 0 && e.flag) { fprintf(stderr, "fortis_plan_run: fused upsample + conv3d shape not taken by the kernel\n"); break; }
                if (rc != 0)
                    rc = fortis_launch_conv3d(src, e.W, dst, o->C, o->D, o->H, o->W, o->F, o->KD, o->KH, o->KW, Do, Ho, Wo, o->pad,
                                              o->pad, o->pad, epi, s);
                break;
            }
            case EX_MAXPOOL: fortis_launch_maxpool2d(src, dst, o->C, o->H, o->W, o->KH, s); break;
            case EX_UPSAMPLE: fortis_launch_upsample(src, dst, o->C, o->D, o->H, o->W, o->sfac, o->nd, s); break;
            case EX_CONCAT: fortis_launch_concat_copy(src, dst + o->coff * o->H, o->C, o->H, o->coff, s); break;
            case EX_PERMUTE: fortis_launch_permute(src, dst, o->C, o->H, o->flag, s); break;
        }
        if (rc != 0) fprintf(stderr, "fortis_plan_run: an op was rejected by its kernel launcher\n");
        mark();
    }
}

// Rows [i0, i0 + n) of a plan whose kernels all work row by row (band_rows > 0), on the plan's own tensors: every
// tensor is addressed i0 rows in.  A boundary transpose reads or writes its host-side tensor as a compact
// column-major block of the band's n rows placed i0 rows (of the tensor's width) into it, so a band's input and
// output are contiguous ranges of the input and output tensors.
static void plan_run_rows(fortis_plan* p, long i0, long n, hipStream_t s)
{
    for (const Exec& e : p->exec) {
        char* src = (char*)p->tptr[e.src];
        char* dst = (char*)p->tptr[e.dst];
        int rc = 0;
        switch (e.kind) {
            case EX_CHAIN: {
                const long K0 = e.chain.L[0].K, NO = e.chain.L[e.chain.nlayers - 1].N;
                fortis_launch_chain(e.chain, (const float*)src + i0 * K0, (float*)dst + i0 * NO, n, s, e.rows);
                break;
            }
            case EX_GEMM: rc = fortis_launch_gemm((const float*)src + i0 * e.K, e.W, e.bias, (float*)dst + i0 * e.N, n, e.N, e.K, e.act, e.alpha, e.out_scale, e.mask_tail, s); break;
            case EX_SCALE: fortis_launch_scale((const float*)src + i0 * e.N, (float*)dst + i0 * e.N, e.vec, n, e.N, e.flag, s); break;
            case EX_MASK: fortis_launch_mask_relu((const float*)src + i0 * e.N, (float*)dst + i0 * e.N, n, e.N, e.mask_tail, s); break;
            case EX_PRE: fortis_launch_boundary_pre(src + i0 * e.N * e.flag, (float*)dst + i0 * e.N, n, e.N, e.p0, e.p1, e.p2, e.flag, s); break;
            case EX_POST: fortis_launch_boundary_post((const float*)src + i0 * e.N, dst + i0 * e.N * e.flag, n, e.N, e.p0, e.flag, s); break;
            default: rc = -1; break;
        }
        if (rc != 0) fprintf(stderr, "fortis_plan_run: an op was rejected by its kernel launcher\n");
    }
}

static const char* const kExecNames[] = { "mlp_chain", "gemm_bias_act", "scale", "mask_relu", "boundary_pre", "boundary_post",
                                          "conv2d", "convt2d", "maxpool2d", "upsample", "concat_copy", "conv3d", "permute" };
const char* fortis_plan_kernel_name(fortis_plan* p, int idx)
{
    if (!p || !p->finalized || idx < 0 || idx >= (int)p->exec.size()) return "";
    return kExecNames[p->exec[idx].kind];
}
void fortis_plan_profile(fortis_plan* p, int enable)
{
    if (!p) return;
    p->prof = enable != 0;
    p->ev_used = 0;
    if (!enable) { for (hipEvent_t e : p->ev) HIP_OK(hipEventDestroy(e)); p->ev.clear(); }
}
int fortis_plan_profile_read(fortis_plan* p, float* ms_per_kernel)
{
    if (!p || !p->finalized) return -1;
    const size_t per = p->exec.size() + 1;
    const int passes = (int)(p->ev_used / per);
    for (size_t k = 0; k < p->exec.size(); k++) ms_per_kernel[k] = 0.f;
    if (passes == 0) return 0;
    HIP_OK(hipEventSynchronize(p->ev[p->ev_used - 1]));
    for (int n = 0; n < passes; n++)
        for (size_t k = 0; k < p->exec.size(); k++) {
            float ms = 0.f;
            HIP_OK(hipEventElapsedTime(&ms, p->ev[n * per + k], p->ev[n * per + k + 1]));
            ms_per_kernel[k] += ms;
        }
    p->ev_used = 0;
    return passes;
}

void* fortis_plan_tensor_ptr(fortis_plan* p, int t)
{
    if (!p || !p->finalized || t < 0 || t >= (int)p->tptr.size()) return nullptr;
    return p->tptr[t];
}
int fortis_plan_num_kernels(fortis_plan* p) { return p && p->finalized ? (int)p->exec.size() : -1; }

}  // extern "C"

int fortis_plan_as_chain(fortis_plan* p, ChainDesc* out)
{
    if (!p || !p->finalized || p->exec.size() != 1 || p->exec[0].kind != EX_CHAIN) return -1;
    *out = p->exec[0].chain;
    return 0;
}

// Run-time extents: a row-wise plan runs on any row count.  Up to the rows its buffers were sized for only
// the launch extents change; beyond that every tensor grows in proportion and the buffers are assigned anew
// (the weights do not depend on the row count).  Plans with tensor windows keep their size.
static int plan_set_rows(fortis_plan* p, long rows)
{
    if (!p || !p->finalized || p->rows0 <= 0 || rows <= 0) return -1;
    if (rows > p->rows0) {
        for (int v : p->view_of) if (v >= 0) return -1;
        std::vector<long> old(p->tbytes);
        for (long& b : p->tbytes) b = (long)(((__int128)b * rows + p->rows0 - 1) / p->rows0);
        HIP_OK(hipStreamSynchronize(fortis_stream_get()));      // nothing in flight may still use the old buffers
        if (assign_buffers(p) != 0) {
            p->tbytes = old;
            if (assign_buffers(p) != 0) { fprintf(stderr, "fortis_plan: could not restore the plan's buffers\n"); p->finalized = false; }
            return -1;
        }
        p->rows0 = rows;
        for (Exec& e : p->exec) e.rows_cap = rows;
    }
    for (Exec& e : p->exec) e.rows = rows;
    return 0;
}

// ================================ step binding and entries ========================================
void fortis_stencil_reset_internal();

struct Step {
    fortis_plan* plan = nullptr;
    fortis_host_t h;
    void *din = nullptr, *dout = nullptr;
    void *X = nullptr, *Y = nullptr;          // pinned pack/unpack staging (driver/fortis_shim.py:102-106)
    hipGraphExec_t gexec = nullptr;
    int ncalls = 0;
    long count0 = 0;
};
static Step g_step;

static void drop_graph()
{
    if (g_step.gexec) { HIP_OK(hipGraphExecDestroy(g_step.gexec)); g_step.gexec = nullptr; }
    g_step.ncalls = 0;
}

extern "C" {

int fortis_step_bind(fortis_plan* p, const fortis_host_t* host)
{
    if (!p || !p->finalized || !host) return bad("step_bind: plan not finalized or host facts missing");
    if (host->n_in <= 0 || host->n_out <= 0 || (host->in_esz != 4 && host->in_esz != 8) || (host->out_esz != 4 && host->out_esz != 8))
        return bad("step_bind: bad sizes");
    if (p->tbytes[p->in_t] < host->n_in * host->in_esz || p->tbytes[p->out_t] < host->n_out * host->out_esz)
        return bad("step_bind: model input/output tensors smaller than the host's arrays");
    if (host->verdict == FORTIS_VERDICT_BATCHED && (host->count <= 0 || host->n_in % host->count || host->n_out % host->count))
        return bad("step_bind: batched verdict needs a row count dividing n_in and n_out");
    drop_graph();
    if (g_step.X) { HIP_OK(hipHostFree(g_step.X)); g_step.X = nullptr; }
    if (g_step.Y) { HIP_OK(hipHostFree(g_step.Y)); g_step.Y = nullptr; }
    g_step.plan = p;
    g_step.h = *host;
    g_step.din = p->tptr[p->in_t];
    g_step.dout = p->tptr[p->out_t];
    g_step.count0 = host->count;
    return 0;
}
void fortis_step_reset(void)
{
    drop_graph();
    if (g_step.X) { HIP_OK(hipHostFree(g_step.X)); }
    if (g_step.Y) { HIP_OK(hipHostFree(g_step.Y)); }
    g_step = Step();
    fortis_stencil_reset_internal();
}
int fortis_step_graph_active(void) { return g_step.gexec != nullptr; }

// A step file registers its binder instead of binding at load time: the binder runs at the first use of an
// entry point, like setup() in the reference's shim (driver/fortis_shim.py:64-73, `if (!din) setup();`), when
// the host's global vectors that the plan copies (boundary and lifted normalisation vectors) hold their values.
static void (*g_bind_on_use)(void) = nullptr;
void fortis_step_on_first_use(void (*bind)(void)) { g_bind_on_use = bind; }
static void bind_if_pending()
{
    if (g_step.plan || !g_bind_on_use) return;
    void (*f)(void) = g_bind_on_use;
    g_bind_on_use = nullptr;
    f();
}

static bool bound(const char* who)
{
    bind_if_pending();
    if (!g_step.plan) { fprintf(stderr, "%s: no step bound (fortis_step_bind was not called)\n", who); return false; }
    return true;
}

static long g_forward_gen = 0;   // bumped by every forward pass of the bound step
void* fortis_model_input(void) { bind_if_pending(); return g_step.din; }
void* fortis_model_output(void) { bind_if_pending(); return g_step.dout; }
long fortis_step_generation(void) { return g_forward_gen; }   // internal: lets the scatter entry notice a new forward pass

void mlp_forward_dev(void)
{
    if (!bound("mlp_forward_dev")) return;
    g_forward_gen++;
    hipStream_t s = fortis_stream_get();
    if (g_step.gexec) { HIP_OK(hipGraphLaunch(g_step.gexec, s)); return; }
    // Replay pays on this runtime only for steps of several kernels: one graph launch costs about as much as
    // five plain launches here (the opposite of the CUDA case FORTIS_GRAPH was built for), so a step of fewer
    // than FORTIS_GRAPH_MIN_KERNELS kernels (default 6) keeps running eagerly.  The rule depends on the plan
    // alone, never on timing, and no extra forward pass runs inside a caller's call.  FORTIS_GRAPH_KEEP in the
    // environment captures whatever the step's length.
    static int min_kernels = -1;
    if (min_kernels < 0) { const char* e = getenv("FORTIS_GRAPH_MIN_KERNELS"); min_kernels = e ? atoi(e) : 6; }
    const bool wanted = g_step.h.graph || getenv("FORTIS_GRAPH") != 0;
    const bool pays = (int)g_step.plan->exec.size() >= min_kernels || getenv("FORTIS_GRAPH_KEEP") != 0;
    const int cap = (++g_step.ncalls == 2) && wanted && pays;
    if (cap) {
        fortis_capturing = 1;
        if (hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal) != hipSuccess) {
            fortis_capturing = 0;
            (void)hipGetLastError();
            fprintf(stderr, "fortis: graph capture failed, running eagerly\n");
            fortis_plan_run(g_step.plan);
            return;
        }
    }
    fortis_plan_run(g_step.plan);
    if (cap) {
        hipGraph_t g = nullptr;
        fortis_capturing = 0;
        if (hipStreamEndCapture(s, &g) == hipSuccess && g && hipGraphInstantiate(&g_step.gexec, g, nullptr, nullptr, 0) == hipSuccess) {
            HIP_OK(hipGraphLaunch(g_step.gexec, s));
        } else {
            fprintf(stderr, "fortis: graph capture failed, running eagerly\n");
            g_step.gexec = nullptr;
            (void)hipGetLastError();
            fortis_plan_run(g_step.plan);
        }
        if (g) HIP_OK(hipGraphDestroy(g));
    }
}

static void setup_xy()
{
    // page-locked staging is allocated, never registered over existing host memory; without it the entries that
    // stage cannot run at all, which ends the program like the reference's failed specialisation does
    if (hipHostMalloc(&g_step.X, (size_t)g_step.h.n_in * g_step.h.in_esz, hipHostMallocDefault) != hipSuccess ||
        hipHostMalloc(&g_step.Y, (size_t)g_step.h.n_out * g_step.h.out_esz, hipHostMallocDefault) != hipSuccess) {
        fprintf(stderr, "fortis: no page-locked host memory for the staging buffers (%ld + %ld bytes)\n",
                g_step.h.n_in * g_step.h.in_esz, g_step.h.n_out * g_step.h.out_esz);
        exit(1);
    }
}

// ---- large host arrays: copies through page-locked staging, filled and drained by a few host threads --------
// A copy straight from or to pageable host memory runs at about 20 GB/s here (the runtime stages it on one
// thread) and existing host memory cannot be page-locked in place.  Arrays of 8 MB and more therefore go in
// chunks through the page-locked staging buffers (g_step.X / g_step.Y): worker threads copy chunks between
// the host array and staging while the DMA engine moves the chunks already copied.
// FORTIS_NO_STAGED_COPY=1 keeps the plain copies.
static void copy_streaming(void* dst, const void* src, size_t n);
#define STAGE_CHUNK ((size_t)4 << 20)
#define STAGE_THREADS 4
static bool staged_copies(size_t n)
{
    return n >= 2 * STAGE_CHUNK && getenv("FORTIS_NO_STAGED_COPY") == nullptr;
}
static void staged_h2d(void* dev, const void* host, void* stage, size_t n, hipStream_t s)
{
    const size_t nchunks = (n + STAGE_CHUNK - 1) / STAGE_CHUNK;
    std::atomic<size_t> next(0);
    auto work = [&]() {
        for (size_t c = next.fetch_add(1); c < nchunks; c = next.fetch_add(1)) {
            const size_t o = c * STAGE_CHUNK, len = o + STAGE_CHUNK < n ? STAGE_CHUNK : n - o;
            copy_streaming((char*)stage + o, (const char*)host + o, len);
            HIP_OK(hipMemcpyAsync((char*)dev + o, (char*)stage + o, len, hipMemcpyHostToDevice, s));
        }
    };
    std::thread th[STAGE_THREADS - 1];
    for (auto& t : th) t = std::thread(work);
    work();
    for (auto& t : th) t.join();       // every chunk's copy is enqueued: what follows on the stream sees the whole array
}
static void staged_d2h(void* host, const void* dev, void* stage, size_t n, hipStream_t s)
{
    const size_t nchunks = (n + STAGE_CHUNK - 1) / STAGE_CHUNK;
    static std::vector<hipEvent_t> ev;
    while (ev.size() < nchunks) {
        hipEvent_t e;
        HIP_OK(hipEventCreateWithFlags(&e, hipEventDisableTiming));
        ev.push_back(e);
    }
    for (size_t c = 0; c < nchunks; c++) {
        const size_t o = c * STAGE_CHUNK, len = o + STAGE_CHUNK < n ? STAGE_CHUNK : n - o;
        HIP_OK(hipMemcpyAsync((char*)stage + o, (const char*)dev + o, len, hipMemcpyDeviceToHost, s));
        HIP_OK(hipEventRecord(ev[c], s));
    }
    std::atomic<size_t> next(0);
    auto work = [&]() {
        for (size_t c = next.fetch_add(1); c < nchunks; c = next.fetch_add(1)) {
            const size_t o = c * STAGE_CHUNK, len = o + STAGE_CHUNK < n ? STAGE_CHUNK : n - o;
            HIP_OK(hipEventSynchronize(ev[c]));
            copy_streaming((char*)host + o, (const char*)stage + o, len);
        }
    };
    std::thread th[STAGE_THREADS - 1];
    for (auto& t : th) t = std::thread(work);
    work();
    for (auto& t : th) t.join();
}

void mlp_upload(void* in)
{
    if (!bound("mlp_upload")) return;
    const size_t n = (size_t)g_step.h.n_in * g_step.h.in_esz;
    hipStream_t s = fortis_stream_get();
    if (staged_copies(n)) {
        if (!g_step.X) setup_xy();
        // the staging buffer is reused: the previous call's chunks must have left it
        HIP_OK(hipStreamSynchronize(s));
        staged_h2d(g_step.din, in, g_step.X, n, s);
        return;
    }
    HIP_OK(hipMemcpyAsync(g_step.din, in, n, hipMemcpyHostToDevice, s));
}
void mlp_download(void* out)
{
    if (!bound("mlp_download")) return;
    hipStream_t s = fortis_stream_get();
    const size_t n = (size_t)g_step.h.n_out * g_step.h.out_esz;
    if (staged_copies(n)) {
        if (!g_step.Y) setup_xy();
        staged_d2h(out, g_step.dout, g_step.Y, n, s);
        return;
    }
    HIP_OK(hipMemcpyAsync(out, g_step.dout, n, hipMemcpyDeviceToHost, s));
    HIP_OK(hipStreamSynchronize(s));
}

void fortis_pack(void* row, int col)
{
    if (!bound("fortis_pack")) return;
    if (!g_step.X) setup_xy();
    const size_t nin = (size_t)(g_step.h.n_in / g_step.count0) * g_step.h.in_esz;
    memcpy((char*)g_step.X + (size_t)col * nin, row, nin);
}
void fortis_unpack(void* row, int col)
{
    if (!bound("fortis_unpack")) return;
    if (!g_step.Y) setup_xy();
    const size_t nout = (size_t)(g_step.h.n_out / g_step.count0) * g_step.h.out_esz;
    memcpy(row, (char*)g_step.Y + (size_t)col * nout, nout);
}

void mlp_forward_batched(void* in, void* out)
{
    if (!bound("mlp_forward_batched")) return;
    const fortis_host_t& h = g_step.h;
    hipStream_t s = fortis_stream_get();
    if (h.verdict != FORTIS_VERDICT_BATCHED) { fprintf(stderr, "mlp_forward_batched: the bound step is not a batched build\n"); return; }
    const size_t NIN = (size_t)(h.n_in / g_step.count0) * h.in_esz, NOUT = (size_t)(h.n_out / g_step.count0) * h.out_esz;
    if (h.expanded) {
        if (!g_step.X) setup_xy();
        if (!h.gather) HIP_OK(hipMemcpyAsync(g_step.din, g_step.X, NIN * h.count, hipMemcpyHostToDevice, s));
        mlp_forward_dev();
        if (!h.scatter) {
            HIP_OK(hipMemcpyAsync(g_step.Y, g_step.dout, NOUT * h.count, hipMemcpyDeviceToHost, s));
            HIP_OK(hipStreamSynchronize(s));
        }
        return;
    }
    if (h.step == 1 && h.minc == 1) {
        const bool big_in = staged_copies(NIN * h.count), big_out = staged_copies(NOUT * h.count);
        if ((big_in || big_out) && !g_step.X) setup_xy();
        if (big_in) { HIP_OK(hipStreamSynchronize(s)); staged_h2d(g_step.din, in, g_step.X, NIN * h.count, s); }
        else HIP_OK(hipMemcpyAsync(g_step.din, in, NIN * h.count, hipMemcpyHostToDevice, s));
        mlp_forward_dev();
        if (big_out) { staged_d2h(out, g_step.dout, g_step.Y, NOUT * h.count, s); return; }
        HIP_OK(hipMemcpyAsync(out, g_step.dout, NOUT * h.count, hipMemcpyDeviceToHost, s));
        HIP_OK(hipStreamSynchronize(s));
        return;
    }
    // strided / offset loop: rows minc, minc+|step|, ... of the host arrays (driver/fortis_shim.py:119-121, a
    // cudaMemcpy2D there).  Pitched copies from and to pageable memory are executed row by row by the runtime,
    // so the rows are packed by the CPU into page-locked staging and cross the bus as one copy each way.
    const long st = h.step < 0 ? -h.step : h.step;
    if (!g_step.X) setup_xy();
    for (long r = 0; r < h.count; r++)
        memcpy((char*)g_step.X + (size_t)r * NIN, (const char*)in + (size_t)(h.minc - 1 + r * st) * NIN, NIN);
    HIP_OK(hipMemcpyAsync(g_step.din, g_step.X, NIN * h.count, hipMemcpyHostToDevice, s));
    mlp_forward_dev();
    HIP_OK(hipMemcpyAsync(g_step.Y, g_step.dout, NOUT * h.count, hipMemcpyDeviceToHost, s));
    HIP_OK(hipStreamSynchronize(s));
    for (long r = 0; r < h.count; r++)
        memcpy((char*)out + (size_t)(h.minc - 1 + r * st) * NOUT, (const char*)g_step.Y + (size_t)r * NOUT, NOUT);
}

// ---- whole-array call on large host arrays, in row bands -------------------------------------------------------
// Rows are independent, so the call is cut into a few bands: while band b computes, band b + 1 crosses the bus and
// band b - 1 comes back (two copy streams beside the persistent one, events between them; all default priority).
// Host arrays are pageable and cannot be page-locked in place here, so every band goes through the page-locked
// staging buffers; a column-major boundary array is packed band by band into compact column-major blocks (one run
// per feature), which is the layout plan_run_rows gives a boundary transpose.  FORTIS_BANDS=n sets the count
// (1: the whole array at once, as without this path).
static hipStream_t g_up = nullptr, g_down = nullptr;
// memcpy whose stores do not go through the CPU's caches: the bands' copies write megabytes that the CPU does not read
// again (staging that the DMA engine reads, a host array the caller reads much later), and an ordinary store first
// reads the line it is about to overwrite, which is a third of the memory traffic of a copy that is bound by it.
// FORTIS_PLAIN_MEMCPY=1 keeps memcpy.
typedef float hv4f __attribute__((ext_vector_type(4)));
static void copy_streaming(void* dst, const void* src, size_t n)
{
    static const bool plain = getenv("FORTIS_PLAIN_MEMCPY") != nullptr;
    char* d = (char*)dst;
    const char* s = (const char*)src;
    if (plain || n < 4096) { memcpy(d, s, n); return; }
    const size_t head = (16 - ((uintptr_t)d & 15)) & 15;
    memcpy(d, s, head);
    d += head; s += head; n -= head;
    const size_t nv = n / 64;
    for (size_t i = 0; i < nv; i++) {
        hv4f a, b, c, e;
        memcpy(&a, s + 64 * i, 16); memcpy(&b, s + 64 * i + 16, 16); memcpy(&c, s + 64 * i + 32, 16); memcpy(&e, s + 64 * i + 48, 16);
        __builtin_nontemporal_store(a, (hv4f*)(d + 64 * i));
        __builtin_nontemporal_store(b, (hv4f*)(d + 64 * i + 16));
        __builtin_nontemporal_store(c, (hv4f*)(d + 64 * i + 32));
        __builtin_nontemporal_store(e, (hv4f*)(d + 64 * i + 48));
    }
    memcpy(d + 64 * nv, s + 64 * nv, n - 64 * nv);
    __atomic_thread_fence(__ATOMIC_SEQ_CST);      // the streamed stores are visible before the copy is reported done
}
// Host copies are what bounds such a call (the bus and the GPU are faster than four threads copy), so the runs of a
// band are dealt to a pool of threads that lives as long as the process (FORTIS_COPY_THREADS, default 12; starting
// threads for every band cost about 0.1 ms each time).
struct CopyPool {
    std::mutex m;
    std::condition_variable go, done;
    const std::function<void(long)>* fn = nullptr;
    long nruns = 0, gen = 0;
    std::atomic<long> next{0};
    int busy = 0, nthreads = 0;
    void worker()
    {
        long seen = 0;
        for (;;) {
            const std::function<void(long)>* f;
            long n;
            {
                std::unique_lock<std::mutex> l(m);
                go.wait(l, [&] { return gen != seen; });
                seen = gen; f = fn; n = nruns;
            }
            for (long k = next.fetch_add(1); k < n; k = next.fetch_add(1)) (*f)(k);
            {
                std::lock_guard<std::mutex> l(m);
                if (--busy == 0) done.notify_one();
            }
        }
    }
    void run(long n, const std::function<void(long)>& f)
    {
        if (!nthreads) {
            const char* e = getenv("FORTIS_COPY_THREADS");
            nthreads = e ? atoi(e) : 12;
            if (nthreads < 1) nthreads = 1;
            if (nthreads > 32) nthreads = 32;
            for (int t = 1; t < nthreads; t++) std::thread([this] { worker(); }).detach();
        }
        {
            std::lock_guard<std::mutex> l(m);
            fn = &f; nruns = n; next = 0; busy = nthreads - 1; gen++;
        }
        go.notify_all();
        for (long k = next.fetch_add(1); k < n; k = next.fetch_add(1)) f(k);
        std::unique_lock<std::mutex> l(m);
        done.wait(l, [&] { return busy == 0; });
    }
};
static void parallel_runs(long nruns, const std::function<void(long)>& run)
{
    static CopyPool* pool = new CopyPool();      // never destroyed: its threads wait for work until the process ends
    pool->run(nruns, run);
}
static int forward_banded(void* in, void* out)
{
    fortis_plan* p = g_step.plan;
    const fortis_host_t& h = g_step.h;
    const long rows = p->band_rows;
    const char* env = getenv("FORTIS_BANDS");
    const int want = env ? atoi(env) : 0;
    long nb = want > 0 ? want : rows / 6144;            // whole bands of about 8192 rows, half bands at both ends
    if (nb > 8) nb = 8;
    if (nb < 2 || rows <= 0 || h.n_in % rows || h.n_out % rows || p->in_t == p->out_t) return -1;
    const long win = h.n_in / rows, wout = h.n_out / rows;           // elements per row
    const size_t ein = (size_t)h.in_esz, eout = (size_t)h.out_esz;
    const bool in_cm = p->exec.front().kind == EX_PRE, out_cm = p->exec.back().kind == EX_POST;
    hipStream_t s = fortis_stream_get();
    if (!g_up) { HIP_OK(hipStreamCreateWithFlags(&g_up, hipStreamNonBlocking)); HIP_OK(hipStreamCreateWithFlags(&g_down, hipStreamNonBlocking)); }
    static std::vector<hipEvent_t> ev;
    while (ev.size() < (size_t)3 * 8) { hipEvent_t e; HIP_OK(hipEventCreateWithFlags(&e, hipEventDisableTiming)); ev.push_back(e); }
    if (!g_step.X) setup_xy();
    HIP_OK(hipStreamSynchronize(s));                    // the staging buffers and the tensors are free again
    HIP_OK(hipStreamSynchronize(g_up));
    HIP_OK(hipStreamSynchronize(g_down));
    // band edges: the first and the last band are half bands (the first computation starts, and the last copy back
    // ends, half a band sooner), every edge a multiple of 128 rows
    long edge[10];
    {
        const long q = (rows / (2 * (nb - 1)) + 127) / 128 * 128;
        edge[0] = 0;
        for (long b = 1; b <= nb; b++) { const long e = q * (2 * b - 1); edge[b] = b == nb || e > rows ? rows : e; }
    }
    g_forward_gen++;
    for (long b = 0; b < nb; b++) {
        const long i0 = edge[b], n = edge[b + 1] - edge[b];
        if (n <= 0) continue;
        char* stage = (char*)g_step.X + (size_t)i0 * win * ein;
        if (in_cm) parallel_runs(win, [&](long k) { copy_streaming(stage + (size_t)k * n * ein, (const char*)in + ((size_t)k * rows + i0) * ein, (size_t)n * ein); });
        else {
            const size_t bytes = (size_t)n * win * ein, piece = (bytes / 32 + 4095) & ~(size_t)4095;
            parallel_runs(32, [&](long k) { const size_t o = (size_t)k * piece; if (o < bytes) copy_streaming(stage + o, (const char*)in + (size_t)i0 * win * ein + o, o + piece < bytes ? piece : bytes - o); });
        }
        HIP_OK(hipMemcpyAsync((char*)g_step.din + (size_t)i0 * win * ein, stage, (size_t)n * win * ein, hipMemcpyHostToDevice, g_up));
        HIP_OK(hipEventRecord(ev[3 * b], g_up));
        HIP_OK(hipStreamWaitEvent(s, ev[3 * b], 0));
        plan_run_rows(p, i0, n, s);
        HIP_OK(hipEventRecord(ev[3 * b + 1], s));
        HIP_OK(hipStreamWaitEvent(g_down, ev[3 * b + 1], 0));
        HIP_OK(hipMemcpyAsync((char*)g_step.Y + (size_t)i0 * wout * eout, (char*)g_step.dout + (size_t)i0 * wout * eout, (size_t)n * wout * eout, hipMemcpyDeviceToHost, g_down));
        HIP_OK(hipEventRecord(ev[3 * b + 2], g_down));
    }
    for (long b = 0; b < nb; b++) {
        const long i0 = edge[b], n = edge[b + 1] - edge[b];
        if (n <= 0) continue;
        const char* stage = (const char*)g_step.Y + (size_t)i0 * wout * eout;
        HIP_OK(hipEventSynchronize(ev[3 * b + 2]));
        if (out_cm) parallel_runs(wout, [&](long k) { copy_streaming((char*)out + ((size_t)k * rows + i0) * eout, stage + (size_t)k * n * eout, (size_t)n * eout); });
        else {
            const size_t bytes = (size_t)n * wout * eout, piece = (bytes / 32 + 4095) & ~(size_t)4095;
            parallel_runs(32, [&](long k) { const size_t o = (size_t)k * piece; if (o < bytes) copy_streaming((char*)out + (size_t)i0 * wout * eout + o, stage + o, o + piece < bytes ? piece : bytes - o); });
        }
    }
    HIP_OK(hipStreamSynchronize(s));
    return 0;
}

void mlp_forward(void* in, void* out)
{
    if (!bound("mlp_forward")) return;
    const fortis_host_t& h = g_step.h;
    hipStream_t s = fortis_stream_get();
    if (h.verdict == FORTIS_VERDICT_BATCHED) {
        // a call outside the distributed loop: one row through the batched model (driver/fortis_shim.py:122)
        const size_t NIN = (size_t)(h.n_in / g_step.count0) * h.in_esz, NOUT = (size_t)(h.n_out / g_step.count0) * h.out_esz;
        HIP_OK(hipMemcpyAsync(g_step.din, in, NIN, hipMemcpyHostToDevice, s));
        mlp_forward_dev();
        HIP_OK(hipMemcpyAsync(out, g_step.dout, NOUT, hipMemcpyDeviceToHost, s));
        HIP_OK(hipStreamSynchronize(s));
        return;
    }
    // Small whole-array calls skip both copies: the input is written into page-locked host memory that the
    // first kernel reads over the bus, and the last kernel writes the output into page-locked host memory.
    // Two copy commands cost more than the step itself at these sizes.  (After such a call the resident
    // device buffers behind fortis_model_input/output are not refreshed; hosts that use the resident entries
    // go through mlp_upload / mlp_download, which always copy.)
    const size_t nin = (size_t)h.n_in * h.in_esz, nout = (size_t)h.n_out * h.out_esz;
    fortis_plan* p = g_step.plan;
    bool direct = nin <= 32 * 1024 && nout <= 32 * 1024 && !getenv("FORTIS_NO_ZEROCOPY") && p->in_t != p->out_t;
    for (size_t t = 0; direct && t < p->view_of.size(); t++)
        if (p->view_of[t] == p->in_t || p->view_of[t] == p->out_t) direct = false;
    if (direct) {
        if (!g_step.X) setup_xy();
        memcpy(g_step.X, in, nin);
        void* din = p->tptr[p->in_t];
        void* dout = p->tptr[p->out_t];
        p->tptr[p->in_t] = g_step.X;
        p->tptr[p->out_t] = g_step.Y;
        g_forward_gen++;
        fortis_plan_run(p);
        p->tptr[p->in_t] = din;
        p->tptr[p->out_t] = dout;
        HIP_OK(hipStreamSynchronize(s));
        memcpy(out, g_step.Y, nout);
        return;
    }
    // large arrays of a step whose kernels all work row by row: in row bands, copies under the computation (after
    // such a call the resident buffers hold a boundary array band by band, not as the host's array)
    if (staged_copies(nin) && staged_copies(nout) && p->band_rows > 0 && forward_banded(in, out) == 0) return;
    mlp_upload(in);
    mlp_forward_dev();
    mlp_download(out);
}

void fortis_begin(int count)
{
    if (!bound("fortis_begin")) return;
    fortis_host_t& h = g_step.h;
    if (h.verdict != FORTIS_VERDICT_BATCHED || count <= 0) {
        fprintf(stderr, "fortis_begin: %d rows cannot be specialised (the bound step is %s)\n", count,
                h.verdict != FORTIS_VERDICT_BATCHED ? "not a batched build" : "batched");
        exit(1);   // the reference stub exits when it cannot specialise (driver/fortis_stub.c:23)
    }
    if (count == h.count) return;
    const long per = g_step.plan->rows0 / g_step.count0;   // model rows per cell (enclosing-loop distribution)
    const long nin_row = h.n_in / g_step.count0, nout_row = h.n_out / g_step.count0;
    if (plan_set_rows(g_step.plan, (long)count * per) != 0) {
        fprintf(stderr, "fortis_begin: the bound model cannot be re-sized to %d rows (not row-wise, tensor windows, or out of memory)\n", count);
        exit(1);
    }
    if (count > g_step.count0) {
        // the step grew: its buffers moved and the host-side staging is too small
        g_step.count0 = count;
        h.n_in = nin_row * count; h.n_out = nout_row * count;
        g_step.din = g_step.plan->tptr[g_step.plan->in_t];
        g_step.dout = g_step.plan->tptr[g_step.plan->out_t];
        if (g_step.X) { HIP_OK(hipHostFree(g_step.X)); g_step.X = nullptr; }
        if (g_step.Y) { HIP_OK(hipHostFree(g_step.Y)); g_step.Y = nullptr; }
    }
    h.count = count;
    drop_graph();
}

// ---- timing ----------------------------------------------------------------------------------------
float fortis_time_ms(void (*fn)(void*), void* arg, int iters)
{
    hipStream_t s = fortis_stream_get();
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
    HIP_OK(hipEventRecord(e0, s));
    for (int i = 0; i < iters; i++) fn(arg);
    HIP_OK(hipEventRecord(e1, s));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    HIP_OK(hipEventDestroy(e0)); HIP_OK(hipEventDestroy(e1));
    return ms;
}
// A step made of several enqueues, clocked part by part: events between the parts, no host wait inside a
// pass, so every part runs right behind the one before it as it does in the step itself.
int fortis_time_parts_ms(int nparts, void (*const* fns)(void*), void* const* args, int iters, float* ms_out)
{
    if (nparts <= 0 || nparts > 16 || iters <= 0 || iters > 4096 || !fns || !ms_out) return -1;
    hipStream_t s = fortis_stream_get();
    std::vector<hipEvent_t> ev((size_t)iters * (nparts + 1));
    for (auto& e : ev) HIP_OK(hipEventCreate(&e));
    for (int it = 0; it < iters; it++) {
        hipEvent_t* e = &ev[(size_t)it * (nparts + 1)];
        HIP_OK(hipEventRecord(e[0], s));
        for (int k = 0; k < nparts; k++) {
            fns[k](args ? args[k] : nullptr);
            HIP_OK(hipEventRecord(e[k + 1], s));
        }
    }
    HIP_OK(hipEventSynchronize(ev.back()));
    for (int k = 0; k < nparts; k++) ms_out[k] = 0.f;
    for (int it = 0; it < iters; it++)
        for (int k = 0; k < nparts; k++) {
            float ms = 0.f;
            HIP_OK(hipEventElapsedTime(&ms, ev[(size_t)it * (nparts + 1) + k], ev[(size_t)it * (nparts + 1) + k + 1]));
            ms_out[k] += ms;
        }
    for (auto& e : ev) HIP_OK(hipEventDestroy(e));
    return 0;
}
static void run_plan_cb(void* p) { fortis_plan_run((fortis_plan*)p); }
float fortis_plan_time_ms(fortis_plan* p, int iters, int use_graph)
{
    if (!p || !p->finalized || iters <= 0) return -1.f;
    hipStream_t s = fortis_stream_get();
    if (!use_graph) return fortis_time_ms(run_plan_cb, p, iters);
    hipGraph_t g = nullptr;
    hipGraphExec_t ge = nullptr;
    fortis_plan_run(p);   // first pass eager: function attributes and lazy state settle outside capture
    HIP_OK(hipStreamSynchronize(s));
    if (hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal) != hipSuccess) return -1.f;
    fortis_plan_run(p);
    if (hipStreamEndCapture(s, &g) != hipSuccess || !g || hipGraphInstantiate(&ge, g, nullptr, nullptr, 0) != hipSuccess) {
        (void)hipGetLastError();
        if (g) HIP_OK(hipGraphDestroy(g));
        return -1.f;
    }
    HIP_OK(hipGraphLaunch(ge, s));
    HIP_OK(hipStreamSynchronize(s));
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0)); HIP_OK(hipEventCreate(&e1));
    HIP_OK(hipEventRecord(e0, s));
    for (int i = 0; i < iters; i++) HIP_OK(hipGraphLaunch(ge, s));
    HIP_OK(hipEventRecord(e1, s));
    HIP_OK(hipEventSynchronize(e1));
    float ms = 0.f;
    HIP_OK(hipEventElapsedTime(&ms, e0, e1));
    HIP_OK(hipEventDestroy(e0)); HIP_OK(hipEventDestroy(e1));
    HIP_OK(hipGraphExecDestroy(ge)); HIP_OK(hipGraphDestroy(g));
    return ms;
}

}  // extern "C"
