"""Model plan builder: the op list fortis-fuse would emit for a model, handed to the library.

In the reference the exporter produces linalg MLIR and `fortis-opt -fortis-fuse` turns it into
kernels plus fortis_gemm / fortis_conv* calls (compiler/FortisFuse.cpp:575-771).  No MLIR tool
chain exists beside this backend, so the same information (ops in program order, shapes, weights)
is given to the library directly through fortis_plan_* (include/fortis_step.h).
"""
import ctypes as C

import numpy as np

from ._lib import lib

ACT = {None: 0, "none": 0, "relu": 1, "leaky": 2}


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


class Plan:
    """Thin owner of a fortis_plan*.  Tensor ids are ints; shapes are the caller's business."""

    def __init__(self):
        self._L = lib()
        self._p = self._L.fortis_plan_create()
        self._keep = []
        self.in_tensor = self.out_tensor = None

    def close(self):
        if self._p:
            self._L.fortis_plan_destroy(self._p)
            self._p = None

    @property
    def handle(self):
        return self._p

    def _ok(self, rc, what):
        if rc != 0:
            raise ValueError(f"fortis_plan_{what} rejected its arguments (see stderr)")

    def tensor(self, nelem, esz=4):
        t = self._L.fortis_plan_tensor(self._p, int(nelem) * esz)
        if t < 0:
            raise ValueError("fortis_plan_tensor failed")
        return t

    def view(self, base, elem_offset, nelem, esz=4):
        t = self._L.fortis_plan_view(self._p, base, int(elem_offset) * esz, int(nelem) * esz)
        if t < 0:
            raise ValueError("fortis_plan_view failed (see stderr)")
        return t

    def linear(self, src, dst, W, bias, B, act=None, alpha=0.0):
        W = _f32(W)
        N, K = W.shape
        b = None if bias is None else _f32(bias)
        self._ok(self._L.fortis_plan_linear(self._p, src, dst, _p(W), _p(b), B, K, N, ACT[act], alpha), "linear")

    def scale(self, src, dst, vec, rows, divide):
        v = _f32(vec)
        self._ok(self._L.fortis_plan_scale(self._p, src, dst, _p(v), rows, v.size, 1 if divide else 0), "scale")

    def mask_relu(self, src, dst, rows, n, tail):
        self._ok(self._L.fortis_plan_mask_relu(self._p, src, dst, rows, n, tail), "mask_relu")

    def boundary_pre(self, src, dst, NI, NK, mean=None, vmax=None, vmin=None, host_dtype=np.float32):
        esz = np.dtype(host_dtype).itemsize
        vs = [None if v is None else np.ascontiguousarray(v, dtype=host_dtype) for v in (mean, vmax, vmin)]
        self._ok(self._L.fortis_plan_boundary_pre(self._p, src, dst, NI, NK, _p(vs[0]), _p(vs[1]), _p(vs[2]), esz), "boundary_pre")

    def boundary_post(self, src, dst, NI, NK, scale=None, host_dtype=np.float32):
        esz = np.dtype(host_dtype).itemsize
        s = None if scale is None else np.ascontiguousarray(scale, dtype=host_dtype)
        self._ok(self._L.fortis_plan_boundary_post(self._p, src, dst, NI, NK, _p(s), esz), "boundary_post")

    def conv2d(self, src, dst, W, bias, C_, H, Wd, stride=1, pad=0, act=None, alpha=0.0, bn=None, bn_eps=1e-5,
               coff=0, ctot=0):
        W = _f32(W)
        F, Cw, KH, KW = W.shape
        assert Cw == C_
        b = None if bias is None else _f32(bias)
        g = be = m = v = None
        if bn is not None:
            g, be, m, v = [_f32(t) for t in bn]
        self._ok(self._L.fortis_plan_conv2d(self._p, src, dst, _p(W), _p(b), _p(g), _p(be), _p(m), _p(v), bn_eps, C_, H, Wd,
                                            F, KH, KW, stride, pad, ACT[act], alpha, coff, ctot), "conv2d")

    def convt2d(self, src, dst, W, bias, C_, H, Wd, stride, pad=0, output_padding=0, act=None, alpha=0.0, coff=0, ctot=0):
        W = _f32(W)
        Cw, F, KH, KW = W.shape
        assert Cw == C_
        b = None if bias is None else _f32(bias)
        self._ok(self._L.fortis_plan_convt2d(self._p, src, dst, _p(W), _p(b), C_, H, Wd, F, KH, KW, stride, pad,
                                             output_padding, ACT[act], alpha, coff, ctot), "convt2d")

    def maxpool2d(self, src, dst, C_, H, Wd, k=2):
        self._ok(self._L.fortis_plan_maxpool2d(self._p, src, dst, C_, H, Wd, k), "maxpool2d")

    def upsample(self, src, dst, C_, D, H, Wd, s=2, nd=2):
        self._ok(self._L.fortis_plan_upsample(self._p, src, dst, C_, D, H, Wd, s, nd), "upsample")

    def concat_copy(self, src, dst, C_, S, coff, ctot):
        self._ok(self._L.fortis_plan_concat_copy(self._p, src, dst, C_, S, coff, ctot), "concat_copy")

    def conv3d(self, src, dst, W, bias, C_, D, H, Wd, pad=0, act=None, alpha=0.0, res=-1):
        W = _f32(W)
        F, Cw, K, K2, K3 = W.shape
        assert Cw == C_ and K == K2 == K3
        b = None if bias is None else _f32(bias)
        self._ok(self._L.fortis_plan_conv3d(self._p, src, dst, res, _p(W), _p(b), C_, D, H, Wd, F, K, pad, ACT[act], alpha), "conv3d")

    def permute(self, src, dst, C_, S, to_channels_first):
        self._ok(self._L.fortis_plan_permute(self._p, src, dst, C_, S, 1 if to_channels_first else 0), "permute")

    def finalize(self, in_tensor, out_tensor):
        self._ok(self._L.fortis_plan_finalize(self._p, in_tensor, out_tensor), "finalize")
        self.in_tensor, self.out_tensor = in_tensor, out_tensor
        return self

    # --- running and moving data (through the C ABI) ---
    def run(self):
        self._L.fortis_plan_run(self._p)

    def ptr(self, tensor):
        return self._L.fortis_plan_tensor_ptr(self._p, tensor)

    def write(self, tensor, array):
        a = np.ascontiguousarray(array)
        self._L.fortis_h2d(self.ptr(tensor), _p(a), a.nbytes)

    def read(self, tensor, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        self._L.fortis_d2h(_p(out), self.ptr(tensor), out.nbytes)
        return out

    def forward(self, x, out_shape, out_dtype=np.float32):
        self.write(self.in_tensor, x)
        self.run()
        return self.read(self.out_tensor, out_shape, out_dtype)

    @property
    def num_kernels(self):
        return self._L.fortis_plan_num_kernels(self._p)

    def kernel_names(self):
        return [self._L.fortis_plan_kernel_name(self._p, k).decode() for k in range(self.num_kernels)]

    def profile(self, enable=True):
        self._L.fortis_plan_profile(self._p, 1 if enable else 0)

    def profile_read(self):
        """-> (passes, [(kernel name, total ms over the passes)])"""
        n = self.num_kernels
        ms = (C.c_float * n)()
        passes = self._L.fortis_plan_profile_read(self._p, ms)
        return passes, [(self._L.fortis_plan_kernel_name(self._p, k).decode(), float(ms[k])) for k in range(n)]

    def time_ms(self, iters, graph=False):
        return self._L.fortis_plan_time_ms(self._p, iters, 1 if graph else 0)


def mlp_plan(Ws, bs, acts, rows, alphas=None, in_norms=None, out_norms=None, mask_tail=0, plan_cls=None):
    """Linear stack as a plan: optional x/in_norms, Linear+act layers, optional *out_norms, optional
    masked-ReLU head (benchmarks/climsim/export_wide.py:27-28; mom6_zb/export_zb.py:10-16).  plan_cls: a class
    with Plan's interface to fill instead (the op-list recorder of fortis_amd.shim_hip)."""
    p = (plan_cls or Plan)()
    widths = [Ws[0].shape[1]] + [w.shape[0] for w in Ws]
    t_in = p.tensor(rows * widths[0])
    cur = t_in
    if in_norms is not None:
        t = p.tensor(rows * widths[0])
        p.scale(cur, t, in_norms, rows, divide=True)
        cur = t
    for l, (W, b) in enumerate(zip(Ws, bs)):
        t = p.tensor(rows * widths[l + 1])
        p.linear(cur, t, W, b, rows, acts[l], 0.0 if alphas is None else float(alphas[l]))
        cur = t
    if out_norms is not None:
        t = p.tensor(rows * widths[-1])
        p.scale(cur, t, out_norms, rows, divide=False)
        cur = t
    if mask_tail:
        t = p.tensor(rows * widths[-1])
        p.mask_relu(cur, t, rows, widths[-1], mask_tail)
        cur = t
    return p.finalize(t_in, cur)
