#!/usr/bin/env python3
"""Reader of the model's linalg text: model_args.mlir (what driver/fortis_outline.py:13-24 writes: the
torch-mlir linalg-on-tensors export with its weight constants turned into function arguments) -> ops.json, the
op groups in program order that fortis_amd.shim_hip turns into the plan calls of step_tables.c.

    python -m fortis_amd.mlir_ops <model_args.mlir> <outline.json> <outdir>      # writes <outdir>/ops.json

In the CUDA build these groups are decided by fortis-fuse (compiler/FortisFuse.cpp:575-771) and end up as
kernels and fortis_gemm / fortis_conv* calls inside model.o; for this backend the same decisions are taken by
the plan at finalize (bias / activation / scale folded into the producing GEMM or conv, narrow stacks fused
into one kernel), so the reader only has to name the operations.  It works on the text with regular
expressions, like the reference's own driver scripts (driver/fortis_outline.py, driver/fortis_shim.py).

What it recognises (anything else is an error that names the statement):
  * a Linear layer as torch-mlir writes it: linalg.transpose of a weight argument, linalg.fill of zero,
    linalg.matmul (or linalg.batch_matmul-free 2-D form), then a linalg.generic that adds a rank-1 argument
    broadcast over the rows;
  * activations as elementwise linalg.generic: ReLU (arith.cmpf ugt/ogt against 0 + arith.select, or
    arith.maximumf / arith.maxnumf with 0), LeakyReLU (compare, multiply by a constant, select);
  * per-feature scaling: a generic that divides or multiplies by a rank-1 argument broadcast over the rows
    (mom6_zb/export_zb.py:14-16 `x / in_norms`, `y * out_norms`);
  * the boundary wrapper @fortis_main that driver/fortis_emit2d.py:20-52 puts around the model: its two
    transposing generics with the lifted expressions (a - mean) / (max - min) [-> truncf] and
    [extf ->] y / scale over the host's extra arguments;
  * linalg.conv_2d_nchw_fchw / linalg.conv_3d_ncdhw_fcdhw with unit dilation over a tensor.pad of the input (or
    none), a bias added by a generic broadcast over the channel dimension, and linalg.pooling_nchw_max 2 x 2.
No .mlir file is checked into the reference, so the statement forms above are those of the reference's emitters
where one exists (fortis_emit2d.py, fortis_outline.py) and of the torch-mlir exporter's usual output otherwise.
"""
import json
import os
import re
import sys

import numpy as np

from .shim_hip import OpList, tensor_type


class MlirError(ValueError):
    pass


_TY = r"tensor<[^>]+>"


def _shape(t):
    return tensor_type(t)[0]


def _func(src, name=None):
    """(name, [(arg, type)], result type, body text) of func.func @name (the first one when name is None)."""
    pat = r"func\.func (?:private )?@(%s)\(((?:%%\w+: %s(?:, )?)*)\) -> (%s)(?: attributes \{.*?\})? \{" % (name or r"\w+", _TY, _TY)
    m = re.search(pat, src, re.S)
    if not m:
        raise MlirError("no func.func %s with tensor arguments and one tensor result" % ("@" + name if name else ""))
    depth, p = 1, m.end()
    while depth and p < len(src):
        depth += {"{": 1, "}": -1}.get(src[p], 0)
        p += 1
    return m.group(1), re.findall(r"(%%\w+): (%s)" % _TY, m.group(2)), m.group(3), src[m.end():p - 1]


_GENERIC = re.compile(r"(%[\w#]+) = linalg\.generic \{indexing_maps = \[(.*?)\], iterator_types = \[(.*?)\]\} "
                      r"ins\((.*?) : (.*?)\) outs\((%[\w#]+) : (" + _TY + r")\) \{\s*\^bb0\((.*?)\):(.*?)linalg\.yield (%[\w#]+) : \w+\s*\} -> (" + _TY + ")", re.S)
_SIMPLE = [
    ("empty", re.compile(r"(%[\w#]+) = tensor\.empty\(\) : (" + _TY + ")")),
    ("const", re.compile(r"(%[\w#]+) = arith\.constant (-?[\d.eE+-]+|0x[0-9A-Fa-f]+) : (f32|f64)")),
    ("fill", re.compile(r"(%[\w#]+) = linalg\.fill ins\((%[\w#]+) : \w+\) outs\((%[\w#]+) : (" + _TY + r")\) -> " + _TY)),
    ("transpose", re.compile(r"(%[\w#]+) = linalg\.transpose ins\((%[\w#]+) : (" + _TY + r")\) outs\((%[\w#]+) : (" + _TY + r")\) permutation = \[1, 0\]")),
    ("matmul", re.compile(r"(%[\w#]+) = linalg\.matmul ins\((%[\w#]+), (%[\w#]+) : (" + _TY + "), (" + _TY + r")\) outs\((%[\w#]+) : (" + _TY + r")\) -> " + _TY)),
    ("pad", re.compile(r"(%[\w#]+) = tensor\.pad (%[\w#]+) low\[([\d, ]+)\] high\[([\d, ]+)\] \{.*?tensor\.yield (%[\w#]+) : \w+\s*\} : (" + _TY + ") to (" + _TY + ")", re.S)),
    ("conv", re.compile(r"(%[\w#]+) = linalg\.conv_(2d_nchw_fchw|3d_ncdhw_fcdhw) \{dilations = dense<1> : tensor<\dxi64>, strides = dense<(\d+)> : tensor<\dxi64>\} "
                        r"ins\((%[\w#]+), (%[\w#]+) : (" + _TY + "), (" + _TY + r")\) outs\((%[\w#]+) : (" + _TY + r")\) -> " + _TY)),
    ("maxpool", re.compile(r"(%[\w#]+) = linalg\.pooling_nchw_max \{dilations = dense<1> : tensor<2xi64>, strides = dense<(\d+)> : tensor<2xi64>\} "
                           r"ins\((%[\w#]+), (%[\w#]+) : (" + _TY + "), (" + _TY + r")\) outs\((%[\w#]+) : (" + _TY + r")\) -> " + _TY)),
    ("call", re.compile(r"(%[\w#]+) = (?:func\.)?call @(\w+)\((%[\w#]+)\) : \((" + _TY + r")\) -> (" + _TY + ")")),
    ("return", re.compile(r"return (%[\w#]+) : (" + _TY + ")")),
]


def _statements(body):
    """The statements of a function body in program order: (kind, match).  Statements inside the region of a
    linalg.generic or a tensor.pad belong to that statement and are not listed."""
    out = [(m.start(), m.end(), "generic", m) for m in _GENERIC.finditer(body)]
    out += [(m.start(), m.end(), "pad", m) for m in dict(_SIMPLE)["pad"].finditer(body)]
    regions = [(a, b) for a, b, _, _ in out]
    for kind, rx in _SIMPLE:
        if kind == "pad":
            continue
        for m in rx.finditer(body):
            if not any(a <= m.start() < b for a, b in regions):
                out.append((m.start(), m.end(), kind, m))
    return [(k, m) for _, _, k, m in sorted(out, key=lambda s: s[0])]


def _body_ops(text):
    return [(m.group(1), m.group(2), [a.strip() for a in m.group(3).split(",")])
            for m in re.finditer(r"(%[\w#]+) = (arith\.\w+|math\.\w+)\s+(.*?) : ", text)]


class _Reader:
    def __init__(self, ops, arg_names):
        self.ops, self.arg = ops, arg_names           # SSA argument -> "x" | "w<i>" | "g<i>"
        self.val = {}                                 # SSA value -> descriptor dict
        self.tensor_of = {}                           # SSA value -> plan tensor index

    def fail(self, m, why):
        raise MlirError("%s: %s" % (why, " ".join(m.group(0).split())[:160]))

    def T(self, v, ty, esz=4):
        if v not in self.tensor_of:
            self.tensor_of[v] = self.ops.tensor(int(np.prod(_shape(ty))), esz)
        return self.tensor_of[v]

    def scalar(self, v):
        d = self.val.get(v)
        return d["value"] if d and d["kind"] == "const" else None

    def generic(self, m):
        res, maps, iters, ins, in_tys, out, out_ty, bbargs, body, yielded, res_ty = m.groups()
        ins = [a.strip() for a in ins.split(",")]
        in_tys = re.findall(_TY, in_tys)
        maps = re.findall(r"affine_map<\((.*?)\) -> \((.*?)\)>", maps)
        bb = [a.split(":")[0].strip() for a in bbargs.split(",")]
        bops = _body_ops(body)
        if "reduction" in iters:
            self.fail(m, "a reduction written as linalg.generic is not a form this reader names")
        shape = _shape(res_ty)
        src = ins[0]
        # boundary pre / post of driver/fortis_emit2d.py: first operand read transposed
        if len(shape) == 2 and maps[0][1].replace(" ", "") == "d1,d0":
            return self.boundary(m, res, res_ty, ins, in_tys, bb, bops, yielded)
        # a rank-1 argument broadcast into the result shape (body yields its input): the bias a convolution starts from
        if len(ins) == 1 and not bops and src in self.arg and len(_shape(in_tys[0])) == 1 and yielded == bb[0]:
            self.val[res] = dict(kind="bias_bcast", name=self.arg[src])
            return
        if src not in self.tensor_of and src not in self.arg:
            self.fail(m, "operand %s has no producer this reader knows" % src)
        s_t = self.T(src, in_tys[0])
        names = {bb[i]: ins[i] for i in range(len(ins))}
        kinds = [o[1] for o in bops]
        # x + bias (rank-1 argument broadcast over all but one dimension)
        if len(ins) == 2 and kinds == ["arith.addf"] and ins[1] in self.arg and len(_shape(in_tys[1])) == 1:
            prod = self.val.get(src)
            if not prod or prod["kind"] not in ("linear", "conv") or prod.get("bias") is not None:
                self.fail(m, "a bias add that does not follow a matmul or convolution")
            prod["bias"] = self.arg[ins[1]]
            self.val[res] = prod
            self.tensor_of[res] = self.tensor_of[src]
            prod["op"]["b"] = prod["bias"]
            return
        # x / vec, x * vec (rank-1 argument broadcast over the rows)
        if len(ins) == 2 and kinds in (["arith.divf"], ["arith.mulf"]) and ins[1] in self.arg and len(_shape(in_tys[1])) == 1 and len(shape) == 2:
            first = bops[0][2][0]
            if names.get(first) != src:
                self.fail(m, "vector / x is not a per-feature scaling")
            d_t = self.T(res, res_ty)
            self.ops.ops.append(dict(op="scale", src=s_t, dst=d_t, vec=self.arg[ins[1]], rows=shape[0], n=shape[1], divide=kinds == ["arith.divf"]))
            self.val[res] = dict(kind="elementwise")
            return
        # activations
        if len(ins) == 1:
            act = alpha = None
            if kinds in (["arith.cmpf", "arith.select"],) and self._zero(bops[0][2][-1]):
                act, alpha = "relu", 0.0
            elif kinds in (["arith.maximumf"], ["arith.maxnumf"]) and any(self._zero(a) for a in bops[0][2]):
                act, alpha = "relu", 0.0
            elif kinds == ["arith.cmpf", "arith.mulf", "arith.select"]:
                c = [self.scalar(a) for a in bops[1][2] if self.scalar(a) is not None]
                if len(c) == 1 and self._zero(bops[0][2][-1]):
                    act, alpha = "leaky", float(c[0])
            if act:
                prod = self.val.get(src)
                if prod and prod["kind"] in ("linear", "conv") and prod["op"].get("act", "none") == "none":
                    prod["op"].update(act=act, alpha=alpha)
                    self.val[res] = prod
                    self.tensor_of[res] = self.tensor_of[src]
                    return
                self.fail(m, "an activation that does not follow a matmul or convolution")
        self.fail(m, "an elementwise linalg.generic this reader does not name")

    def _zero(self, v):
        c = self.scalar(v.strip())
        return c is not None and float(c) == 0.0

    def boundary(self, m, res, res_ty, ins, in_tys, bb, bops, yielded):
        src, host_esz = ins[0], None
        g = [self.arg.get(v) for v in ins[1:]]
        if any(x is None or not x.startswith("g") for x in g):
            self.fail(m, "a transposing generic whose extra operands are not the host's vectors")
        names = {bb[i]: (ins[i] if i == 0 else g[i - 1]) for i in range(len(ins))}
        kinds = [o[1] for o in bops if o[1] not in ("arith.truncf", "arith.extf")]
        in_elt, out_elt = tensor_type(in_tys[0])[1], tensor_type(res_ty)[1]
        rows_first = _shape(res_ty)
        if src in self.arg and self.arg[src] == "x":                                  # pre: host (NK, NI) -> X[NI][NK]
            NI, NK = rows_first
            host_esz = 8 if in_elt == "f64" else 4
            mean = vmax = vmin = None
            if kinds == ["arith.subf", "arith.subf", "arith.divf"]:
                a = [o for o in bops if o[1] == "arith.subf"]
                mean = names.get(a[0][2][1]); vmax = names.get(a[1][2][0]); vmin = names.get(a[1][2][1])
                if names.get(a[0][2][0]) != src or None in (mean, vmax, vmin):
                    self.fail(m, "the lifted pre expression is not (a - mean) / (max - min)")
            elif kinds:
                self.fail(m, "the lifted pre expression is not (a - mean) / (max - min)")
            s_t = self.T(src, in_tys[0], host_esz)
            d_t = self.T(res, res_ty)
            self.ops.ops.append(dict(op="boundary_pre", src=s_t, dst=d_t, NI=NI, NK=NK, mean=mean, vmax=vmax, vmin=vmin, esz=host_esz))
            self.val[res] = dict(kind="elementwise")
            return
        NK, NI = rows_first                                                             # post: Y[NI][NK] -> host (NK, NI)
        host_esz = 8 if out_elt == "f64" else 4
        scale = None
        if kinds == ["arith.divf"]:
            d = [o for o in bops if o[1] == "arith.divf"][0]
            scale = names.get(d[2][1])
            if scale is None:
                self.fail(m, "the lifted post expression is not y / scale")
        elif kinds:
            self.fail(m, "the lifted post expression is not y / scale")
        if src not in self.tensor_of:
            self.fail(m, "operand %s has no producer this reader knows" % src)
        d_t = self.T(res, res_ty, host_esz)
        self.ops.ops.append(dict(op="boundary_post", src=self.tensor_of[src], dst=d_t, NI=NI, NK=NK, scale=scale, esz=host_esz))
        self.val[res] = dict(kind="elementwise")


def read_ops(src, outline):
    """model_args.mlir text + outline.json content -> OpList (ops in program order)."""
    ops = OpList()
    n_in = len(outline["inputs"])
    entry = "mlp_kernel" if re.search(r"func\.func @mlp_kernel\(", src) else "fortis_main" if re.search(r"func\.func @fortis_main\(", src) else None
    name, args, out_ty, body = _func(src, entry)
    # argument roles: input 0 is the model's input, further inputs are host vectors g<i>, the rest weights w<i>;
    # a model called from a boundary wrapper takes its own input and then weights
    roles = {a: ("x" if i == 0 else ("g%d" % (i - 1) if i < n_in else "w%d" % (i - n_in))) for i, (a, _) in enumerate(args)}
    wroles, inner_body = {}, ""
    callee = re.search(r"call @(\w+)\(", body)
    if callee:
        inner_name, inner_args, inner_out, inner_body = _func(src, callee.group(1))
        wroles = {a: ("x" if i == 0 else "w%d" % (i - 1)) for i, (a, _) in enumerate(inner_args)}
    rd = _Reader(ops, roles)
    result = [None]

    def run(reader, text, arg_types):
        for kind, m in _statements(text):
            if kind == "generic":
                reader.generic(m)
            elif kind == "empty":
                reader.val[m.group(1)] = dict(kind="empty")
            elif kind == "const":
                tok = m.group(2)
                reader.val[m.group(1)] = dict(kind="const", value=float(tok) if not tok.startswith("0x") else float(np.array([int(tok, 16)], np.uint32).view(np.float32)[0]))
            elif kind == "fill":
                c = reader.scalar(m.group(2))
                if c is None:
                    reader.fail(m, "a fill with something other than a constant")
                reader.val[m.group(1)] = dict(kind="zero" if c == 0.0 else "filled", value=c)     # -inf starts a max pool
            elif kind == "transpose":
                w = reader.arg.get(m.group(2))
                if not w or not w.startswith("w"):
                    reader.fail(m, "a transpose of something other than a weight argument")
                reader.val[m.group(1)] = dict(kind="wT", w=w, shape=_shape(m.group(3)))
            elif kind == "matmul":
                res, a, b, a_ty, b_ty, acc, acc_ty = m.groups()
                wt = reader.val.get(b)
                if not wt or wt["kind"] != "wT":
                    reader.fail(m, "a matmul whose right operand is not a transposed weight argument")
                if reader.val.get(acc, {}).get("kind") != "zero":
                    reader.fail(m, "a matmul that accumulates into something other than a zero fill")
                B, K = _shape(a_ty)
                N = wt["shape"][0]
                op = dict(op="linear", src=reader.T(a, a_ty), dst=reader.T(res, acc_ty), w=wt["w"], b=None, B=B, K=K, N=N, act="none", alpha=0.0)
                ops.ops.append(op)
                reader.val[res] = dict(kind="linear", op=op, bias=None)
            elif kind == "pad":
                res, src_v, low, high, fillv, a_ty, b_ty = m.groups()
                lo, hi = [int(v) for v in low.split(",")], [int(v) for v in high.split(",")]
                if lo != hi or any(lo[:2]) or len(set(lo[2:])) != 1 or reader.scalar(fillv) != 0.0:
                    reader.fail(m, "a pad that is not the same zero border on every spatial side")
                reader.val[res] = dict(kind="padded", of=src_v, ty=a_ty, pad=lo[2])
            elif kind == "conv":
                res, which, stride, xin, w, x_ty, w_ty, acc, acc_ty = m.groups()
                pad, x_src, xs_ty = 0, xin, x_ty
                if reader.val.get(xin, {}).get("kind") == "padded":
                    pad, x_src, xs_ty = reader.val[xin]["pad"], reader.val[xin]["of"], reader.val[xin]["ty"]
                init = reader.val.get(acc, {})
                if init.get("kind") not in ("zero", "bias_bcast") or reader.arg.get(w, "")[:1] != "w":
                    reader.fail(m, "a convolution this reader does not name (accumulator neither zero nor a broadcast bias, or weights not an argument)")
                xs, ws = _shape(xs_ty), _shape(w_ty)
                if which.startswith("2d"):
                    op = dict(op="conv2d", src=reader.T(x_src, xs_ty), dst=reader.T(res, acc_ty), w=reader.arg[w], b=None, bn=[None] * 4, eps=1e-5,
                              C=xs[1], H=xs[2], W=xs[3], F=ws[0], KH=ws[2], KW=ws[3], stride=int(stride), pad=pad, act="none", alpha=0.0, coff=0, ctot=0)
                else:
                    if int(stride) != 1 or len(set(ws[2:])) != 1:
                        reader.fail(m, "a strided or non-cubic 3-D convolution")
                    op = dict(op="conv3d", src=reader.T(x_src, xs_ty), dst=reader.T(res, acc_ty), res=-1, w=reader.arg[w], b=None, C=xs[1], D=xs[2], H=xs[3],
                              W=xs[4], F=ws[0], K=ws[2], pad=pad, act="none", alpha=0.0)
                if init["kind"] == "bias_bcast":
                    op["b"] = init["name"]
                ops.ops.append(op)
                reader.val[res] = dict(kind="conv", op=op, bias=op["b"])
            elif kind == "maxpool":
                res, stride, xin, win, x_ty, win_ty, acc, acc_ty = m.groups()
                k = _shape(win_ty)
                xs = _shape(x_ty)
                if k != [2, 2] or int(stride) != 2 or reader.val.get(acc, {}).get("value") != float("-inf"):
                    reader.fail(m, "a max pool other than 2 x 2 stride 2 started from -inf")
                ops.ops.append(dict(op="maxpool2d", src=reader.T(xin, x_ty), dst=reader.T(res, acc_ty), C=xs[1], H=xs[2], W=xs[3], k=2))
                reader.val[res] = dict(kind="elementwise")
            elif kind == "call":
                res, callee, a, a_ty, r_ty = m.groups()
                inner = _Reader(ops, dict(wroles))
                x_arg = [k for k, v in wroles.items() if v == "x"][0]
                inner.tensor_of[x_arg] = reader.tensor_of[a]
                ret = run(inner, inner_body, None)
                reader.tensor_of[res] = inner.tensor_of[ret]
                reader.val[res] = dict(kind="elementwise")
            elif kind == "return":
                return m.group(1)
        raise MlirError("function body without a return of a tensor")

    ret = run(rd, body, None)
    x_arg = [a for a, r in roles.items() if r == "x"][0]
    if x_arg not in rd.tensor_of or ret not in rd.tensor_of:
        raise MlirError("the model's input or result never reaches an operation this reader names")
    ops.finalize(rd.tensor_of[x_arg], rd.tensor_of[ret])
    return ops


def generate(model_path, outline_path, outdir):
    ops = read_ops(open(model_path).read(), json.load(open(outline_path)))
    path = os.path.join(outdir, "ops.json")
    with open(path, "w") as f:
        json.dump(ops.as_json(), f)
    print("mlir_ops: %d operations, %d tensors -> %s" % (len(ops.ops), len(ops.tensors), path))
    return path


if __name__ == "__main__":
    if len(sys.argv) != 4:
        sys.exit(__doc__)
    generate(sys.argv[1], sys.argv[2], sys.argv[3])
