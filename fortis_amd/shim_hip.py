#!/usr/bin/env python3
"""The FORTIS_BACKEND=hip consumer of the shim contract: what driver/fortis_shim.py does for the CUDA
build (read the `fortis.host` / `fortis.graph` attributes of the fused module and outline.json, write
shim.c), done for this backend -- it writes step_tables.c, a file of plan calls and host facts that
binds the step in libfortis_rt.so, and the link line that replaces driver/fortisc.in:61-63.

    python -m fortis_amd.shim_hip <m4.mlir> <outline.json> <outdir> [ops.json]

Same first three arguments as driver/fortis_shim.py:4.  What it reads:
  * the attribute dictionary on `func.func @mlp_kernel` in m4.mlir, in the syntax
    driver/fortis_hostattr.py:11-28 writes (parsed here with the semantics of fortis_shim.py:9-38);
  * outline.json (driver/fortis_outline.py:34): tensor types of the model's inputs, weights and output;
  * ops.json (default <outdir>/ops.json): the op groups of the fused module in program order.  In the CUDA
    build these are the kernels and fortis_gemm / fortis_conv* calls inside model.o
    (compiler/FortisFuse.cpp:575-771); no MLIR tool chain exists beside this backend, so the same list
    reaches the generator as a file.  Schema: see `OpList`.
FORTIS_GATHER / FORTIS_SCATTER in the environment are the build-time switches of fortis_shim.py:107-112.
The weights stay what they are in the CUDA build, the constant globals w0..wN of weights.o
(driver/fortis_outline.py:28-31); `write_weights_c` writes a stand-in for that object where
mlir-translate is absent.
"""
import json
import os
import re
import sys

import numpy as np

ACT = {None: 0, "none": 0, "relu": 1, "leaky": 2}
VERDICT_C = {"batched": "FORTIS_VERDICT_BATCHED", "boundary": "FORTIS_VERDICT_BOUNDARY"}


# ---- attribute dictionary ------------------------------------------------------------------------
class AttrError(ValueError):
    pass


def parse_attr(text, pos=0):
    """One value of the attribute syntax at text[pos:]: `{k = v, ...}`, `[v, ...]`, "string", true, false,
    or an integer with an optional `: iN` type.  Returns (value, position behind it)."""
    n = len(text)

    def skip(p):
        while p < n and text[p] in " \t\r\n":
            p += 1
        return p

    def value(p):
        p = skip(p)
        if p >= n:
            raise AttrError("attribute text ends inside a value")
        ch = text[p]
        if ch == "{":
            out, p = {}, skip(p + 1)
            while text[p:p + 1] != "}":
                m = re.compile(r"([\w.]+)\s*=").match(text, p)
                if not m:
                    raise AttrError("expected `key =` at %r" % text[p:p + 24])
                out[m.group(1)], p = value(m.end())
                p = skip(p)
                if text[p:p + 1] == ",":
                    p = skip(p + 1)
                elif text[p:p + 1] != "}":
                    raise AttrError("expected `,` or `}` at %r" % text[p:p + 24])
            return out, p + 1
        if ch == "[":
            out, p = [], skip(p + 1)
            while text[p:p + 1] != "]":
                v, p = value(p)
                out.append(v)
                p = skip(p)
                if text[p:p + 1] == ",":
                    p = skip(p + 1)
                elif text[p:p + 1] != "]":
                    raise AttrError("expected `,` or `]` at %r" % text[p:p + 24])
            return out, p + 1
        if ch == '"':
            e = text.find('"', p + 1)
            if e < 0:
                raise AttrError("unterminated string")
            return text[p + 1:e], e + 1
        m = re.compile(r"(true|false|-?\d+)(\s*:\s*i\d+)?").match(text, p)
        if not m:
            raise AttrError("unsupported attribute value at %r" % text[p:p + 24])
        tok = m.group(1)
        return (tok == "true") if tok in ("true", "false") else int(tok), m.end()

    return value(pos)


def func_attrs(src):
    """Attributes of `func.func @mlp_kernel(...)`; {} when the function carries none."""
    m = re.search(r"func\.func @mlp_kernel\(.*?\)\s*(?:->\s*\S+\s*)?attributes\s*", src, re.S)
    if not m:
        return {}
    return parse_attr(src, m.end())[0]


def tensor_type(t):
    m = re.fullmatch(r"tensor<((?:\d+x)+)(f32|f64)>", t)
    if not m:
        raise ValueError("unsupported tensor type %r" % t)
    return [int(d) for d in m.group(1).rstrip("x").split("x")], m.group(2)


def numel(t):
    return int(np.prod(tensor_type(t)[0]))


def esz(t):
    return 8 if tensor_type(t)[1] == "f64" else 4


def host_facts(attrs, outline, env=None):
    """The fortis_host_t fields (include/fortis_step.h) from the attributes and outline.json, with the
    decisions of driver/fortis_shim.py:94-133."""
    env = os.environ if env is None else env
    H = attrs.get("fortis.host", {})
    inputs, out_t = outline["inputs"], outline["output"]
    bnd = H.get("boundary")
    hostg = (bnd["pre"] + bnd["post"]) if bnd else H.get("lift", {}).get("globals", [])
    if len(hostg) != len(inputs) - 1:
        raise ValueError("%d extra inputs but %d host globals in fortis.host" % (len(inputs) - 1, len(hostg)))
    f = dict(n_in=numel(inputs[0]), n_out=numel(out_t), in_esz=esz(inputs[0]), out_esz=esz(out_t),
             verdict="FORTIS_VERDICT_WHOLE", expanded=0, count=0, lo=1, step=1, minc=1,
             graph=1 if attrs.get("fortis.graph", False) else 0, gather=0, scatter=0)
    v = H.get("verdict")
    if v == "batched":
        lp = H["loop"]
        f.update(verdict=VERDICT_C["batched"], count=lp["count"], lo=lp["lo"], step=lp["step"], minc=lp["minc"])
        if f["n_in"] % lp["count"] or f["n_out"] % lp["count"]:
            raise ValueError("loop count %d does not divide the model's input/output sizes" % lp["count"])
        if "expand" in H:
            f["expanded"] = 1
            f["gather"] = 1 if env.get("FORTIS_GATHER") else 0
            f["scatter"] = 1 if env.get("FORTIS_SCATTER") else 0
    elif v == "boundary":
        f["verdict"] = VERDICT_C["boundary"]
    return f, hostg


# ---- op list ---------------------------------------------------------------------------------------
class OpList:
    """The op groups of a fused module as data, and a recorder with the method names of fortis_amd.plan.Plan,
    so that the same model-building code fills either a live plan or the op-list file.

    ops.json: {"tensors": [{"elems": n, "esz": 4} | {"view_of": t, "offset": elems, "elems": n, "esz": 4}],
               "input": t, "output": t, "ops": [{"op": name, ...fields of the fortis_plan_<name> call...}]}
    Weight operands are named "w<i>" (outline.json's i-th weight), host-global vectors "g<i>" (the i-th extra
    input of the model, i.e. fortis.host's boundary pre/post or lift globals), absent ones null."""

    def __init__(self):
        self.tensors, self.ops, self.weights = [], [], []
        self.in_tensor = self.out_tensor = None

    # -- operands
    def _w(self, a):
        if a is None:
            return None
        if isinstance(a, str):                    # already a name ("g0"): a host global
            return a
        self.weights.append(np.ascontiguousarray(a, dtype=np.float32))
        return "w%d" % (len(self.weights) - 1)

    # -- the Plan interface
    def tensor(self, nelem, esz=4):
        self.tensors.append(dict(elems=int(nelem), esz=esz))
        return len(self.tensors) - 1

    def view(self, base, elem_offset, nelem, esz=4):
        self.tensors.append(dict(view_of=base, offset=int(elem_offset), elems=int(nelem), esz=esz))
        return len(self.tensors) - 1

    def linear(self, src, dst, W, bias, B, act=None, alpha=0.0):
        N, K = np.asarray(W).shape
        self.ops.append(dict(op="linear", src=src, dst=dst, w=self._w(W), b=self._w(bias), B=int(B), K=int(K), N=int(N), act=act or "none", alpha=float(alpha)))

    def scale(self, src, dst, vec, rows, divide):
        n = int(np.asarray(vec).size) if not isinstance(vec, str) else None
        self.ops.append(dict(op="scale", src=src, dst=dst, vec=self._w(vec), rows=int(rows), n=n, divide=bool(divide)))

    def mask_relu(self, src, dst, rows, n, tail):
        self.ops.append(dict(op="mask_relu", src=src, dst=dst, rows=int(rows), n=int(n), tail=int(tail)))

    def boundary_pre(self, src, dst, NI, NK, mean=None, vmax=None, vmin=None, host_dtype=np.float32):
        self.ops.append(dict(op="boundary_pre", src=src, dst=dst, NI=int(NI), NK=int(NK), mean=mean, vmax=vmax, vmin=vmin,
                             esz=np.dtype(host_dtype).itemsize))

    def boundary_post(self, src, dst, NI, NK, scale=None, host_dtype=np.float32):
        self.ops.append(dict(op="boundary_post", src=src, dst=dst, NI=int(NI), NK=int(NK), scale=scale, esz=np.dtype(host_dtype).itemsize))

    def conv2d(self, src, dst, W, bias, C_, H, Wd, stride=1, pad=0, act=None, alpha=0.0, bn=None, bn_eps=1e-5, coff=0, ctot=0):
        F, _, KH, KW = np.asarray(W).shape
        g = be = m = v = None
        if bn is not None:
            g, be, m, v = [self._w(t) for t in bn]
        self.ops.append(dict(op="conv2d", src=src, dst=dst, w=self._w(W), b=self._w(bias), bn=[g, be, m, v], eps=float(bn_eps), C=int(C_), H=int(H),
                             W=int(Wd), F=int(F), KH=int(KH), KW=int(KW), stride=int(stride), pad=int(pad), act=act or "none",
                             alpha=float(alpha), coff=int(coff), ctot=int(ctot)))

    def convt2d(self, src, dst, W, bias, C_, H, Wd, stride, pad=0, output_padding=0, act=None, alpha=0.0, coff=0, ctot=0):
        _, F, KH, KW = np.asarray(W).shape
        self.ops.append(dict(op="convt2d", src=src, dst=dst, w=self._w(W), b=self._w(bias), C=int(C_), H=int(H), W=int(Wd), F=int(F), KH=int(KH),
                             KW=int(KW), stride=int(stride), pad=int(pad), opad=int(output_padding), act=act or "none",
                             alpha=float(alpha), coff=int(coff), ctot=int(ctot)))

    def maxpool2d(self, src, dst, C_, H, Wd, k=2):
        self.ops.append(dict(op="maxpool2d", src=src, dst=dst, C=int(C_), H=int(H), W=int(Wd), k=int(k)))

    def upsample(self, src, dst, C_, D, H, Wd, s=2, nd=2):
        self.ops.append(dict(op="upsample", src=src, dst=dst, C=int(C_), D=int(D), H=int(H), W=int(Wd), s=int(s), nd=int(nd)))

    def concat_copy(self, src, dst, C_, S, coff, ctot):
        self.ops.append(dict(op="concat_copy", src=src, dst=dst, C=int(C_), S=int(S), coff=int(coff), ctot=int(ctot)))

    def conv3d(self, src, dst, W, bias, C_, D, H, Wd, pad=0, act=None, alpha=0.0, res=-1):
        F, _, K, _, _ = np.asarray(W).shape
        self.ops.append(dict(op="conv3d", src=src, dst=dst, res=int(res), w=self._w(W), b=self._w(bias), C=int(C_), D=int(D), H=int(H), W=int(Wd),
                             F=int(F), K=int(K), pad=int(pad), act=act or "none", alpha=float(alpha)))

    def permute(self, src, dst, C_, S, to_channels_first):
        self.ops.append(dict(op="permute", src=src, dst=dst, C=int(C_), S=int(S), to_channels_first=bool(to_channels_first)))

    def finalize(self, in_tensor, out_tensor):
        self.in_tensor, self.out_tensor = in_tensor, out_tensor
        return self

    # -- files
    def as_json(self):
        return dict(tensors=self.tensors, input=self.in_tensor, output=self.out_tensor, ops=self.ops)

    def outline(self, in_type, out_type, extra_inputs=()):
        """outline.json content for this model (driver/fortis_outline.py:34)."""
        return dict(inputs=[in_type] + list(extra_inputs),
                    weights=["tensor<%sxf32>" % "x".join(str(d) for d in w.shape) for w in self.weights], output=out_type)


def write_weights_c(outdir, arrays):
    """Stand-in for weights.o (driver/fortis_outline.py:28-31; fortisc.in:50-51): w<i>.bin files and a C file that
    pulls them into 64-byte aligned constant globals w0..wN with .incbin.  Returns the C path."""
    lines = ["/* stand-in for weights.o: the model's weight constants as the globals w0..wN */"]
    for i, a in enumerate(arrays):
        path = os.path.abspath(os.path.join(outdir, "w%d.bin" % i))
        np.ascontiguousarray(a, dtype=np.float32).tofile(path)
        lines.append('__asm__(".section .rodata\\n .balign 64\\n .globl w%d\\n w%d:\\n .incbin \\"%s\\"\\n .previous\\n");' % (i, i, path))
    cpath = os.path.join(outdir, "weights.c")
    with open(cpath, "w") as f:
        f.write("\n".join(lines) + "\n")
    return cpath


# ---- emission --------------------------------------------------------------------------------------
def _operand(name, nweights, hostg, what):
    """C expression of a weight / host-global operand."""
    if name is None:
        return "0"
    m = re.fullmatch(r"([wg])(\d+)", name)
    if not m:
        raise ValueError("%s: operand %r is neither w<i>, g<i> nor null" % (what, name))
    i = int(m.group(2))
    if m.group(1) == "w":
        if i >= nweights:
            raise ValueError("%s: %s but outline.json lists %d weights" % (what, name, nweights))
        return "w%d" % i
    if i >= len(hostg):
        raise ValueError("%s: %s but fortis.host names %d host globals" % (what, name, len(hostg)))
    return hostg[i]


def emit_step(attrs, outline, ops, env=None):
    """-> text of step_tables.c."""
    facts, hostg = host_facts(attrs, outline, env)
    nw = len(outline["weights"])
    T = ops["tensors"]
    if not T or not ops["ops"]:
        raise ValueError("ops.json: empty model")
    for name in ("input", "output"):
        if not isinstance(ops.get(name), int) or not 0 <= ops[name] < len(T):
            raise ValueError("ops.json: bad %s tensor" % name)
    if T[ops["input"]]["elems"] * T[ops["input"]].get("esz", 4) < facts["n_in"] * facts["in_esz"] or \
       T[ops["output"]]["elems"] * T[ops["output"]].get("esz", 4) < facts["n_out"] * facts["out_esz"]:
        raise ValueError("ops.json: the model's input/output tensors are smaller than outline.json's types")
    L = ["/* generated by fortis_amd/shim_hip.py (FORTIS_BACKEND=hip): plan of the fused module + host facts */",
         "#include <stdio.h>", "#include <stdlib.h>", '#include "fortis_step.h"']
    if nw:
        L.append("extern float " + ", ".join("w%d[]" % i for i in range(nw)) + ";")
    for g, ty in zip(hostg, outline["inputs"][1:]):
        L.append("extern %s %s[];" % ("double" if esz(ty) == 8 else "float", g))
    L += ['#define OK(call) do { if ((call) < 0) { fprintf(stderr, "fortis step: %s failed\\n", #call); exit(1); } } while (0)',
          "/* runs at the first use of an entry point, like setup() in the CUDA shim: host globals hold their",
          "   run-time values by then */",
          "static void fortis_bind_step(void)", "{", "    fortis_plan* p = fortis_plan_create();", "    int t[%d];" % len(T)]
    for i, t in enumerate(T):
        es = t.get("esz", 4)
        if "view_of" in t:
            if not 0 <= t["view_of"] < i:
                raise ValueError("ops.json: tensor %d is a window of a later tensor" % i)
            L.append("    OK(t[%d] = fortis_plan_view(p, t[%d], %dL * %d, %dL * %d));" % (i, t["view_of"], t["offset"], es, t["elems"], es))
        else:
            L.append("    OK(t[%d] = fortis_plan_tensor(p, %dL * %d));" % (i, t["elems"], es))

    def tid(o, key):
        v = o[key]
        if not isinstance(v, int) or not -1 <= v < len(T) or (v < 0 and key != "res"):
            raise ValueError("ops.json: op %r names tensor %r" % (o["op"], v))
        return "t[%d]" % v if v >= 0 else "-1"

    def act(o):
        if o.get("act", "none") not in ACT:
            raise ValueError("ops.json: unknown activation %r" % o["act"])
        return "%d, %sf" % (ACT[o.get("act", "none")], repr(float(o.get("alpha", 0.0))))

    for n, o in enumerate(ops["ops"]):
        k = o["op"]
        W = lambda key: _operand(o.get(key), nw, hostg, "op %d (%s)" % (n, k))
        s, d = tid(o, "src"), tid(o, "dst")
        if k == "linear":
            c = "fortis_plan_linear(p, %s, %s, %s, %s, %dL, %d, %d, %s)" % (s, d, W("w"), W("b"), o["B"], o["K"], o["N"], act(o))
        elif k == "scale":
            nvec = o.get("n")
            if nvec is None:
                raise ValueError("ops.json: scale needs its vector length n")
            c = "fortis_plan_scale(p, %s, %s, %s, %dL, %d, %d)" % (s, d, W("vec"), o["rows"], nvec, 1 if o["divide"] else 0)
        elif k == "mask_relu":
            c = "fortis_plan_mask_relu(p, %s, %s, %dL, %d, %d)" % (s, d, o["rows"], o["n"], o["tail"])
        elif k == "boundary_pre":
            c = "fortis_plan_boundary_pre(p, %s, %s, %dL, %d, %s, %s, %s, %d)" % (s, d, o["NI"], o["NK"], W("mean"), W("vmax"), W("vmin"), o["esz"])
        elif k == "boundary_post":
            c = "fortis_plan_boundary_post(p, %s, %s, %dL, %d, %s, %d)" % (s, d, o["NI"], o["NK"], W("scale"), o["esz"])
        elif k == "conv2d":
            bn = o.get("bn") or [None] * 4
            bnc = ", ".join(_operand(b, nw, hostg, "op %d (conv2d bn)" % n) for b in bn)
            c = "fortis_plan_conv2d(p, %s, %s, %s, %s, %s, %sf, %d, %d, %d, %d, %d, %d, %d, %d, %s, %d, %d)" % (
                s, d, W("w"), W("b"), bnc, repr(float(o.get("eps", 1e-5))), o["C"], o["H"], o["W"], o["F"], o["KH"], o["KW"],
                o["stride"], o["pad"], act(o), o.get("coff", 0), o.get("ctot", 0))
        elif k == "convt2d":
            c = "fortis_plan_convt2d(p, %s, %s, %s, %s, %d, %d, %d, %d, %d, %d, %d, %d, %d, %s, %d, %d)" % (
                s, d, W("w"), W("b"), o["C"], o["H"], o["W"], o["F"], o["KH"], o["KW"], o["stride"], o["pad"], o.get("opad", 0), act(o),
                o.get("coff", 0), o.get("ctot", 0))
        elif k == "maxpool2d":
            c = "fortis_plan_maxpool2d(p, %s, %s, %d, %d, %d, %d)" % (s, d, o["C"], o["H"], o["W"], o["k"])
        elif k == "upsample":
            c = "fortis_plan_upsample(p, %s, %s, %d, %d, %d, %d, %d, %d)" % (s, d, o["C"], o["D"], o["H"], o["W"], o["s"], o["nd"])
        elif k == "concat_copy":
            c = "fortis_plan_concat_copy(p, %s, %s, %d, %dL, %d, %d)" % (s, d, o["C"], o["S"], o["coff"], o["ctot"])
        elif k == "conv3d":
            c = "fortis_plan_conv3d(p, %s, %s, %s, %s, %s, %d, %d, %d, %d, %d, %d, %d, %s)" % (
                s, d, tid(o, "res") if "res" in o else "-1", W("w"), W("b"), o["C"], o["D"], o["H"], o["W"], o["F"], o["K"], o["pad"], act(o))
        elif k == "permute":
            c = "fortis_plan_permute(p, %s, %s, %d, %dL, %d)" % (s, d, o["C"], o["S"], 1 if o["to_channels_first"] else 0)
        else:
            raise ValueError("ops.json: unknown op %r" % k)
        L.append("    OK(%s);" % c)
    L.append("    OK(fortis_plan_finalize(p, t[%d], t[%d]));" % (ops["input"], ops["output"]))
    L.append("    fortis_host_t host = { .n_in = %(n_in)dL, .n_out = %(n_out)dL, .in_esz = %(in_esz)d, .out_esz = %(out_esz)d, .verdict = %(verdict)s,\n"
             "                           .expanded = %(expanded)d, .count = %(count)dL, .lo = %(lo)dL, .step = %(step)dL, .minc = %(minc)dL,\n"
             "                           .graph = %(graph)d, .gather = %(gather)d, .scatter = %(scatter)d };" % facts)
    L += ["    OK(fortis_step_bind(p, &host));", "}",
          "__attribute__((constructor)) static void fortis_register_step(void) { fortis_step_on_first_use(fortis_bind_step); }"]
    return "\n".join(L) + "\n", facts


def link_line(prefix="$PREFIX", rocm="/opt/rocm"):
    """What replaces the link of driver/fortisc.in:61-63: no model.o / shim.o / vendor libraries."""
    return ("$B/flang -O3 $HOSTOBJ $W/step_tables.o $W/weights.o -L%s/lib -lfortis_rt -Wl,-rpath,%s/lib "
            "-L%s/lib -lamdhip64 -Wl,-rpath,%s/lib -o $OUT" % (prefix, prefix, rocm, rocm))


def generate(m4_path, outline_path, outdir, ops_path=None, env=None):
    attrs = func_attrs(open(m4_path).read())
    outline = json.load(open(outline_path))
    ops = json.load(open(ops_path or os.path.join(outdir, "ops.json")))
    text, facts = emit_step(attrs, outline, ops, env)
    path = os.path.join(outdir, "step_tables.c")
    with open(path, "w") as f:
        f.write(text)
    with open(os.path.join(outdir, "link_hip.txt"), "w") as f:
        f.write(link_line() + "\n")
    H = attrs.get("fortis.host", {})
    print("shim[hip]: verdict=%s batch=%s repeat=%s graph=%d in=%s out=%s ops=%d" % (
        H.get("verdict"), H.get("batch"), H.get("repeat"), facts["graph"], outline["inputs"][0], outline["output"], len(ops["ops"])))
    return path


if __name__ == "__main__":
    if len(sys.argv) < 4:
        sys.exit(__doc__)
    generate(sys.argv[1], sys.argv[2], sys.argv[3], sys.argv[4] if len(sys.argv) > 4 else None)
