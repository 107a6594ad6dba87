"""Per-build generated files of a FORTIS_BACKEND=hip build, written from Python arguments: the module-side
inputs of fortis_amd/shim_hip.py (m4.mlir's attribute line, outline.json, ops.json, a weights.o stand-in) for
models given as numpy arrays, and the C file that replaces the generated gather.cu
(driver/fortis_gather_emit.py).  The step file itself always comes out of shim_hip.generate, the one
generator: nothing here writes plan calls."""
import json
import os

import numpy as np

from . import shim_hip


def host_attr(verdict="whole", shape=(1,), batch=1, repeat=0, graph=False, loop=None, expand=None, lift=None, boundary=None):
    """The attribute dictionary driver/fortis_hostattr.py:11-28 attaches to the model entry, as MLIR text.
    loop: dict(lo, step, count, minc, in, out, post_download); expand: dict(in, out, count, nin, nout);
    lift: dict(globals=[...], in=...); boundary: dict(in, in_elt, out, out_elt, pre=[...], post=[...])."""
    q = lambda v: '"%s"' % v
    i64 = lambda v: "%d : i64" % int(v)
    parts = ["version = 1 : i64", "shape = [%s]" % ", ".join(str(x) for x in shape), "batch = " + i64(batch),
             "repeat = " + i64(repeat), "verdict = " + q(verdict),
             'provenance = {shape = "proven", repeat = "proven", dependence = "proven", lift = "proven", layout = "proven", '
             'scope = "proven", aliasing = "checked", purity = "checked", fp_order = "assumed"}']
    if loop:
        parts.append("loop = {lo = %s, step = %s, count = %s, minc = %s, in = %s, out = %s, post_download = %s}" % (
            i64(loop["lo"]), i64(loop["step"]), i64(loop["count"]), i64(loop["minc"]), q(loop.get("in", "x")), q(loop.get("out", "y")),
            "true" if loop.get("post_download") else "false"))
    if expand:
        parts.append("expand = {in = %s, out = %s, count = %s, nin = %s, nout = %s}" % (
            q(expand.get("in", "x")), q(expand.get("out", "y")), i64(expand["count"]), i64(expand["nin"]), i64(expand["nout"])))
    if lift:
        parts.append("lift = {globals = [%s], in = %s}" % (", ".join(q(g) for g in lift["globals"]), q(lift.get("in", "x"))))
    if boundary:
        parts.append("boundary = {in = %s, in_elt = %s, out = %s, out_elt = %s, pre = [%s], post = [%s]}" % (
            q(boundary["in"]), q(boundary["in_elt"]), q(boundary["out"]), q(boundary["out_elt"]),
            ", ".join(q(g) for g in boundary["pre"]), ", ".join(q(g) for g in boundary["post"])))
    attrs = "fortis.host = {" + ", ".join(parts) + "}"
    if graph:
        attrs += ", fortis.graph = true"
    return attrs


def module_stub(attr_text, outline):
    """The one line of m4.mlir the shim generators read: the signature of @mlp_kernel with its attributes."""
    args = ", ".join("%%arg%d: %s" % (i, t) for i, t in enumerate(outline["inputs"] + outline["weights"] + [outline["output"]]))
    return "module {\n  func.func @mlp_kernel(%s) attributes {%s} {\n    return\n  }\n}\n" % (args, attr_text)


def step_files(outdir, oplist, attr_text, in_type, out_type, extra_inputs=(), env=None):
    """Writes, under outdir, what a FORTIS_BACKEND=hip build holds for one model: m4.mlir (attribute line only),
    outline.json, ops.json, then runs the generator (-> step_tables.c, link_hip.txt) and writes the weights
    stand-in (weights.c + w<i>.bin).  Returns [step_tables.c, weights.c]."""
    os.makedirs(outdir, exist_ok=True)
    outline = oplist.outline(in_type, out_type, extra_inputs)
    with open(os.path.join(outdir, "m4.mlir"), "w") as f:
        f.write(module_stub(attr_text, outline))
    json.dump(outline, open(os.path.join(outdir, "outline.json"), "w"))
    json.dump(oplist.as_json(), open(os.path.join(outdir, "ops.json"), "w"))
    c = shim_hip.generate(os.path.join(outdir, "m4.mlir"), os.path.join(outdir, "outline.json"), outdir, env=env)
    return [c, shim_hip.write_weights_c(outdir, oplist.weights)]


def emit_mlp_step(outdir, Ws, bs, acts, rows, alphas=None, in_norms=None, out_norms=None, verdict="whole",
                  graph=False, expanded=False, count=0, lo=1, step=1, minc=1, gather=False, scatter=False):
    """Step files for a Linear(+activation) stack over `rows` rows with optional input division / output
    multiplication vectors (mom6_zb/export_zb.py:10-16)."""
    from . import plan as P
    ol = P.mlp_plan(Ws, bs, acts, rows, alphas=alphas, in_norms=in_norms, out_norms=out_norms, plan_cls=shim_hip.OpList)
    nin, nout = int(Ws[0].shape[1]), int(Ws[-1].shape[0])
    kw = {}
    if verdict == "batched":
        kw["loop"] = dict(lo=lo, step=step, count=count, minc=minc)
        if expanded:
            kw["expand"] = dict(count=count, nin=rows * nin // count, nout=rows * nout // count)
    env = dict(FORTIS_GATHER="1" if gather else "", FORTIS_SCATTER="1" if scatter else "")
    attr = host_attr(verdict, shape=(nin,), batch=count or rows, graph=graph, **kw)
    return step_files(outdir, ol, attr, "tensor<%dx%dxf32>" % (rows, nin), "tensor<%dx%dxf32>" % (rows, nout), env=env)


def emit_conv3d_step(outdir, W, b, shape, pad=1, act=None, alpha=0.0, graph=False):
    """Step files for one conv3d (+ activation) on an NCDHW tensor of `shape` = (C, D, H, W), stride 1
    (frontend/export_conv.py:4)."""
    C_, D, H, Wd = (int(v) for v in shape)
    F, K = int(W.shape[0]), int(W.shape[2])
    Do, Ho, Wo = D + 2 * pad - K + 1, H + 2 * pad - K + 1, Wd + 2 * pad - K + 1
    ol = shim_hip.OpList()
    t0, t1 = ol.tensor(C_ * D * H * Wd), ol.tensor(F * Do * Ho * Wo)
    ol.conv3d(t0, t1, W, b, C_, D, H, Wd, pad, act, alpha)
    ol.finalize(t0, t1)
    attr = host_attr("whole", shape=(1, C_, D, H, Wd), graph=graph)
    return step_files(outdir, ol, attr, "tensor<1x%dx%dx%dx%dxf32>" % (C_, D, H, Wd), "tensor<1x%dx%dx%dx%dxf32>" % (F, Do, Ho, Wo))


def _table_c(name, t):
    """One fortis_stencil_t (the ctypes mirror filled by stencil.build_table) as a C initialiser."""
    def ref(r):
        return "{%d, %d, %dL, %dL, %dL}" % (r.array, r.planar, r.base, r.si, r.sj)

    def arr(vals, fmt="%d"):
        return "{" + ", ".join(fmt % v for v in vals) + "}"

    na = t.narrays
    f = [".narrays = %d" % na, ".total = " + arr([t.total[a] for a in range(na)], "%dL"),
         ".plane = " + arr([t.plane[a] for a in range(na)], "%dL"), ".nrefs = %d" % t.nrefs,
         ".refs = {" + ", ".join(ref(t.refs[r]) for r in range(t.nrefs)) + "}", ".nscal = %d" % t.nscal]
    if t.nscal:
        f.append(".scal = {" + ", ".join(ref(t.scal[r]) for r in range(t.nscal)) + "}")
    f.append(".nins = %d" % t.nins)
    if t.nins:
        f.append(".ins = {" + ", ".join("{0x%x, %d, %d}" % (t.ins[n].op, t.ins[n].a, t.ins[n].b) for n in range(t.nins)) + "}")
    f.append(".nconst = %d" % t.nconst)
    if t.nconst:
        # hexadecimal floating literals: the table holds the exact bits the builder computed
        f.append(".consts = " + "{" + ", ".join(float(t.consts[n]).hex() + "f" for n in range(t.nconst)) + "}")
        f.append(".cdouble = " + arr([t.cdouble[n] for n in range(t.nconst)]))
        f.append(".dconsts = " + "{" + ", ".join(float(t.dconsts[n]).hex() for n in range(t.nconst)) + "}")
    f += [".count = %dL" % t.count, ".nk = %d" % t.nk, ".klo = %d" % t.klo, ".nargs = %d" % t.nargs, ".ilo = %d" % t.ilo,
          ".jlo = %d" % t.jlo, ".ni = %d" % t.ni, ".nj = %d" % t.nj, ".sx = %d" % t.sx, ".cells = 0",
          ".elt = " + arr([t.elt[a] for a in range(na)])]
    return "static const fortis_stencil_t %s = {\n    %s };" % (name, ",\n    ".join(f))


def emit_stencil_tables(path, gather_desc, scatter_desc, loop, kdist=None):
    """Writes the C file that takes the place of the generated gather.cu (driver/fortis_gather_emit.py):
    the two tables, their configuration at load time, and the entries `fortis_gather` / `fortis_scatter`
    with the argument lists the generator gives them (gather: the enclosing-loop ints unless the loop is
    distributed, then one pointer per array, :62-64; scatter: the ints, then the pointers, :84)."""
    from . import stencil as S

    cty = {"f32": "float", "f64": "double"}
    kd_ok = bool(kdist and kdist.get("ok"))
    # the header declares the two entries with the ZB instance's argument lists; this file defines them for
    # the descriptor at hand, so the header's declarations are renamed out of the way
    L = ["/* generated by fortis_amd/emit.py: stencil tables of the lifted gather / scatter */",
         '#define fortis_gather fortis_gather_zb_form\n#define fortis_scatter fortis_scatter_zb_form\n#include "fortis_step.h"\n'
         '#undef fortis_gather\n#undef fortis_scatter']
    inits, entries = [], []
    for role, desc, tname, cfg in (("gather", gather_desc, "fortis_G", "fortis_gather_config"),
                                   ("scatter", scatter_desc, "fortis_S", "fortis_scatter_config")):
        if not desc or not desc.get("ok", True):
            continue
        t = S.build_table(desc, loop, kdist, role)
        L.append(_table_c(tname, t))
        inits.append("    if (%s(&%s) != 0) { fprintf(stderr, \"fortis: %s table rejected\\n\"); exit(1); }" % (cfg, tname, role))
        nint = 0 if (role == "gather" and kd_ok) else len(desc.get("args", []))
        const = "const " if role == "gather" else ""
        params = ["int a%d" % i for i in range(nint)] + ["%s%s* H%d" % (const, cty[a["elt"]], i) for i, a in enumerate(desc["arrays"])]
        body = "    %svoid* H[%d] = { %s };\n" % (const, len(desc["arrays"]), ", ".join("H%d" % i for i in range(len(desc["arrays"]))))
        if nint:
            body += "    int a[%d] = { %s };\n    fortis_%s_v(a, H);" % (nint, ", ".join("a%d" % i for i in range(nint)), role)
        else:
            body += "    fortis_%s_v(0, H);" % role
        entries.append("void fortis_%s(%s)\n{\n%s\n}" % (role, ", ".join(params), body))
    L.insert(2, "#include <stdio.h>\n#include <stdlib.h>")
    L.append("__attribute__((constructor)) static void fortis_config_tables(void)\n{\n" + "\n".join(inits) + "\n}")
    L += entries
    with open(path, "w") as f:
        f.write("\n".join(L) + "\n")
    return path
