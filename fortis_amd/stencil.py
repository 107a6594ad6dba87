"""Stencil-lift descriptors -> library tables.

Takes the reference's own descriptor files as they are (mom6_zb/gather.json, scatter.json,
zb_loop_verdict.json, kdist.json; schema written by driver/fortis_gather.py:201-210) and produces
the `fortis_stencil_t` tables of include/fortis_step.h.  This is the role driver/fortis_gather_emit.py
plays in the reference, except that it fills a table instead of printing CUDA source.
"""
import ctypes as C
import json
import re

import numpy as np

from ._lib import MAX_ARRAYS, MAX_CONST, MAX_INS, MAX_REFS, MAX_SCAL, Ins, Ref, Stencil

_TOKEN = re.compile(r"\s*(tv|S\d+|sqrtf|expf|logf|tanhf|fmaxf|fminf|(?:\d+\.\d*|\.\d+|\d+)(?:[eE][-+]?\d+)?f?|[()+\-*/,])")
_UNARY = {"sqrtf": 7, "expf": 8, "logf": 9, "tanhf": 10}
_BINARY_FN = {"fmaxf": 4, "fminf": 5}
INS_F64 = 0x100
OP_NEG, OP_F32 = 6, 11


def compile_exprs(exprs, scalar_f64=None):
    """C expression strings as the reference's lifter writes them (driver/fortis_gather.py:89-121:
    tv, S<n>, literals with or without an f suffix, + - * /, unary minus, sqrtf/expf/logf/tanhf,
    fmaxf/fminf) -> ([(op, a, b)], [(value, is_double)]).

    Operand codes: 0 tv, 1+n scalar S<n>, 16+n constant n, 32+n result n.  Expressions apply in
    order, each replacing tv (driver/fortis_gather_emit.py:59-61, 79-80).  Evaluation order is the
    C parse: left-associative, * and / before + and -.  Types are C's: tv float, S<n> double where
    scalar_f64[n], a literal double without its f suffix; an arithmetic result is double when an
    operand is (INS_F64 in its op), the f-suffixed functions return float, and an expression of
    type double ends in an explicit conversion, the assignment to the float tv."""
    ins, consts, typ = [], [], {0: False}
    for n in range(MAX_SCAL):     # without a scalar list every S<n> is taken as float
        if scalar_f64 is None or n < len(scalar_f64):
            typ[1 + n] = bool(scalar_f64[n]) if scalar_f64 is not None else False

    def emit(op, a, b, f64):
        ins.append((op | (INS_F64 if f64 else 0), a, b))
        code = 32 + len(ins) - 1
        typ[code] = f64
        return code

    def const(value, f64):
        entry = (float(value) if f64 else float(np.float32(value)), f64)
        if entry in consts and not (entry[0] == 0 and np.signbit(entry[0]) != np.signbit(consts[consts.index(entry)][0])):
            code = 16 + consts.index(entry)        # a literal seen before (same value, same type) is one constant
            typ[code] = f64
            return code
        consts.append(entry)
        code = 16 + len(consts) - 1
        typ[code] = f64
        return code

    def parse_one(text, tvcode):
        toks = _TOKEN.findall(text)
        if "".join(toks) != re.sub(r"\s+", "", text):
            raise ValueError(f"unsupported token in lifted expression: {text!r}")
        pos = 0

        def peek():
            return toks[pos] if pos < len(toks) else None

        def take():
            nonlocal pos
            if pos >= len(toks):
                raise ValueError(f"unexpected end of {text!r}")
            pos += 1
            return toks[pos - 1]

        def expect(t):
            if take() != t:
                raise ValueError(f"expected {t!r} in {text!r}")

        def atom():
            t = take()
            if t == "(":
                v = additive()
                expect(")")
                return v
            if t == "tv":
                return tvcode
            if t in _UNARY:
                expect("(")
                v = additive()
                expect(")")
                return emit(_UNARY[t], v, v, False)
            if t in _BINARY_FN:
                expect("(")
                v = additive()
                expect(",")
                w = additive()
                expect(")")
                return emit(_BINARY_FN[t], v, w, False)
            if t[0] == "S":
                n = int(t[1:])
                if 1 + n not in typ:
                    raise ValueError(f"{t} is not a scalar of this descriptor ({text!r})")
                return 1 + n
            if t in "+-*/),":
                raise ValueError(f"unexpected {t!r} in {text!r}")
            return const(float(t.rstrip("f")), not t.endswith("f"))

        def unary():
            if peek() == "-":
                take()
                if peek() not in (None, "tv", "(", "-") and peek()[0] not in "Ssetf":
                    t = take()       # a negated literal is the literal of the opposite sign, exactly
                    return const(-float(t.rstrip("f")), not t.endswith("f"))
                v = unary()
                return emit(OP_NEG, v, v, typ[v])
            return atom()

        def multiplicative():
            v = unary()
            while peek() in ("*", "/"):
                op = 2 if take() == "*" else 3
                w = unary()
                v = emit(op, v, w, typ[v] or typ[w])
            return v

        def additive():
            v = multiplicative()
            while peek() in ("+", "-"):
                op = 0 if take() == "+" else 1
                w = multiplicative()
                v = emit(op, v, w, typ[v] or typ[w])
            return v

        v = additive()
        if pos != len(toks):
            raise ValueError(f"trailing tokens in {text!r}")
        if typ[v]:
            v = emit(OP_F32, v, v, False)     # tv = <double expression>;
        return v

    cur = 0
    for e in exprs:
        cur = parse_one(e, cur)
    if cur != 0 and cur < 32:
        # an expression that is a bare operand ("S0"): materialise the assignment
        cur = emit(OP_F32, cur, cur, False)
    if len(ins) > MAX_INS or len(consts) > MAX_CONST:
        raise ValueError("lifted expressions too long for the stencil table")
    return ins, consts


def _ref(arrays, entry):
    shape = arrays[entry["array"]]["shape"]
    strides = [1]
    for d in shape[:-1]:
        strides.append(strides[-1] * d)
    base = si = sj = 0
    planar = 0
    vdims = [d for d, (kind, _) in enumerate(entry["idx"]) if kind == "v"]
    if vdims and vdims != list(range(len(shape) - len(vdims), len(shape))):
        raise ValueError("plane dims must be the trailing dims")   # driver/fortis_gather_emit.py:21
    for d, (kind, off) in enumerate(entry["idx"]):
        if kind == "v":
            planar = 1
            continue
        base += (off - 1) * strides[d]
        if kind == "i":
            si += strides[d]
        elif kind == "j":
            sj += strides[d]
        else:
            raise ValueError(f"unknown index kind {kind!r}")
    return Ref(entry["array"], planar, base, si, sj)


def build_table(desc, loop, kdist=None, role="gather", cells=None, sx=None):
    """desc: parsed gather.json or scatter.json; loop: parsed loop.json; kdist: parsed kdist.json or None.
    cells: optional int32 array of 0-based active cell indices replacing the rectangle."""
    if not desc.get("ok", True):
        raise ValueError("descriptor says the lift was rejected")
    for a in desc["arrays"]:
        if a["elt"] not in ("f32", "f64"):     # driver/fortis_gather_emit.py:13
            raise ValueError(f"stencil array element type {a['elt']!r} is neither f32 nor f64")
    if len(desc["arrays"]) > MAX_ARRAYS:
        raise ValueError("too many arrays")
    t = Stencil()
    nk, klo = (kdist["nk"], kdist["loop"]["lo"]) if kdist and kdist.get("ok") else (1, 0)
    entries = desc["slots"] if role == "gather" else sorted(desc["stores"], key=lambda s: s["slot"])
    if role == "scatter" and [s["slot"] for s in entries] != list(range(desc["n"])):
        raise ValueError("scatter needs exactly one store per output slot")
    if len(entries) != desc["n"] or len(entries) > MAX_REFS or len(desc["scalars"]) > MAX_SCAL:
        raise ValueError("slot / scalar count out of range")
    t.narrays = len(desc["arrays"])
    used = {}
    for e in list(entries) + list(desc["scalars"]):
        used.setdefault(e["array"], e)
    for ai, a in enumerate(desc["arrays"]):
        total = int(np.prod(a["shape"]))
        e = used.get(ai)
        nv = sum(1 for kind, _ in e["idx"] if kind == "v") if e else 0
        plane = int(np.prod(a["shape"][:len(a["shape"]) - nv]))
        t.total[ai], t.plane[ai] = total, plane
        t.elt[ai] = 8 if a["elt"] == "f64" else 4
    t.nrefs = len(entries)
    for n, e in enumerate(entries):
        t.refs[n] = _ref(desc["arrays"], e)
    t.nscal = len(desc["scalars"])
    for n, s in enumerate(desc["scalars"]):
        if s["name"] != f"S{n}":
            raise ValueError("scalars must be named S0, S1, ... in order")
        t.scal[n] = _ref(desc["arrays"], s)
    ins, consts = compile_exprs(desc["exprs"], [desc["arrays"][s["array"]]["elt"] == "f64" for s in desc["scalars"]])
    t.nins = len(ins)
    for n, (op, a, b) in enumerate(ins):
        t.ins[n] = Ins(op, a, b)
    t.nconst = len(consts)
    for n, (c, f64) in enumerate(consts):
        t.consts[n] = c
        t.cdouble[n] = 1 if f64 else 0
        t.dconsts[n] = c
    # under loop distribution the gather loses its int args, the scatter keeps them (gather_emit.py:62, 84)
    t.nargs = 0 if (role == "gather" and nk > 1) else len(desc.get("args", []))
    t.nk, t.klo = nk, klo
    # loop.json's batch: cells per enclosing-loop iteration as the loop analysis writes it (4736 for
    # ZB), or already multiplied by nk once fortisc has accepted the distribution (driver/fortisc.sh:44;
    # the emitter divides it back, driver/fortis_gather_emit.py:12).  Both are accepted.
    batch = loop["batch"]
    count = batch
    if nk > 1:
        ni_, outer = loop["inner"]["n"], loop.get("outer")
        per_iter = ni_ * (outer["hi"] - outer["lo"] + 1) if outer and "hi" in outer else None
        if per_iter is None or batch == per_iter * nk:
            count = batch // nk
        elif batch != per_iter:
            raise ValueError(f"loop batch {batch} matches neither {per_iter} nor {per_iter}*{nk}")
    t.count = count
    t.ilo, t.ni = loop["inner"]["lo"], loop["inner"]["n"]
    if loop.get("outer"):
        t.jlo, t.nj = loop["outer"]["lo"], count // t.ni
    else:
        t.jlo, t.nj = 0, 1
    t.sx = sx if sx is not None else desc["arrays"][0]["shape"][0]
    keep = None
    if cells is not None:
        keep = np.ascontiguousarray(cells, dtype=np.int32)
        t.count = len(keep)
        t.cells = keep.ctypes.data_as(C.POINTER(C.c_int))
    t._keep = keep
    return t


def load_tables(gather_path, scatter_path, loop_path, kdist_path=None, cells=None):
    g = json.load(open(gather_path))
    s = json.load(open(scatter_path))
    lp = json.load(open(loop_path))
    kd = json.load(open(kdist_path)) if kdist_path else None
    return (build_table(g, lp, kd, "gather", cells), build_table(s, lp, kd, "scatter", cells), g, s, lp, kd)
