"""The lifter's whole expression grammar and fp64 host arrays (driver/fortis_gather.py:89-121,
driver/fortis_gather_emit.py:13, 57-61, 76-81): the oracle's evaluator against closed forms and the
pinned fp32 oracle, the product's table compiler, and which kernels a table is routed to.  CPU only."""
import copy
import ctypes as C
import json
import os

import numpy as np
import pytest

import fortis_amd
from fortis_amd import configs, stencil as S
from oracle import oracle as O


def _zb_desc(golden):
    return [json.load(open(os.path.join(golden, f"zb_{n}.json"))) for n in ("gather", "scatter", "loop", "kdist")]


def test_typed_oracle_equals_the_pinned_fp32_oracle_on_the_reference_descriptors(golden):
    gd, sd, lp, kd = _zb_desc(golden)
    F = O.zb_fields()
    Pp = O.zb_prep(F)
    garr = [Pp["sh_xy_h"], F["sh_xx"], Pp["vort_xy_h"], Pp["norm_h"]]
    X = O.stencil_gather(gd, garr, 4736, 15, 3, 3, 64)
    Xt = O.stencil_gather_typed(gd, [np.asarray(a).reshape(-1, order="F") for a in garr], 4736, 15, 3, 3, 64)
    assert np.array_equal(X.view(np.uint32), Xt.view(np.uint32))
    Y = np.random.default_rng(2).standard_normal((4736, 3)).astype(np.float32)
    base = [Pp["norm_h"].reshape(-1, order="F"), F["kappa_h"].reshape(-1, order="F"), np.zeros(68 * 78, np.float32),
            np.zeros(68 * 78 * 15, np.float32), np.zeros(68 * 78 * 15, np.float32)]
    a = [np.ascontiguousarray(x, dtype=np.float32).copy() for x in base]
    b = [x.copy() for x in a]
    for kk in (0, 7, 14):
        O.stencil_scatter(sd, a, Y, 4736, kk, 3, 3, 64)
        O.stencil_scatter_typed(sd, b, Y, 4736, kk, 3, 3, 64)
    for x, y in zip(a, b):
        assert np.array_equal(x.view(np.uint32), y.view(np.uint32))


def test_c_eval_closed_forms_and_promotion():
    tv = np.array([1e-8, -3.5, 0.0, 2.25, 7.0], np.float32)
    # fp32 throughout: 1e-8f + 1.0f rounds to 1.0f, so the difference is exactly 0
    assert np.array_equal(O.c_eval("(tv + 1.0f) - 1.0f", {"tv": tv})[:1], np.zeros(1, np.float32))
    # a double literal promotes: (double)tv + 1.0 - 1.0 keeps tv to about 2^-52, value computed by hand in binary64
    d = O.c_eval("(tv + 1.0) - 1.0", {"tv": tv})
    assert d.dtype == np.float64 and d[0] == (float(tv[0]) + 1.0) - 1.0 and d[0] != 0.0
    # a double scalar promotes the same way, a float one does not
    assert O.c_eval("tv * S0", {"tv": tv, "S0": np.full(5, 0.1, np.float64)}).dtype == np.float64
    assert O.c_eval("tv * S0", {"tv": tv, "S0": np.full(5, 0.1, np.float32)}).dtype == np.float32
    # functions take and return float; sqrtf(x*x) == |x| where x*x is exact or merely rounded once
    assert np.array_equal(O.c_eval("sqrtf(tv * tv)", {"tv": tv[1:]}), np.abs(tv[1:]))
    assert np.array_equal(O.c_eval("fmaxf(tv, 0.0f)", {"tv": tv}), np.maximum(tv, 0))
    assert np.array_equal(O.c_eval("fminf(tv, 2.0f) - (-tv)", {"tv": tv}), np.minimum(tv, np.float32(2)) + tv)
    # precedence and left association: a - b - c, a / b * c
    assert O.c_eval("tv - 1.0f - 2.0f", {"tv": tv})[3] == np.float32(-0.75)
    assert O.c_eval("tv / 2.0f * 4.0f", {"tv": tv})[4] == np.float32(14.0)


def test_c_eval_transcendentals_pinned_by_special_values_and_identities():
    """expf / logf / tanhf of the evaluator against what the mathematics fixes, not against a retyped formula:
    exact special values, published constants to two fp32 ulps, inverse and symmetry relations.  Swapping any two
    of the three names, or mapping one to another function, fails at least one line."""
    z, one = np.zeros(4, np.float32), np.ones(4, np.float32)
    ev = lambda text, tv: O.c_eval(text, {"tv": np.asarray(tv, np.float32)})
    for fn in ("expf(tv)", "logf(tv)", "tanhf(tv)"):
        assert ev(fn, one).dtype == np.float32                  # float in, float out (the f-suffixed C functions)
    assert np.array_equal(ev("expf(tv)", z), one)               # e^0 = 1
    assert np.array_equal(ev("logf(tv)", one), z)               # ln 1 = 0
    assert np.array_equal(ev("tanhf(tv)", z), z)                # tanh 0 = 0
    ulp = lambda v: np.spacing(np.float32(abs(v)))
    for text, x, want in (("expf(tv)", 1.0, 2.718281828459045), ("expf(tv)", -1.0, 0.36787944117144233),
                          ("logf(tv)", 2.0, 0.6931471805599453), ("logf(tv)", 10.0, 2.302585092994046),
                          ("tanhf(tv)", 0.5, 0.46211715726000974), ("tanhf(tv)", 1.0, 0.7615941559557649)):
        got = float(ev(text, [x])[0])
        assert abs(got - want) <= 2 * ulp(want), (text, x, got)
    x = np.linspace(-8, 8, 161).astype(np.float32)
    back = ev("logf(expf(tv))", x)                              # ln(e^x) = x
    assert np.abs(back - x).max() <= 8 * 2.0 ** -23 * 8
    t = ev("tanhf(tv)", x)
    assert np.array_equal(ev("tanhf(-tv)", x), -t)              # odd
    assert (np.abs(t) <= 1).all() and (np.diff(t) >= 0).all() and t[-1] > 0.999999
    e = ev("expf(tv)", x)
    assert (e > 0).all() and (np.diff(e) > 0).all()
    # tanh x = (e^2x - 1) / (e^2x + 1), evaluated in binary64 from the pinned exponential's argument
    ref = np.expm1(2 * x.astype(np.float64)) / (np.exp(2 * x.astype(np.float64)) + 1)
    assert np.abs(t - ref).max() <= 2.0 ** -22
    assert np.isnan(ev("logf(tv)", [-1.0])[0]) and ev("logf(tv)", [0.0])[0] == -np.inf


def test_table_compiler_types_follow_c():
    F64 = S.INS_F64
    # all fp32: no flags, no conversions; the reference's own ZB expressions
    ins, consts = S.compile_exprs(["(tv / (S0 + 1.000000e-30f))"], [False])
    assert ins == [(0, 1, 16), (3, 0, 32)] and consts == [(float(np.float32(1e-30)), False)]
    ins, _ = S.compile_exprs(["(((tv * S0) * S0) * S1)"], [False, False])
    assert ins == [(2, 0, 1), (2, 32, 1), (2, 33, 2)]
    # a double scalar: the product is double, the assignment to tv converts
    ins, _ = S.compile_exprs(["tv * S0"], [True])
    assert ins == [(2 | F64, 0, 1), (S.OP_F32, 32, 32)]
    # the conversion happens per expression: two expressions round twice
    ins, _ = S.compile_exprs(["tv * S0", "tv * S0"], [True])
    assert ins == [(2 | F64, 0, 1), (S.OP_F32, 32, 32), (2 | F64, 33, 1), (S.OP_F32, 34, 34)]
    # a double literal promotes, an f-suffixed one does not; a negated literal is a literal
    ins, consts = S.compile_exprs(["tv * -0.1", "tv * 0.1f"], [])
    assert ins == [(2 | F64, 0, 16), (S.OP_F32, 32, 32), (2, 33, 17)]
    assert consts == [(-0.1, True), (float(np.float32(0.1)), False)]
    # functions return float whatever they are given
    ins, _ = S.compile_exprs(["sqrtf(tv * S0)"], [True])
    assert ins == [(2 | F64, 0, 1), (7, 32, 32)]
    ins, _ = S.compile_exprs(["fmaxf(tv, S0) + (-S1)"], [False, True])
    assert ins == [(4, 0, 1), (6 | F64, 2, 2), (0 | F64, 32, 33), (S.OP_F32, 34, 34)]
    for bad in ("tv +", "powf(tv, 2.0f)", "tv * S3", "fmaxf(tv)", "(tv"):
        with pytest.raises(ValueError):
            S.compile_exprs([bad], [False])


def test_route_of_tables(golden):
    """Needs the library but no GPU: the check runs on the host."""
    L = fortis_amd.load()
    gd, sd, lp, kd = _zb_desc(golden)
    assert L.fortis_stencil_route(C.byref(S.build_table(gd, lp, kd, "gather"))) == 0
    assert L.fortis_stencil_route(C.byref(S.build_table(sd, lp, kd, "scatter"))) == 0

    def variant(fn):
        d = copy.deepcopy(gd)
        fn(d)
        return S.build_table(d, lp, kd, "gather")

    t = variant(lambda d: d["arrays"][3].__setitem__("elt", "f64"))
    assert t.elt[3] == 8 and L.fortis_stencil_route(C.byref(t)) == 1 and L.fortis_stencil_check(C.byref(t)) == 0
    assert L.fortis_stencil_route(C.byref(variant(lambda d: d.__setitem__("exprs", ["(tv / (S0 + 1.0e-30))"])))) == 1
    assert L.fortis_stencil_route(C.byref(variant(lambda d: d.__setitem__("exprs", ["sqrtf(tv)"])))) == 1
    assert L.fortis_stencil_route(C.byref(variant(lambda d: d.__setitem__("exprs", ["((tv * tv) + tv)"])))) == 1
    bad = S.build_table(gd, lp, kd, "gather")
    bad.ins[0].op = 12
    assert L.fortis_stencil_route(C.byref(bad)) == -1 and L.fortis_stencil_check(C.byref(bad)) == -1
    bad = S.build_table(gd, lp, kd, "gather")
    bad.elt[0] = 2
    assert L.fortis_stencil_route(C.byref(bad)) == -1


def test_emitted_table_file_compiles_for_other_arities_and_types(golden, tmp_path):
    """The C the emitter writes in place of gather.cu: entries with the generator's argument lists
    (driver/fortis_gather_emit.py:62-64, 84) for a descriptor with fp64 arrays, functions and no loop
    distribution (so the gather keeps its int argument); it must compile against the public header, and
    the tables inside must be the ones build_table makes."""
    import subprocess
    from fortis_amd import emit
    gd, sd, lp, kd = _zb_desc(golden)
    gd, sd = copy.deepcopy(gd), copy.deepcopy(sd)
    gd["arrays"][3]["elt"] = "f64"
    gd["exprs"] = ["(tv / (S0 + 1.0e-30))", "sqrtf(fmaxf(tv, 0.0f))"]
    sd["arrays"][3]["elt"] = sd["arrays"][4]["elt"] = "f64"
    path = emit.emit_stencil_tables(str(tmp_path / "tables.c"), gd, sd, lp, None)
    text = open(path).read()
    assert "void fortis_gather(int a0, const float* H0, const float* H1, const float* H2, const double* H3)" in text
    assert "void fortis_scatter(int a0, float* H0, float* H1, float* H2, double* H3, double* H4)" in text
    assert ".elt = {4, 4, 4, 8}" in text and ".cdouble = {1, 0}" in text and "0x107" not in text and "{0x103, 0, 32}" in text
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    r = subprocess.run(["gcc", "-Wall", "-Werror", "-c", "-I", inc, path, "-o", str(tmp_path / "tables.o")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_tables_that_reach_outside_their_arrays_are_refused(golden, capfd):
    """The kernels index the arrays with no bounds checks of their own, so a descriptor whose offsets or
    rectangle leave an array's plane (as a range of memory: a column offset that merely wraps into the
    neighbouring row is the lifter's business) is refused at configuration, on the host."""
    L = fortis_amd.load()
    gd, sd, lp, kd = _zb_desc(golden)

    def route(fn, role="gather", cells=None):
        g, s_, l = copy.deepcopy(gd), copy.deepcopy(sd), copy.deepcopy(lp)
        fn(g, s_, l)
        t = S.build_table(g if role == "gather" else s_, l, kd, role, cells=cells)
        return L.fortis_stencil_route(C.byref(t))

    assert route(lambda g, s_, l: None) == 0
    assert route(lambda g, s_, l: g["slots"][0]["idx"][1].__setitem__(1, -3)) == -1          # A(i-1, j-3, k) with j from 3
    assert route(lambda g, s_, l: g["slots"][26]["idx"][1].__setitem__(1, 3)) == -1          # A(..., j+3) with j up to 76 of 78
    assert route(lambda g, s_, l: l["outer"].update(lo=10, hi=83)) == -1                     # rectangle shifted past the last row
    assert route(lambda g, s_, l: s_["stores"][0]["idx"][1].__setitem__(1, 5), "scatter") == -1
    assert route(lambda g, s_, l: g["scalars"][0]["idx"][1].__setitem__(1, -3)) == -1
    ok_cells = np.array([1 + 1 * 68, 40 + 50 * 68], np.int32)
    assert route(lambda g, s_, l: None, cells=ok_cells) == 0
    assert route(lambda g, s_, l: None, cells=np.array([0], np.int32)) == -1                 # the corner has no i-1 neighbour
    assert route(lambda g, s_, l: None, cells=np.array([67 + 77 * 68], np.int32)) == -1
    assert "reaches elements" in capfd.readouterr().err
