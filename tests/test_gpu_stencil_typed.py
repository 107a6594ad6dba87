"""The general stencil kernels on the GPU through the C ABI: fp64 host arrays, double literals, the
lifter's functions and expressions that are not one chain on the slot value
(driver/fortis_gather.py:89-121, driver/fortis_gather_emit.py:13, 57-61, 76-81), against the oracle's
typed evaluator.  Bit-exact except expf/logf/tanhf (device and CUDA libm are not correctly rounded:
1e-6 relative)."""
import copy
import ctypes as C

import numpy as np
import pytest

from fortis_amd import configs, plan as P, stencil as S, step as ST
from oracle import oracle as O
from util import DevBuf, bits_equal, maxrel, ptrs

pytestmark = pytest.mark.gpu

SX, SY, NZ = 37, 29, 4
COUNT = (SX - 4) * (SY - 4)


@pytest.fixture(autouse=True)
def _fresh_step(L):
    yield
    ST.reset()


def _case(gexprs=None, sexprs=None, g64=(), s64=()):
    gd, sd, lp, kd = configs.zb_descriptors(SX, SY, NZ)
    gd, sd = copy.deepcopy(gd), copy.deepcopy(sd)
    if gexprs is not None:
        gd["exprs"] = gexprs
    if sexprs is not None:
        sd["exprs"] = sexprs
    for a in g64:
        gd["arrays"][a]["elt"] = "f64"
    for a in s64:
        sd["arrays"][a]["elt"] = "f64"
    A = configs.zb_arrays(SX, SY, NZ)
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    # fp64 arrays carry bits below fp32 precision, so that a premature rounding to float shows
    rng = np.random.default_rng(11)
    garr = [a.astype(np.float64) * (1 + 1e-9 * rng.standard_normal(a.size)) if i in g64 else a for i, a in enumerate(garr)]
    sarr = [A["norm_h"], A["kappa_h"], np.zeros(SX * SY, np.float32), np.zeros(SX * SY * NZ, np.float32), np.zeros(SX * SY * NZ, np.float32)]
    sarr = [a.astype(np.float64) * (1 + 1e-9 * rng.standard_normal(a.size)) if i in s64 else a for i, a in enumerate(sarr)]
    return gd, sd, lp, kd, garr, sarr


def _gather(L, gd, lp, kd, garr):
    gt = S.build_table(gd, lp, kd, "gather")
    assert L.fortis_stencil_route(C.byref(gt)) == 1
    bufs = [DevBuf(L, a) for a in garr]
    n = len(gd["slots"])
    dX = DevBuf(L, nbytes=COUNT * NZ * n * 4)
    L.fortis_stencil_gather_dev(C.byref(gt), ptrs(bufs), dX.ptr)
    X = dX.get((COUNT * NZ, n))
    for b in bufs + [dX]:
        b.free()
    return X


@pytest.mark.parametrize("exprs,g64", [
    (["(tv / (S0 + 1.000000e-30f))"], (3,)),                    # fp64 scalar array: the division is done in double
    (["(tv / (S0 + 1.0e-30))"], ()),                             # double literal on fp32 arrays
    (["(tv * S0)", "(tv * S0)"], (0, 3)),                        # fp64 slot array, rounded to float per expression
    (["((tv * tv) + tv)"], ()),                                  # not a chain on the slot value
    (["(sqrtf(fmaxf(tv, 0.0f)) * S0)", "(fminf(tv, 2.0f) - (-S0))"], ()),
    (["((-tv) / -3.0f)"], (1,)),
    # the slot value as the right operand of a step, in float and in double
    (["(S0 / tv)", "(2.0 - tv)"], (3,)),
    # one fp64 step feeding another: the running value cannot be cut to a float between them
    (["((tv * S0) * S0)"], (3,)),
    # a per-cell subexpression beside the chain on the slot value
    (["(sqrtf(fmaxf(tv, 0.0f)) / ((S0 * S0) + 1.0f))"], ()),
    (["((tv - S0) / ((S0 * S0) + 1.0f))"], (3,)),
    # more steps than the chain form holds
    (["(((((((((tv + 1.0f) * 2.0f) - 3.0f) * 0.5f) + S0) * S0) - 1.0f) * 2.0f) + 0.25f)"], ()),
])
def test_general_gather_bit_exact(L, gpu, exprs, g64):
    gd, sd, lp, kd, garr, _ = _case(gexprs=exprs, g64=g64)
    X = _gather(L, gd, lp, kd, garr)
    ref = O.stencil_gather_typed(gd, garr, COUNT, NZ, 3, 3, SX - 4)
    assert bits_equal(X, ref)
    # a case with an fp64 scalar exercises what it is meant to: evaluating it all in fp32 gives another answer
    if 3 in g64:
        gd32 = copy.deepcopy(gd)
        for a in gd32["arrays"]:
            a["elt"] = "f32"
        ref32 = O.stencil_gather_typed(gd32, [np.asarray(a, np.float32) for a in garr], COUNT, NZ, 3, 3, SX - 4)
        assert not bits_equal(ref32, ref)


def test_fp64_division_with_operands_at_the_ends_of_the_range(L, gpu):
    """tv / S0 with S0 an fp64 array: the general gather divides a row's slot values by one double.  Numerators of
    either zero, infinities, NaNs, denormals and the largest floats, and divisors that are zero, infinite, NaN,
    denormal or beyond 2^+-400, sprinkled over otherwise ordinary data, must give the bits of an IEEE double
    division rounded to float, whichever way a row's division is carried out."""
    gd, sd, lp, kd, garr, _ = _case(gexprs=["(tv / S0)"], g64=(3,))
    rng = np.random.default_rng(23)
    xs = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1e-39, 3.4028235e38, -3.4028235e38, 1.1754944e-38], np.float32)
    cs = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 5e-324, 1e-310, 1e-200, -1e-200, 1e200, -1e200, 1.7e308,
                   2.0 ** -400, 2.0 ** 400, 2.0 ** -401, 2.0 ** 401, -3.0, 1e-30, 1e30], np.float64)
    for a in garr[:3]:
        at = rng.random(a.size) < 0.02
        a[at] = rng.choice(xs, at.sum())
        pz = rng.random(a.size) < 0.05                          # +0 alone is common (masked cells) and stays on the short form
        a[pz] = 0.0
    at = rng.random(garr[3].size) < 0.15
    garr[3][at] = rng.choice(cs, at.sum())
    with np.errstate(all="ignore"):
        ref = O.stencil_gather_typed(gd, garr, COUNT, NZ, 3, 3, SX - 4)
    X = _gather(L, gd, lp, kd, garr)
    same = (X.view(np.uint32) == ref.view(np.uint32)) | (np.isnan(X) & np.isnan(ref))
    assert same.all()
    fin = np.isfinite(ref)
    assert 0.3 < fin.mean() < 0.99 and (ref == 0).sum() > 100 and np.signbit(ref[ref == 0]).any()


@pytest.mark.parametrize("g64", [(), (1, 3)])
def test_wide_stencil_and_long_expression(L, gpu, g64):
    """A 5 x 5 neighbourhood of three arrays (75 slots) with a 21-operation expression: more slots than one
    launch of the kernels holds (they go 32 at a time, the last launch 11) and more operations than the fused
    form chains; an fp32 chain-form table of 75 slots takes the general kernels too.  Gather bit-exact; the
    scatter of 40 outputs per cell onto five arrays' worth of stores likewise."""
    gd, sd, lp, kd, garr, sarr = _case(g64=g64)
    gd["slots"] = [dict(array=a, idx=[["i", di], ["j", dj], ["v", 0]]) for a in range(3) for dj in (-2, -1, 0, 1, 2) for di in (-2, -1, 0, 1, 2)]
    gd["n"] = 75
    gt = S.build_table(gd, lp, kd, "gather")
    assert gt.nrefs == 75 and L.fortis_stencil_route(C.byref(gt)) == 1       # chain form, but wider than the fused kernels
    X = _gather(L, gd, lp, kd, garr)
    assert bits_equal(X, O.stencil_gather_typed(gd, garr, COUNT, NZ, 3, 3, SX - 4))
    gd["exprs"] = ["((((((((((tv + 1.0f) * 2.0f) - 3.0f) * 0.5f) + S0) * S0) - 1.0f) * 2.0f) + 0.25f) / (S0 + 2.0f))",
                   "(((((((((tv * 0.5f) + 0.125f) * S0) - tv) + ((S0 * S0) + 1.0f)) * 0.75f) - 2.0f) + (tv * tv)) * 1.5f)"]
    assert S.build_table(gd, lp, kd, "gather").nins >= 21
    X = _gather(L, gd, lp, kd, garr)
    assert bits_equal(X, O.stencil_gather_typed(gd, garr, COUNT, NZ, 3, 3, SX - 4))
    # scatter: 40 outputs per cell, store q to array 2 + q % 3 of the ZB scatter descriptor at (i + q / 3 - 6, j)
    sd = copy.deepcopy(sd)
    sd["n"] = 40
    sd["stores"] = [dict(slot=q, array=2 + q % 3, idx=([["i", q // 3 - 6], ["j", 0]] if q % 3 == 0 else [["i", q // 3 - 6], ["j", 0], ["v", 0]])) for q in range(40)]
    # a cell list 16 apart along i, so that no two cells' 14 shifted stores into one array meet
    cells = np.array([(i - 1) + (j - 1) * SX for j in range(3, SY - 1) for i in (9, 25)], np.int32)
    cnt = len(cells)
    st = S.build_table(sd, lp, kd, "scatter", cells=cells)
    assert st.nrefs == 40 and L.fortis_stencil_route(C.byref(st)) == 1
    Y = np.random.default_rng(5).standard_normal((cnt * NZ, 40)).astype(np.float32)
    ref = [a.copy() for a in sarr]
    sb = [DevBuf(L, a) for a in sarr]
    dY = DevBuf(L, Y)
    for kk in range(NZ):
        L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY.ptr + kk * cnt * 40 * 4), kk)
        O.stencil_scatter_typed(sd, ref, Y[kk * cnt:(kk + 1) * cnt], cnt, kk, cells=cells)
    for b, r in zip(sb[2:], ref[2:]):
        got = b.get(r.shape, r.dtype)
        assert np.array_equal(got.view(np.uint8), r.view(np.uint8)) and np.abs(r).max() > 0
    for b in sb + [dY]:
        b.free()


def test_general_gather_libm_functions(L, gpu):
    gd, sd, lp, kd, garr, _ = _case(gexprs=["(tanhf(tv) + expf((tv * 0.5f)))", "logf((tv + 3.0f))"])
    X = _gather(L, gd, lp, kd, garr)
    ref = O.stencil_gather_typed(gd, garr, COUNT, NZ, 3, 3, SX - 4)
    ok = np.isfinite(ref)
    assert ok.mean() > 0.9 and np.array_equal(np.isfinite(X), ok)
    assert np.abs(X[ok] - ref[ok]).max() <= 1e-6 * np.abs(ref[ok]).max()


@pytest.mark.parametrize("exprs,s64", [
    (["(((tv * S0) * S0) * S1)"], (0, 3)),                      # fp64 scalar and fp64 written array
    (["(((tv * S0) * S0) * S1)"], (2, 3, 4)),                   # every written array fp64
    (["(sqrtf((tv * tv)) * 0.25)", "(tv + S1)"], (1,)),
])
def test_general_scatter_bit_exact(L, gpu, exprs, s64):
    gd, sd, lp, kd, _, sarr = _case(sexprs=exprs, s64=s64)
    st = S.build_table(sd, lp, kd, "scatter")
    assert L.fortis_stencil_route(C.byref(st)) == 1
    Y = np.random.default_rng(4).standard_normal((COUNT * NZ, 3)).astype(np.float32)
    ref = [a.copy() for a in sarr]
    sb = [DevBuf(L, a) for a in sarr]
    dY = DevBuf(L, Y)
    for kk in range(NZ):
        L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY.ptr + kk * COUNT * 3 * 4), kk)
        O.stencil_scatter_typed(sd, ref, Y[kk * COUNT:(kk + 1) * COUNT], COUNT, kk, 3, 3, SX - 4)
    for b, r in zip(sb[2:], ref[2:]):
        got = b.get(r.shape, r.dtype)
        assert np.array_equal(got.view(np.uint8), r.view(np.uint8)) and np.abs(r).max() > 0
    for b in sb + [dY]:
        b.free()


def test_host_entries_with_fp64_arrays(L, gpu):
    """fortis_gather(...) -> mlp_forward_batched() -> do k: fortis_scatter(k, ...) on a host whose norm, kappa
    and stress arrays are double precision: uploads, staging planes and the copy-back use 8-byte elements."""
    gd, sd, lp, kd, garr, sarr = _case(g64=(3,), s64=(0, 1, 3, 4))
    sarr[0] = garr[3]                                              # one norm array on the host
    gt, st = S.build_table(gd, lp, kd, "gather"), S.build_table(sd, lp, kd, "scatter")
    net = configs.zb_mlp((20,))
    rows = COUNT * NZ
    plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows)
    ST.bind(plan, rows * 27, rows * 3, verdict="batched", expanded=True, count=rows, gather=True, scatter=True)
    ST.gather_config(gt)
    ST.scatter_config(st)
    ST.fortis_gather_v([], garr)
    ST.mlp_forward_batched()
    X = np.empty((rows, 27), np.float32)
    Y = np.empty((rows, 3), np.float32)
    L.fortis_d2h(X.ctypes.data, L.fortis_model_input(), X.nbytes)
    assert bits_equal(X, O.stencil_gather_typed(gd, garr, COUNT, NZ, 3, 3, SX - 4))
    host = [a.copy() for a in sarr]
    for k in range(1, NZ + 1):
        ST.fortis_scatter_v([k], host)
    L.fortis_d2h(Y.ctypes.data, L.fortis_model_output(), Y.nbytes)
    assert maxrel(Y, O.mlp_f64(net["Ws"], net["bs"], net["acts"], X)) < 1e-5
    ref = [a.copy() for a in sarr]
    txy_last = None
    for kk in range(NZ):
        O.stencil_scatter_typed(sd, ref, Y[kk * COUNT:(kk + 1) * COUNT], COUNT, kk, 3, 3, SX - 4)
    for got, r in zip(host, ref):
        assert got.dtype == r.dtype and np.array_equal(got.view(np.uint8), r.view(np.uint8))
    assert host[3].dtype == np.float64 and np.abs(host[3]).max() > 0
    # the fused single-kernel step declines such tables instead of reading doubles as floats
    assert L.fortis_stencil_step_fused(C.byref(gt), C.byref(st), plan.handle, None, None, None) == -1
