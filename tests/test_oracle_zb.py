"""Pins the CPU oracle's ZB functions against data the reference itself holds or produced:
the fixture written from the reference's own Fortran host + native forward, the known-answer
vector in zb_nn.npz, and the closed-form index expressions of the checked-in gather kernel."""
import json
import os

import numpy as np
import pytest

from oracle import oracle as O
from util import bits_equal, maxrel


@pytest.fixture(scope="module")
def zb(golden):
    W = np.load(os.path.join(golden, "zb_nn.npz"))
    G = np.load(os.path.join(golden, "zb_native_golden.npz"))
    F = O.zb_fields()
    P = O.zb_prep(F)
    Ws, bs = [W["A0"], W["A1"]], [W["b0"], W["b1"]]
    T = O.zb_step_native(F, P, Ws, bs, W["in_norms"], W["out_norms"])
    return dict(W=W, G=G, F=F, P=P, Ws=Ws, bs=bs, T=T)


def test_known_answer_vector_native(zb):
    # mom6_zb/make_zb_weights.py:18-20 checks this pair to ~6e-8
    W = zb["W"]
    y = O.mlp_native(zb["Ws"], zb["bs"], W["x_test"][None], W["in_norms"], W["out_norms"])
    assert maxrel(y[0], W["y_test"]) < 2e-7


def test_known_answer_vector_f64(zb):
    W = zb["W"]
    y = O.mlp_f64(zb["Ws"], zb["bs"], ["relu", "none"], W["x_test"][None], in_norms=W["in_norms"], out_norms=W["out_norms"])
    assert maxrel(y[0], W["y_test"]) < 2e-7


def test_native_step_equals_reference_build_bitwise(zb):
    """Whole ZB step (field synthesis, interpolation, norm, stencil packing, ANN, de-scaling, corner
    interpolation) against the flang build of mom6_zb/zb_host.f90 + fwd_native_zb.f90."""
    G, T = zb["G"], zb["T"]
    for n, key in enumerate(("Txx", "Tyy", "Txy")):
        a = T[key].reshape(15, 78, 68)
        assert bits_equal(a[G["layers"] - 1], G[key]), key
        assert a.astype(np.float64).sum() == G["checksum"][n], key


def test_gather_scatter_route_equals_native_step(zb, golden):
    """gather -> per-row native MLP -> scatter through the table-driven oracle functions reproduces the
    cell-by-cell host loop bit for bit (RESHAPE order, expression order)."""
    gd = json.load(open(os.path.join(golden, "zb_gather.json")))
    sd = json.load(open(os.path.join(golden, "zb_scatter.json")))
    F, P, W, T = zb["F"], zb["P"], zb["W"], zb["T"]
    X = O.stencil_gather(gd, [P["sh_xy_h"], F["sh_xx"], P["vort_xy_h"], P["norm_h"]], 4736, 15, 3, 3, 64)
    Y = O.mlp_native(zb["Ws"], zb["bs"], X, W["in_norms"], W["out_norms"])
    Txy_h = np.zeros(68 * 78, np.float32)
    Txx = np.zeros(68 * 78 * 15, np.float32)
    Tyy = np.zeros_like(Txx)
    arrs = [P["norm_h"], F["kappa_h"], Txy_h, Txx, Tyy]
    for kk in range(15):
        O.stencil_scatter(sd, arrs, Y[kk * 4736:(kk + 1) * 4736], 4736, kk, 3, 3, 64)
    assert bits_equal(Txx, T["Txx"]) and bits_equal(Tyy, T["Tyy"]) and bits_equal(Txy_h, T["Txy_h"])


def test_gather_closed_form_indices(zb, golden):
    """X[row][q] = A_f[(i+di-1) + (j+dj-1)*68 + kk*5304] / (norm + 1e-30f), q = f*9 + (dj+1)*3 + (di+1),
    row = kk*4736 + col, i = 3 + col%64, j = 3 + col/64 (mom6_zb/gather.cu:15-48)."""
    gd = json.load(open(os.path.join(golden, "zb_gather.json")))
    F, P = zb["F"], zb["P"]
    A = [P["sh_xy_h"], F["sh_xx"], P["vort_xy_h"]]
    X = O.stencil_gather(gd, A + [P["norm_h"]], 4736, 15, 3, 3, 64)
    rng = np.random.default_rng(7)
    for row in rng.integers(0, 71040, 200):
        col, kk = row % 4736, row // 4736
        i, j = 3 + col % 64, 3 + col // 64
        S0 = P["norm_h"][(i - 1) + (j - 1) * 68 + kk * 5304]
        for f in range(3):
            for dj in (-1, 0, 1):
                for di in (-1, 0, 1):
                    q = f * 9 + (dj + 1) * 3 + (di + 1)
                    tv = A[f][(i + di - 1) + (j + dj - 1) * 68 + kk * 5304]
                    assert X[row, q] == np.float32(tv) / (np.float32(S0) + np.float32(1e-30))


def test_cell_list_equals_rectangle(zb, golden):
    gd = json.load(open(os.path.join(golden, "zb_gather.json")))
    F, P = zb["F"], zb["P"]
    arrs = [P["sh_xy_h"], F["sh_xx"], P["vort_xy_h"], P["norm_h"]]
    col = np.arange(4736)
    cells = ((3 + col % 64) - 1) + ((3 + col // 64) - 1) * 68
    Xr = O.stencil_gather(gd, arrs, 4736, 2, 3, 3, 64)
    Xl = O.stencil_gather(gd, arrs, 4736, 2, cells=cells)
    assert bits_equal(Xr, Xl)


def test_expression_compiler_order():
    ins, n, consts = O.compile_exprs(["(((tv * S0) * S0) * S1)"])
    assert n == 3 and [(ins[k].op, ins[k].a, ins[k].b) for k in range(3)] == [(2, 0, 1), (2, 32, 1), (2, 33, 2)]
    ins, n, consts = O.compile_exprs(["(tv / (S0 + 1.000000e-30f))"])
    assert n == 2 and (ins[0].op, ins[0].a, ins[0].b) == (0, 1, 16) and (ins[1].op, ins[1].a, ins[1].b) == (3, 0, 32)
    assert consts[0] == np.float32(1e-30)


def test_native_t_is_the_same_arithmetic(zb):
    """The Fortran-ordered-weights variant timed as the CPU baseline equals the pinned native
    forward bit for bit on the ZB network, and the fp64 chain within rounding on a LeakyReLU net."""
    W = zb["W"]
    X = O.stencil_gather(__import__("json").load(open(os.path.join(os.path.dirname(__file__), "golden", "zb_gather.json"))),
                         [zb["P"]["sh_xy_h"], zb["F"]["sh_xx"], zb["P"]["vort_xy_h"], zb["P"]["norm_h"]], 4736, 1, 3, 3, 64)
    a = O.mlp_native(zb["Ws"], zb["bs"], X, W["in_norms"], W["out_norms"])
    b = O.mlp_native_t(zb["Ws"], zb["bs"], ["relu", None], X, in_norms=W["in_norms"], out_norms=W["out_norms"])
    assert bits_equal(a, b)
    rng = np.random.default_rng(1)
    Ws = [rng.standard_normal((40, 30)).astype(np.float32) / 5, rng.standard_normal((10, 40)).astype(np.float32) / 6]
    bs = [rng.standard_normal(40).astype(np.float32), rng.standard_normal(10).astype(np.float32)]
    Xs = rng.standard_normal((100, 30)).astype(np.float32)
    assert maxrel(O.mlp_native_t(Ws, bs, ["leaky", None], Xs, alphas=[0.15, 0]),
                  O.mlp_f64(Ws, bs, ["leaky", None], Xs, alphas=[0.15, 0])) < 2e-6
