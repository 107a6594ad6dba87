"""Stencil gather / scatter and the fused gather->MLP->scatter step on the GPU, through the C ABI,
against the CPU oracle.  Index maps and expression arithmetic: bit-exact.  Model outputs: 1e-5."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from fortis_amd import configs, plan as P, stencil as S
from oracle import oracle as O
from util import TOL, DevBuf, bits_equal, maxrel, ptrs

pytestmark = pytest.mark.gpu


def golden_tables(golden, cells=None):
    return S.load_tables(*[os.path.join(golden, f"zb_{n}.json") for n in ("gather", "scatter", "loop", "kdist")], cells=cells)


@pytest.fixture(scope="module")
def zbhost(golden):
    W = np.load(os.path.join(golden, "zb_nn.npz"))
    F = O.zb_fields()
    Pp = O.zb_prep(F)
    return dict(W=W, F=F, P=Pp, Ws=[W["A0"], W["A1"]], bs=[W["b0"], W["b1"]],
                garr=[Pp["sh_xy_h"], F["sh_xx"], Pp["vort_xy_h"], Pp["norm_h"]])


def test_gather_reference_geometry_bit_exact(L, gpu, golden, zbhost):
    gt, st, gd, sd, lp, kd = golden_tables(golden)
    bufs = [DevBuf(L, a) for a in zbhost["garr"]]
    dX = DevBuf(L, nbytes=71040 * 27 * 4)
    L.fortis_stencil_gather_dev(C.byref(gt), ptrs(bufs), dX.ptr)
    X = dX.get((71040, 27))
    ref = O.stencil_gather(gd, zbhost["garr"], 4736, 15, 3, 3, 64)
    assert bits_equal(X, ref)
    for b in bufs + [dX]:
        b.free()


@pytest.mark.parametrize("sx,sy,nz", [(48, 58, 10), (9, 7, 1), (133, 70, 3), (520, 40, 2), (1031, 25, 3), (1540, 17, 1)])
def test_gather_scatter_other_grids_bit_exact(L, gpu, sx, sy, nz):
    """48x58x10 -> 44x54 = 2376 cells per layer is the reference's second specialisation size
    (mom6_zb/README.md:37); the next two are ragged (count not a multiple of the block) and tiny; the wide ones
    have rows of about 2, 4 and 6 workgroups, whose gather walks its workgroups in vertical strips."""
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    gt, st = S.build_table(gd, lp, kd, "gather"), S.build_table(sd, lp, kd, "scatter")
    A = configs.zb_arrays(sx, sy, nz)
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    count = (sx - 4) * (sy - 4)
    bufs = [DevBuf(L, a) for a in garr]
    dX = DevBuf(L, nbytes=count * nz * 27 * 4)
    L.fortis_stencil_gather_dev(C.byref(gt), ptrs(bufs), dX.ptr)
    X = dX.get((count * nz, 27))
    assert bits_equal(X, O.stencil_gather(gd, garr, count, nz, 3, 3, sx - 4))
    # scatter of a random Y, one enclosing-loop iteration at a time, onto full-depth device arrays
    Y = np.random.default_rng(4).standard_normal((count * nz, 3)).astype(np.float32)
    host = [A["norm_h"], A["kappa_h"], np.zeros(sx * sy, np.float32), np.zeros(sx * sy * nz, np.float32), np.zeros(sx * sy * nz, np.float32)]
    ref = [a.copy() for a in host]
    sb = [DevBuf(L, a) for a in host]
    dY = DevBuf(L, Y)
    for kk in range(nz):
        L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY.ptr + kk * count * 3 * 4), kk)
        O.stencil_scatter(sd, ref, Y[kk * count:(kk + 1) * count], count, kk, 3, 3, sx - 4)
    for b, r in zip(sb[2:], ref[2:]):
        assert bits_equal(b.get(r.shape), r)
    # every iteration in one launch: the 2-D array gets a plane per iteration, whose last one is what the
    # iteration-by-iteration launches leave in it
    host[2] = np.zeros(sx * sy * nz, np.float32)
    sa = [DevBuf(L, a) for a in host]
    assert L.fortis_stencil_scatter_all_dev(C.byref(st), ptrs(sa), dY.ptr) == 0
    assert bits_equal(sa[3].get(ref[3].shape), ref[3]) and bits_equal(sa[4].get(ref[4].shape), ref[4])
    assert bits_equal(sa[2].get((nz, sx * sy))[nz - 1], ref[2])
    for b in bufs + sb + sa + [dX, dY]:
        b.free()


@pytest.mark.parametrize("n", [1, 2, 4])
def test_scatter_all_iterations_other_output_counts(L, gpu, n):
    """The scatter over all enclosing-loop iterations in one launch walks the iterations inside the kernel for tables
    of at most four outputs per cell: the ZB scatter table cut down to one and two stores and grown to four, seven
    iterations (one full group of five and a tail), against the oracle and against one launch per iteration."""
    import copy
    sx, sy, nz = 70, 37, 7
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    sd, lp = copy.deepcopy(sd), copy.deepcopy(lp)
    sd["n"], lp["out_shape"] = n, [n]
    if n < 3:
        sd["stores"] = [dict(s, slot=s["slot"] - (3 - n)) for s in sd["stores"] if s["slot"] >= 3 - n]
    else:
        sd["arrays"].append({"name": "tzz", "shape": [sx, sy, nz], "elt": "f32"})
        sd["stores"].append({"slot": 3, "array": 5, "idx": [["i", 0], ["j", 0], ["v", 0]]})
    st = S.build_table(sd, lp, kd, "scatter")
    A = configs.zb_arrays(sx, sy, nz)
    count = (sx - 4) * (sy - 4)
    Y = np.random.default_rng(6).standard_normal((count * nz, n)).astype(np.float32)
    host = [A["norm_h"], A["kappa_h"], np.zeros(sx * sy * nz, np.float32)] + [np.zeros(sx * sy * nz, np.float32) for _ in range(len(sd["arrays"]) - 3)]
    # the oracle an iteration at a time; the 2-D array (slot 0 of the full table) gets a plane per iteration on the device
    ref = [a.copy() for a in host]
    flat2d = [A["norm_h"], A["kappa_h"], np.zeros(sx * sy, np.float32)] + [r for r in ref[3:]]
    planes = np.zeros((nz, sx * sy), np.float32)
    for kk in range(nz):
        O.stencil_scatter(sd, flat2d, Y[kk * count:(kk + 1) * count], count, kk, 3, 3, sx - 4)
        planes[kk] = flat2d[2]
    written = sorted({s["array"] for s in sd["stores"]})
    one, per = [DevBuf(L, a) for a in host], [DevBuf(L, a) for a in host]
    dY = DevBuf(L, Y)
    assert L.fortis_stencil_scatter_all_dev(C.byref(st), ptrs(one), dY.ptr) == 0
    for a in written:
        want = planes.reshape(-1) if a == 2 else flat2d[a]
        assert bits_equal(one[a].get(want.shape), want), (n, a)
    for kk in range(nz):
        L.fortis_stencil_scatter_dev(C.byref(st), ptrs(per), C.c_void_p(dY.ptr + kk * count * n * 4), kk)
    for a in written:
        if a != 2:
            assert bits_equal(per[a].get(flat2d[a].shape), flat2d[a]), (n, a)
    for b in one + per + [dY]:
        b.free()


def test_gather_scatter_expressions_on_special_operands(L, gpu):
    """tv / (S0 + 1e-30f) in the gather and ((tv * S0) * S0) * S1 in the scatter with zeros of both signs, denormals, the
    smallest and largest normals, powers of two near the ends of the exponent range, all-ones mantissas, infinities and
    NaNs among numerators, divisors and factors: IEEE results bit for bit (any NaN equals any NaN), in the fp32 kernels
    and, with the arrays in double precision, in the general ones."""
    sx, sy, nz = 40, 30, 2
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    rng = np.random.default_rng(21)
    tiny, big = np.float32(1.1754944e-38), np.float32(3.4028235e38)
    ones = np.array([0x3FFFFFFF, 0x007FFFFF, 0x7F7FFFFF, 0x00000001, 0x80000001, 0x00800000], np.uint32).view(np.float32)
    special = np.concatenate([np.array([0.0, -0.0, 1e-45, -1e-45, 3e-39, tiny, -tiny, 2.0 ** -100, 2.0 ** -64, 2.0 ** -24, 1.0, -1.0, 3.0,
                                        2.0 ** 64, 2.0 ** 100, 2.0 ** 126, big, -big, np.inf, -np.inf, np.nan], np.float32), ones])

    def field(n, share):
        a = rng.standard_normal(n).astype(np.float32)
        pick = rng.random(n) < share
        a[pick] = rng.choice(special, int(pick.sum()))
        return a
    n3 = sx * sy * nz
    A = {"sh_xy_h": field(n3, 0.3), "sh_xx": field(n3, 0.3), "vort_xy_h": field(n3, 0.3), "norm_h": field(n3, 0.3), "kappa_h": field(sx * sy, 0.3)}
    count = (sx - 4) * (sy - 4)

    def same(a, b):
        a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
        return bool(np.all((a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))))
    with np.errstate(all="ignore"):
        for f64 in (False, True):
            gdd, sdd = [{**d, "arrays": [dict(a) for a in d["arrays"]]} for d in (gd, sd)]
            ft = np.float64 if f64 else np.float32
            if f64:
                for d in (gdd, sdd):
                    for a in d["arrays"]:
                        a["elt"] = "f64"
            gt, st = S.build_table(gdd, lp, kd, "gather"), S.build_table(sdd, lp, kd, "scatter")
            garr = [A[k].astype(ft) for k in ("sh_xy_h", "sh_xx", "vort_xy_h", "norm_h")]
            bufs = [DevBuf(L, a) for a in garr]
            dX = DevBuf(L, nbytes=count * nz * 27 * 4)
            L.fortis_stencil_gather_dev(C.byref(gt), ptrs(bufs), dX.ptr)
            X = dX.get((count * nz, 27))
            ref = O.stencil_gather_typed(gdd, garr, count, nz, 3, 3, sx - 4) if f64 else O.stencil_gather(gd, garr, count, nz, 3, 3, sx - 4)
            assert same(X, ref), "gather, f64 arrays: %s" % f64
            if not f64:
                Y = field(count * nz * 3, 0.3).reshape(count * nz, 3)
                host = [A["norm_h"], A["kappa_h"], np.zeros(sx * sy, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
                refs = [a.copy() for a in host]
                sb = [DevBuf(L, a) for a in host]
                dY = DevBuf(L, Y)
                for kk in range(nz):
                    L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY.ptr + kk * count * 3 * 4), kk)
                    O.stencil_scatter(sd, refs, Y[kk * count:(kk + 1) * count], count, kk, 3, 3, sx - 4)
                for b, r in zip(sb[2:], refs[2:]):
                    assert same(b.get(r.shape), r)
                for b in sb + [dY]:
                    b.free()
            for b in bufs + [dX]:
                b.free()


@pytest.mark.parametrize("ncells", [4736, 2376])
def test_gather_scatter_masked_cell_list_bit_exact(L, gpu, ncells):
    """480 x 240 grid with a 1-cell halo and a seeded ~30 % land mask; the first 4736 (2376) usable
    ocean cells form the active list."""
    sx, sy, nz = 482, 242, 2
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    A = configs.zb_arrays(sx, sy, nz, mask_land=0.3)
    cells = configs.zb_cells_from_mask(A["mask"], sx, sy, ncells)
    gt, st = S.build_table(gd, lp, kd, "gather", cells), S.build_table(sd, lp, kd, "scatter", cells)
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    bufs = [DevBuf(L, a) for a in garr]
    dX = DevBuf(L, nbytes=ncells * nz * 27 * 4)
    L.fortis_stencil_gather_dev(C.byref(gt), ptrs(bufs), dX.ptr)
    X = dX.get((ncells * nz, 27))
    assert bits_equal(X, O.stencil_gather(gd, garr, ncells, nz, cells=cells))
    Y = np.random.default_rng(4).standard_normal((ncells * nz, 3)).astype(np.float32)
    host = [A["norm_h"], A["kappa_h"], np.zeros(sx * sy, np.float32), np.zeros(sx * sy * nz, np.float32), np.zeros(sx * sy * nz, np.float32)]
    ref = [a.copy() for a in host]
    sb = [DevBuf(L, a) for a in host]
    dY = DevBuf(L, Y)
    for kk in range(nz):
        L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY.ptr + kk * ncells * 3 * 4), kk)
        O.stencil_scatter(sd, ref, Y[kk * ncells:(kk + 1) * ncells], ncells, kk, cells=cells)
    for b, r in zip(sb[2:], ref[2:]):
        assert bits_equal(b.get(r.shape), r)
    # every iteration in one launch: the 2-D array gets a plane per iteration, whose last one is what the
    # iteration-by-iteration launches leave in it
    host[2] = np.zeros(sx * sy * nz, np.float32)
    sa = [DevBuf(L, a) for a in host]
    assert L.fortis_stencil_scatter_all_dev(C.byref(st), ptrs(sa), dY.ptr) == 0
    assert bits_equal(sa[3].get(ref[3].shape), ref[3]) and bits_equal(sa[4].get(ref[4].shape), ref[4])
    assert bits_equal(sa[2].get((nz, sx * sy))[nz - 1], ref[2])
    for b in bufs + sb + sa + [dX, dY]:
        b.free()


def _fused(L, gt, st, plan, garr, sarr_host, rows, nout=3):
    gb = [DevBuf(L, a) for a in garr]
    sb = [DevBuf(L, a) for a in sarr_host]
    dY = DevBuf(L, nbytes=rows * nout * 4)
    rc = L.fortis_stencil_step_fused(C.byref(gt), C.byref(st), plan.handle, ptrs(gb), ptrs(sb), dY.ptr)
    assert rc == 0
    L.fortis_sync()
    out = [b.get(a.shape) for b, a in zip(sb, sarr_host)]
    Y = dY.get((rows, nout))
    for b in gb + sb + [dY]:
        b.free()
    return out, Y


def test_fused_step_reference_network_vs_native_host(L, gpu, golden, zbhost):
    """One kernel for gather -> 27-20-3 ANN -> scatter over all 15 layers, against the cell-by-cell
    host loop (which the oracle tests tie bit-for-bit to the reference's own Fortran build)."""
    gt, st, gd, sd, lp, kd = golden_tables(golden)
    W = zbhost["W"]
    plan = P.mlp_plan(zbhost["Ws"], zbhost["bs"], ["relu", None], 71040, in_norms=W["in_norms"], out_norms=W["out_norms"])
    assert plan.num_kernels == 1
    F, Pp = zbhost["F"], zbhost["P"]
    n3 = 68 * 78 * 15
    host = [Pp["norm_h"], F["kappa_h"], np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    out, Y = _fused(L, gt, st, plan, zbhost["garr"], host, 71040)
    T = O.zb_step_native(F, Pp, zbhost["Ws"], zbhost["bs"], W["in_norms"], W["out_norms"])
    assert maxrel(out[3], T["Txx"]) < TOL and maxrel(out[4], T["Tyy"]) < TOL
    assert maxrel(out[2].reshape(15, -1)[14], T["Txy_h"]) < TOL       # the host's 2-D Txy_h holds the last layer
    # golden fixture layers written by the reference build
    G = np.load(os.path.join(golden, "zb_native_golden.npz"))
    assert maxrel(out[3].reshape(15, 78, 68)[G["layers"] - 1], G["Txx"]) < TOL
    # the scatter applied to the kernel's own raw outputs is bit-exact
    ref = [a.copy() for a in host[:2]] + [np.zeros(68 * 78, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    for kk in range(15):
        O.stencil_scatter(sd, ref, Y[kk * 4736:(kk + 1) * 4736], 4736, kk, 3, 3, 64)
    assert bits_equal(out[3], ref[3]) and bits_equal(out[4], ref[4])
    plan.close()


@pytest.mark.parametrize("hidden", [(64, 64), (20,), (128, 32, 8)])
def test_fused_step_config2_network(L, gpu, golden, hidden):
    """Config 2's 27->64->64->3 network (and two other shapes) on the reference geometry, against the
    fp64-accumulated chain run on the oracle's gathered rows."""
    gt, st, gd, sd, lp, kd = golden_tables(golden)
    A = configs.zb_arrays(68, 78, 15)
    net = configs.zb_mlp(hidden)
    plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], 71040)
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    n3 = 68 * 78 * 15
    host = [A["norm_h"], A["kappa_h"], np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    out, Y = _fused(L, gt, st, plan, garr, host, 71040)
    X = O.stencil_gather(gd, garr, 4736, 15, 3, 3, 64)
    Yref = O.mlp_f64(net["Ws"], net["bs"], net["acts"], X)
    assert maxrel(Y, Yref) < TOL
    ref = [a.copy() for a in host[:2]] + [np.zeros(68 * 78, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    for kk in range(15):
        O.stencil_scatter(sd, ref, Yref[kk * 4736:(kk + 1) * 4736], 4736, kk, 3, 3, 64)
    assert maxrel(out[3], ref[3]) < TOL and maxrel(out[4], ref[4]) < TOL
    plan.close()


@pytest.mark.parametrize("ncells", [4736, 2376])
@pytest.mark.parametrize("lists", ["shared", "copies", "permuted"])
def test_fused_step_masked_cell_list_config2(L, gpu, ncells, lists):
    """Config 2 as BASELINE states it: 480 x 240 grid, 1-cell halo, seeded ~30 % land mask, the first 4736
    (2376) ocean cells as the active list, 27 -> 64 -> 64 -> 3 between the gather and the scatter, all in the
    one-launch kernel.  `shared`: both tables name one list object; `copies`: equal lists at two addresses (the
    library still keeps one device copy and decodes a row once); `permuted`: the scatter visits the cells in
    reverse order, so the kernel decodes gather and scatter cells separately."""
    sx, sy, nz = 482, 242, 3
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    A = configs.zb_arrays(sx, sy, nz, mask_land=0.3)
    cells = configs.zb_cells_from_mask(A["mask"], sx, sy, ncells)
    scells = cells if lists == "shared" else cells.copy() if lists == "copies" else np.ascontiguousarray(cells[::-1])
    gt, st = S.build_table(gd, lp, kd, "gather", cells), S.build_table(sd, lp, kd, "scatter", scells)
    net = configs.zb_mlp()
    rows = ncells * nz
    plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows)
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    n2, n3 = sx * sy, sx * sy * nz
    host = [A["norm_h"], A["kappa_h"], np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    out, Y = _fused(L, gt, st, plan, garr, host, rows)
    X = O.stencil_gather(gd, garr, ncells, nz, cells=cells)
    assert maxrel(Y, O.mlp_f64(net["Ws"], net["bs"], net["acts"], X)) < TOL
    # the scatter of the kernel's own Y, and the unfused route (gather kernel -> X -> MLP -> Y -> scatter per layer)
    ref = [a.copy() for a in host[:2]] + [np.zeros(n2, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    txy = np.zeros((nz, n2), np.float32)
    for kk in range(nz):
        O.stencil_scatter(sd, ref, Y[kk * ncells:(kk + 1) * ncells], ncells, kk, cells=scells)
        txy[kk] = ref[2]
        ref[2][:] = 0
    assert bits_equal(out[3], ref[3]) and bits_equal(out[4], ref[4]) and bits_equal(out[2].reshape(nz, n2), txy)
    assert np.abs(ref[3]).max() > 0
    gb, sb = [DevBuf(L, a) for a in garr], [DevBuf(L, a) for a in host]
    dX, dY = plan.ptr(plan.in_tensor), plan.ptr(plan.out_tensor)
    L.fortis_stencil_gather_dev(C.byref(gt), ptrs(gb), C.c_void_p(dX))
    plan.run()
    for kk in range(nz):
        L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY + kk * ncells * 3 * 4), kk)
    L.fortis_sync()
    # (the one-launch kernel ends the network on 4x4x1 matrix products, the small-batch MLP kernel of the unfused route
    # on a 16-wide tile: the same sums in another order, equal within the tolerance, not bit for bit)
    Yu = plan.read(plan.out_tensor, (rows, 3))
    assert maxrel(Yu, Y) < TOL
    ref_u = [a.copy() for a in host[:2]] + [np.zeros(n2, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    for kk in range(nz):
        O.stencil_scatter(sd, ref_u, Yu[kk * ncells:(kk + 1) * ncells], ncells, kk, cells=scells)
    for q in (3, 4):
        assert bits_equal(sb[q].get((n3,)), ref_u[q])
    for b in gb + sb:
        b.free()
    plan.close()


def test_bench_grid_fused_equals_unfused_and_layer_vs_oracle(L, gpu):
    """The benchmark grid, 1028 x 1028 x 15 (15.7 M columns), through properties that do not need the oracle at
    that size: the one-launch fused step and the reference's structure (gather kernel -> X -> MLP -> Y -> one
    scatter per layer) run the same arithmetic and must agree bit for bit in Y and in every written field; one
    layer of X and its scatter are checked against the oracle on that layer's planes."""
    sx, sy, nz = 1028, 1028, 15
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    gt, st = S.build_table(gd, lp, kd, "gather"), S.build_table(sd, lp, kd, "scatter")
    A = configs.zb_arrays(sx, sy, nz)
    count, n2, n3 = (sx - 4) * (sy - 4), sx * sy, sx * sy * nz
    rows = count * nz
    net = configs.zb_mlp()
    plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows)
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    host = [A["norm_h"], A["kappa_h"], np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
    fused_out, fused_Y = _fused(L, gt, st, plan, garr, host, rows)
    # the reference's structure
    gb = [DevBuf(L, a) for a in garr]
    sb = [DevBuf(L, a) for a in host]
    dX = L.fortis_plan_tensor_ptr(plan.handle, plan.in_tensor)
    dY = L.fortis_plan_tensor_ptr(plan.handle, plan.out_tensor)
    L.fortis_stencil_gather_dev(C.byref(gt), ptrs(gb), C.c_void_p(dX))
    plan.run()
    for kk in range(nz):
        L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY + kk * count * 3 * 4), kk)
    L.fortis_sync()
    Y = np.empty((rows, 3), np.float32)
    L.fortis_d2h(Y.ctypes.data, C.c_void_p(dY), Y.nbytes)
    assert bits_equal(Y, fused_Y)
    for q in (3, 4):
        assert bits_equal(sb[q].get(host[q].shape), fused_out[q])
    # the 2-D Txy_h: the layer-by-layer scatters leave the last layer in it, the fused step keeps one plane per layer
    assert bits_equal(sb[2].get((n2,)), fused_out[2].reshape(nz, n2)[nz - 1])
    # every layer scattered by ONE launch (the iterations walked inside the kernel): all three written fields as the
    # fused step leaves them, the 2-D one with a plane per layer
    sa = [DevBuf(L, a) for a in host]
    assert L.fortis_stencil_scatter_all_dev(C.byref(st), ptrs(sa), C.c_void_p(dY)) == 0
    L.fortis_sync()
    for q in (2, 3, 4):
        assert bits_equal(sa[q].get(host[q].shape), fused_out[q])
    for b in sa:
        b.free()
    # layer kk against the oracle: X rows of that layer, and the scatter of the GPU's own Y for it
    kk = 7
    Xk = np.empty((count, 27), np.float32)
    L.fortis_d2h(Xk.ctypes.data, C.c_void_p(dX + kk * count * 27 * 4), Xk.nbytes)
    plane = lambda a: np.ascontiguousarray(a.reshape(nz, n2)[kk])
    gd1, sd1, _, _ = configs.zb_descriptors(sx, sy, 1)
    assert bits_equal(Xk, O.stencil_gather(gd1, [plane(a) for a in garr], count, 1, 3, 3, sx - 4))
    ref = [plane(A["norm_h"]), A["kappa_h"], np.zeros(n2, np.float32), np.zeros(n2, np.float32), np.zeros(n2, np.float32)]
    O.stencil_scatter(sd1, ref, Y[kk * count:(kk + 1) * count], count, 0, 3, 3, sx - 4)
    assert bits_equal(plane(fused_out[3]), ref[3]) and bits_equal(plane(fused_out[4]), ref[4])
    # the fp64-accumulated network on a seeded sample of that layer's rows
    idx = np.random.default_rng(6).choice(count, 512, replace=False)
    assert maxrel(Y[kk * count + idx], O.mlp_f64(net["Ws"], net["bs"], net["acts"], Xk[idx])) < TOL
    for b in gb + sb:
        b.free()
    plan.close()



def test_rows_form_divisions_with_operands_outside_the_short_range(L, gpu):
    """The lane-per-row form of the fused step (taken from 786 k rows on) divides the short way only when a whole wave's
    numerators and divisors lie in [2^-40, 2^40], in the lifted expression tv / (S0 + 1e-30f) and in the network's input
    normalisation alike.  Here a share of the field values lies outside: zeros of both signs,
    denormals, values just outside and on the ends of the range, all-ones mantissas, huge values, infinities, NaNs,
    sparse enough that waves of both kinds occur.  The fused step must equal the unfused structure (whose gather kernel
    always divides the long way) bit for bit in Y and in the written fields (any NaN equals any NaN), and its X of one
    layer must equal the oracle's."""
    sx, sy, nz = 600, 600, 3
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    gt, st = S.build_table(gd, lp, kd, "gather"), S.build_table(sd, lp, kd, "scatter")
    A = configs.zb_arrays(sx, sy, nz)
    rng = np.random.default_rng(33)
    ones = np.array([0x3FFFFFFF, 0x2B7FFFFF, 0x53FFFFFF, 0x007FFFFF, 0x7F7FFFFF, 0x00000001, 0x80000001], np.uint32).view(np.float32)
    special = np.concatenate([np.array([0.0, -0.0, 1e-45, 3e-39, 1.1754944e-38, 2.0 ** -100, 2.0 ** -41, -2.0 ** -41, 2.0 ** -40, -2.0 ** -40,
                                        2.0 ** 40, -2.0 ** 40, 2.0 ** 41, 2.0 ** 64, -2.0 ** 100, 3.4028235e38, np.inf, -np.inf, np.nan], np.float32), ones])
    n2, n3 = sx * sy, sx * sy * nz
    for k in ("sh_xy_h", "sh_xx", "vort_xy_h", "norm_h"):
        a = A[k].reshape(-1)
        pick = rng.random(a.size) < 2e-4
        a[pick] = rng.choice(special, int(pick.sum()))
    count = (sx - 4) * (sy - 4)
    rows = count * nz
    assert rows >= 786432
    net = configs.zb_mlp()
    # input normalisation as in the reference's network (x / in_norms before the first layer): the step's second division
    in_norms = rng.uniform(0.5, 2.0, 27).astype(np.float32)
    out_norms = rng.uniform(0.5, 2.0, 3).astype(np.float32)
    plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows, in_norms=in_norms, out_norms=out_norms)
    assert plan.num_kernels == 1
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    host = [A["norm_h"], A["kappa_h"], np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]

    def same(a, b):
        a, b = np.ascontiguousarray(a, dtype=np.float32), np.ascontiguousarray(b, dtype=np.float32)
        return a.shape == b.shape and bool(np.all((a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))))
    with np.errstate(all="ignore"):
        fused_out, fused_Y = _fused(L, gt, st, plan, garr, host, rows)
        gb, sb = [DevBuf(L, a) for a in garr], [DevBuf(L, a) for a in host]
        dX = L.fortis_plan_tensor_ptr(plan.handle, plan.in_tensor)
        dY = L.fortis_plan_tensor_ptr(plan.handle, plan.out_tensor)
        L.fortis_stencil_gather_dev(C.byref(gt), ptrs(gb), C.c_void_p(dX))
        X = np.empty((rows, 27), np.float32)
        L.fortis_d2h(X.ctypes.data, C.c_void_p(dX), X.nbytes)
        plan.run()
        for kk in range(nz):
            L.fortis_stencil_scatter_dev(C.byref(st), ptrs(sb), C.c_void_p(dY + kk * count * 3 * 4), kk)
        L.fortis_sync()
        Y = np.empty((rows, 3), np.float32)
        L.fortis_d2h(Y.ctypes.data, C.c_void_p(dY), Y.nbytes)
        assert same(Y, fused_Y)
        for q in (3, 4):
            assert same(sb[q].get(host[q].shape), fused_out[q])
        # rows with an operand outside the range, and rows without, both occur in numbers
        bad = ~np.all((np.abs(X) >= 2.0 ** -80) & (np.abs(X) <= 2.0 ** 80), axis=1)
        assert 1000 < int(bad.sum()) < rows // 4
        assert same(X[:count], O.stencil_gather(gd, garr, count, nz, 3, 3, sx - 4)[:count])
    for b in gb + sb:
        b.free()
    plan.close()


@pytest.mark.parametrize("form", ["16", "64"])
@pytest.mark.parametrize("sx,sy,nz,hidden", [(68, 78, 15, (64, 64)), (37, 29, 3, (20,)), (133, 70, 2, (48, 16, 8))])
def test_fused_step_both_fast_forms(L, gpu, form, sx, sy, nz, hidden):
    """The two kernels behind the fused step for uniform-stride tables -- a wave per 16 rows, and a lane per row
    with 64 rows per wave -- are chosen by the row count; both are forced here on grids of either size class
    (ragged counts, a partial last group) in a process of their own, since the choice is read from the
    environment once.  Y against the oracle's gather + fp64-accumulated network, fields bit-equal to the
    oracle's scatter of the kernel's own Y."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = f"""
import sys, ctypes as C, numpy as np
sys.path.insert(0, {root!r}); sys.path.insert(0, {os.path.join(root, 'tests')!r})
import fortis_amd
from fortis_amd import configs, plan as P, stencil as S
from oracle import oracle as O
from util import TOL, DevBuf, bits_equal, maxrel, ptrs
L = fortis_amd.load()
sx, sy, nz, hidden = {sx}, {sy}, {nz}, {hidden!r}
gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
gt, st = S.build_table(gd, lp, kd, "gather"), S.build_table(sd, lp, kd, "scatter")
A = configs.zb_arrays(sx, sy, nz)
count, n2, n3 = (sx - 4) * (sy - 4), sx * sy, sx * sy * nz
rows = count * nz
net = configs.zb_mlp(hidden)
plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows)
garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
host = [A["norm_h"], A["kappa_h"], np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
gb, sb = [DevBuf(L, a) for a in garr], [DevBuf(L, a) for a in host]
dY = DevBuf(L, nbytes=rows * 3 * 4)
assert L.fortis_stencil_step_fused(C.byref(gt), C.byref(st), plan.handle, ptrs(gb), ptrs(sb), dY.ptr) == 0
L.fortis_sync()
Y = dY.get((rows, 3))
X = O.stencil_gather(gd, garr, count, nz, 3, 3, sx - 4)
assert maxrel(Y, O.mlp_f64(net["Ws"], net["bs"], net["acts"], X)) < TOL
ref = [a.copy() for a in host[:2]] + [np.zeros(n2, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
txy = np.zeros((nz, n2), np.float32)
for kk in range(nz):
    O.stencil_scatter(sd, ref, Y[kk * count:(kk + 1) * count], count, kk, 3, 3, sx - 4)
    txy[kk] = ref[2]
assert bits_equal(sb[3].get((n3,)), ref[3]) and bits_equal(sb[4].get((n3,)), ref[4]) and bits_equal(sb[2].get((nz, n2)), txy)
print("forms ok")
"""
    env = dict(os.environ, FORTIS_STENCIL_FORM=form)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=110, env=env)
    assert r.returncode == 0 and "forms ok" in r.stdout, r.stdout + r.stderr


def test_fused_step_rejects_mismatched_tables(L, gpu, golden, capfd):
    gt, st, gd, sd, lp, kd = golden_tables(golden)
    net = configs.toy_mlp(64)
    plan = configs.mlp_case_plan(net)               # 64 inputs, not 27
    assert L.fortis_stencil_step_fused(C.byref(gt), C.byref(st), plan.handle, None, None, None) == -1
    assert "do not match" in capfd.readouterr().err
    plan.close()
