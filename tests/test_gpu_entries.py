"""The host-facing entry points (the generated shim's names, driver/fortis_shim.py:54-135, and the
generated gather/scatter wrappers, mom6_zb/gather.cu:50-57, 82-91) driven the way a Fortran host
drives them."""
import ctypes as C
import os

import numpy as np
import pytest

from fortis_amd import configs, plan as P, stencil as S, step as ST
from oracle import oracle as O
from util import TOL, DevBuf, bits_equal, maxrel

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_step(L):
    yield
    ST.reset()


def _toy(rows=256):
    case = configs.toy_mlp(rows)
    return case, configs.mlp_case_plan(case), O.mlp_f64(case["Ws"], case["bs"], case["acts"], case["X"])


def test_whole_array_call_and_resident_entries(L, gpu):
    """mlp_forward(x, y) and the upload / forward_dev / download triple of benchmarks/toy/bench_dev.f90:4-11."""
    case, plan, ref = _toy()
    ST.bind(plan, case["X"].size, ref.size)
    y = np.empty_like(ref)
    ST.mlp_forward(case["X"], y)
    assert maxrel(y, ref) < TOL
    y2 = np.zeros_like(ref)
    ST.mlp_upload(case["X"])
    for _ in range(3):
        ST.mlp_forward_dev()
    ST.mlp_download(y2)
    assert bits_equal(y, y2)


def test_whole_array_call_large_arrays(L, gpu, monkeypatch):
    """Host arrays of 8 MB and more travel in chunks through page-locked staging, copied by several host threads:
    the result must be the one of the plain copies (FORTIS_NO_STAGED_COPY=1), bit for bit, on arrays whose size
    is not a multiple of the chunk; a sample of rows is checked against the oracle."""
    rows = 41003
    rng = np.random.default_rng(11)
    Ws = [(rng.standard_normal((96, 64)) / 8).astype(np.float32), (rng.standard_normal((72, 96)) / 10).astype(np.float32)]
    bs = [rng.standard_normal(96).astype(np.float32), rng.standard_normal(72).astype(np.float32)]
    X = rng.standard_normal((rows, 64)).astype(np.float32)                 # 10.5 MB in, 11.8 MB out
    plan = P.mlp_plan(Ws, bs, ["relu", None], rows)
    ST.bind(plan, X.size, rows * 72)
    y = np.zeros((rows, 72), np.float32)
    ST.mlp_forward(X, y)
    idx = rng.choice(rows, 256, replace=False)
    assert maxrel(y[idx], O.mlp_f64(Ws, bs, ["relu", None], X[idx])) < TOL
    y2 = np.zeros_like(y)
    ST.mlp_upload(X)
    ST.mlp_forward_dev()
    ST.mlp_download(y2)
    assert bits_equal(y, y2)
    # a second call with other data reuses the staging buffers
    X2 = rng.standard_normal((rows, 64)).astype(np.float32)
    y3 = np.zeros_like(y)
    ST.mlp_forward(X2, y3)
    monkeypatch.setenv("FORTIS_NO_STAGED_COPY", "1")
    ST.reset()
    plan = P.mlp_plan(Ws, bs, ["relu", None], rows)
    ST.bind(plan, X.size, rows * 72)
    y4 = np.zeros_like(y)
    ST.mlp_forward(X2, y4)
    assert bits_equal(y3, y4) and not bits_equal(y3, y)
    # the batched slice form on the same arrays takes the same route
    monkeypatch.delenv("FORTIS_NO_STAGED_COPY")
    ST.reset()
    plan = P.mlp_plan(Ws, bs, ["relu", None], rows)
    ST.bind(plan, X.size, rows * 72, verdict="batched", count=rows, lo=1, step=1, minc=1)
    y5 = np.zeros_like(y)
    ST.mlp_forward_batched(X2, y5)
    assert bits_equal(y5, y4)


def test_graph_capture_on_second_call_and_replay(L, gpu, monkeypatch):
    """fortis.graph set: call 1 eager, call 2 captures and launches, later calls replay
    (driver/fortis_shim.py:82-90).  Every replay must equal the eager result, with eager work and
    synchronisations in between.  FORTIS_GRAPH_KEEP pins the replay (without it the library keeps the
    graph only where it measures faster than plain launches)."""
    monkeypatch.setenv("FORTIS_GRAPH_KEEP", "1")
    case, plan, ref = _toy()
    ST.bind(plan, case["X"].size, ref.size, graph=True)
    outs = []
    rng = np.random.default_rng(3)
    for n in range(6):
        x = case["X"] if n in (0, 5) else rng.uniform(-1, 1, case["X"].shape).astype(np.float32)
        y = np.empty_like(ref)
        ST.mlp_forward(x, y)
        assert ST.graph_active() == (n >= 1)
        assert maxrel(y, O.mlp_f64(case["Ws"], case["bs"], case["acts"], x)) < TOL
        outs.append(y)
        plan.run()                                   # eager work between replays
        L.fortis_sync()
    assert bits_equal(outs[0], outs[5])              # eager call == replayed call on the same input


def test_graph_env_switch(L, gpu, monkeypatch):
    case, plan, ref = _toy()
    ST.bind(plan, case["X"].size, ref.size, graph=False)
    y = np.empty_like(ref)
    ST.mlp_forward(case["X"], y)
    ST.mlp_forward(case["X"], y)
    assert not ST.graph_active()
    ST.reset()
    monkeypatch.setenv("FORTIS_GRAPH", "1")
    monkeypatch.setenv("FORTIS_GRAPH_KEEP", "1")
    ST.bind(plan, case["X"].size, ref.size, graph=False)
    ST.mlp_forward(case["X"], y)
    ST.mlp_forward(case["X"], y)
    assert ST.graph_active() and maxrel(y, ref) < TOL


def test_graph_kept_only_for_steps_of_several_kernels(L, gpu, monkeypatch):
    """Without FORTIS_GRAPH_KEEP a captured graph is kept by a rule on the plan alone (at least
    FORTIS_GRAPH_MIN_KERNELS kernels, default 6: a graph launch costs several plain launches on this runtime),
    never by timing, and a call runs the step exactly once: an in-place op on the resident input shows any
    extra pass."""
    case, plan, ref = _toy()                                     # one fused kernel: stays eager
    ST.bind(plan, case["X"].size, ref.size, graph=True)
    y = np.empty_like(ref)
    first = None
    for n in range(4):
        ST.mlp_forward(case["X"], y)
        assert maxrel(y, ref) < TOL and not ST.graph_active()
        first = y.copy() if first is None else first
        assert bits_equal(y, first)
    ST.reset()
    # seven kernels (wide layers run one GEMM each): captured on call 2, replayed after
    rng = np.random.default_rng(12)
    widths = [40] + [300] * 6 + [24]
    Ws = [(rng.standard_normal((widths[i + 1], widths[i])) / np.sqrt(widths[i])).astype(np.float32) for i in range(7)]
    bs = [rng.standard_normal(widths[i + 1]).astype(np.float32) * np.float32(0.1) for i in range(7)]
    X = rng.standard_normal((500, 40)).astype(np.float32)
    plan7 = P.mlp_plan(Ws, bs, ["relu"] * 6 + [None], 500)
    assert plan7.num_kernels == 7
    ST.bind(plan7, X.size, 500 * 24, graph=True)
    y7, ref7 = np.empty((500, 24), np.float32), O.mlp_f64(Ws, bs, ["relu"] * 6 + [None], X)
    for n in range(4):
        ST.mlp_forward(X, y7)
        assert ST.graph_active() == (n >= 1) and maxrel(y7, ref7) < TOL
    ST.reset()
    # a step that doubles its resident input in place: after k calls the input holds 2^k times the upload,
    # whatever the graph decision on call 2
    monkeypatch.setenv("FORTIS_GRAPH_KEEP", "1")
    p = P.Plan()
    t0, t1 = p.tensor(64 * 8), p.tensor(64 * 8)
    two = np.full(8, 2, np.float32)
    p.scale(t0, t0, two, 64, divide=False)
    p.scale(t0, t1, np.ones(8, np.float32), 64, divide=False)
    p.finalize(t0, t1)
    ST.bind(p, 64 * 8, 64 * 8, graph=True)
    x = rng.standard_normal((64, 8)).astype(np.float32)
    out = np.empty_like(x)
    ST.mlp_upload(x)
    for k in range(1, 5):
        ST.mlp_forward_dev()
        ST.mlp_download(out)
        assert bits_equal(out, x * np.float32(2 ** k)), k
    assert ST.graph_active()
    ST.reset()


def test_pack_batched_unpack(L, gpu):
    """Fissioned per-column loop: fortis_pack x B -> mlp_forward_batched() -> fortis_unpack x B
    (driver/fortis_shim.py:99-115)."""
    case, plan, ref = _toy(200)
    ST.bind(plan, case["X"].size, ref.size, verdict="batched", expanded=True, count=200)
    for col in range(200):
        ST.fortis_pack(case["X"][col], col)
    ST.mlp_forward_batched()
    y = np.empty_like(ref)
    row = np.empty(32, np.float32)
    for col in range(200):
        ST.fortis_unpack(row, col)
        y[col] = row
    assert maxrel(y, ref) < TOL
    # a per-row call outside the loop goes through the same batched model (fortis_shim.py:122)
    ST.mlp_forward(case["X"][7], row)
    assert maxrel(row, ref[7]) < TOL * np.abs(ref).max() / np.abs(ref[7]).max()


def test_batched_slice_forms(L, gpu):
    """Slice form on the host's whole arrays: unit stride (fortis_shim.py:117-118) and the strided
    upload with step 2, first visited column 3 (fortis_shim.py:119-121)."""
    case, plan, ref = _toy(100)
    ST.bind(plan, case["X"].size, ref.size, verdict="batched", count=100, lo=1, step=1, minc=1)
    y = np.empty_like(ref)
    ST.mlp_forward_batched(case["X"], y)
    assert maxrel(y, ref) < TOL
    ST.reset()
    big = np.random.default_rng(9).uniform(-1, 1, (210, 64)).astype(np.float32)
    out = np.zeros((210, 32), np.float32)
    ST.bind(plan, 100 * 64, 100 * 32, verdict="batched", count=100, lo=3, step=2, minc=3)
    ST.mlp_forward_batched(big, out)
    rows = np.arange(100) * 2 + 2                                  # 0-based rows 2, 4, ...
    full = O.mlp_f64(case["Ws"], case["bs"], case["acts"], big[rows])
    assert maxrel(out[rows], full) < TOL
    untouched = np.setdiff1d(np.arange(210), rows)
    assert not out[untouched].any()


def test_boundary_verdict_f64_host_arrays(L, gpu):
    """Boundary verdict: mlp_forward takes the host's own f64 column-major arrays (benchmarks/cam host,
    driver/fortis_emit2d.py:20-52; trt_backend/e3sm_boundary.cu)."""
    rng = np.random.default_rng(4)
    NI, NIN, NOUT = 384, 124, 128
    Ws = [(rng.standard_normal((128, NIN)) / 11).astype(np.float32), (rng.standard_normal((NOUT, 128)) / 11).astype(np.float32)]
    bs = [rng.standard_normal(128).astype(np.float32), rng.standard_normal(NOUT).astype(np.float32)]
    A = np.asfortranarray(rng.standard_normal((NI, NIN)))
    mean, vmax, vmin, scale = rng.standard_normal(NIN), rng.uniform(2, 3, NIN), rng.uniform(0, 1, NIN), rng.uniform(0.5, 2, NOUT)
    p = P.Plan()
    t0, t1, t2, t3, t4 = p.tensor(NI * NIN, 8), p.tensor(NI * NIN), p.tensor(NI * 128), p.tensor(NI * NOUT), p.tensor(NI * NOUT, 8)
    p.boundary_pre(t0, t1, NI, NIN, mean, vmax, vmin, np.float64)
    p.linear(t1, t2, Ws[0], bs[0], NI, "leaky", 0.15)
    p.linear(t2, t3, Ws[1], bs[1], NI, None)
    p.boundary_post(t3, t4, NI, NOUT, scale, np.float64)
    p.finalize(t0, t4)
    assert p.num_kernels == 3                                       # pre, fused 2-layer chain, post
    ST.bind(p, NI * NIN, NI * NOUT, verdict="boundary", in_dtype=np.float64, out_dtype=np.float64)
    B = np.empty((NI, NOUT), np.float64, order="F")
    ST.mlp_forward(A, B)
    X = O.boundary_pre(A, mean, vmax, vmin)
    ref = O.boundary_post(O.mlp_f64(Ws, bs, ["leaky", "none"], X, alphas=[0.15, 0]), scale, np.float64)
    assert maxrel(B, ref) < TOL


@pytest.mark.parametrize("dtype,hidden", [(np.float64, 320), (np.float32, 96)])
def test_boundary_verdict_large_arrays_in_row_bands(L, gpu, monkeypatch, dtype, hidden):
    """A whole-array call on large host arrays runs in row bands (copies of one band under the computation of
    another); the host's column-major boundary arrays are packed band by band.  The result must be the one of the
    whole array at once (FORTIS_BANDS=1), bit for bit, for a ragged last band, with the wide layers on the GEMM
    kernel (hidden 320) and the narrow ones in the chain kernel, and a sample of rows must agree with the oracle."""
    rng = np.random.default_rng(14)
    NI, NIN, NOUT = 30011, 120, 72
    Ws = [(rng.standard_normal((hidden, NIN)) / 11).astype(np.float32), (rng.standard_normal((NOUT, hidden)) / np.sqrt(hidden)).astype(np.float32)]
    bs = [rng.standard_normal(hidden).astype(np.float32), rng.standard_normal(NOUT).astype(np.float32)]
    A = np.asfortranarray(rng.standard_normal((NI, NIN)).astype(dtype))
    mean, vmax, vmin, scale = (v.astype(dtype) for v in (rng.standard_normal(NIN), rng.uniform(2, 3, NIN), rng.uniform(0, 1, NIN), rng.uniform(0.5, 2, NOUT)))
    esz = np.dtype(dtype).itemsize
    outs = []
    for bands in ("3", "1"):
        monkeypatch.setenv("FORTIS_BANDS", bands)
        ST.reset()
        p = P.Plan()
        t0, t1, t2, t3, t4 = p.tensor(NI * NIN, esz), p.tensor(NI * NIN), p.tensor(NI * hidden), p.tensor(NI * NOUT), p.tensor(NI * NOUT, esz)
        p.boundary_pre(t0, t1, NI, NIN, mean, vmax, vmin, dtype)
        p.linear(t1, t2, Ws[0], bs[0], NI, "leaky", 0.15)
        p.linear(t2, t3, Ws[1], bs[1], NI, None)
        p.boundary_post(t3, t4, NI, NOUT, scale, dtype)
        p.finalize(t0, t4)
        ST.bind(p, NI * NIN, NI * NOUT, verdict="boundary", in_dtype=dtype, out_dtype=dtype)
        B = np.zeros((NI, NOUT), dtype, order="F")
        ST.mlp_forward(A, B)
        B2 = np.zeros((NI, NOUT), dtype, order="F")
        ST.mlp_forward(A, B2)                                       # a second call reuses staging and events
        assert bits_equal(B, B2)
        outs.append(B)
    assert bits_equal(outs[0], outs[1])
    idx = np.sort(rng.choice(NI, 400, replace=False))
    X = O.boundary_pre(np.asfortranarray(A[idx]), mean, vmax, vmin)
    ref = O.boundary_post(O.mlp_f64(Ws, bs, ["leaky", "none"], X, alphas=[0.15, 0]), scale, dtype)
    assert maxrel(outs[0][idx], ref) < TOL
    ST.reset()


def test_run_time_extents(L, gpu):
    """fortis_begin(count) (driver/fortis_stub.c:12-31): the step bound for 200 rows serves 120, then 333 (more
    than it was bound for: the reference's stub specialises for any count), then 200 again."""
    case, plan, ref = _toy(200)
    big = configs.toy_mlp(333)
    refbig = O.mlp_f64(big["Ws"], big["bs"], big["acts"], big["X"])
    ST.bind(plan, case["X"].size, ref.size, verdict="batched", expanded=True, count=200)
    row = np.empty(32, np.float32)
    for count, X, R in ((120, case["X"], ref), (333, big["X"], refbig), (200, case["X"], ref)):
        ST.fortis_begin(count)
        for col in range(count):
            ST.fortis_pack(X[col], col)
        ST.mlp_forward_batched()
        y = np.empty((count, 32), np.float32)
        for col in range(count):
            ST.fortis_unpack(row, col)
            y[col] = row
        assert maxrel(y, R[:count]) < TOL, count


def test_run_time_extents_on_the_lifted_zb_step(L, gpu, golden):
    """The run-time-extent host (mom6_zb/zb_host_rt.f90, mom6_zb/README.md:35-37) runs one build at 60x70x15
    (4736 cells per layer) and at 40x50x10 (2376): here one bound step, begun at 71,040 rows with the tables of
    the 68 x 78 x 15 arrays, then re-begun at 23,760 rows with the tables of 48 x 58 x 10 arrays, then at a grid
    larger than the first (100 x 90 x 15 arrays: 123,840 rows).  Gather rows bit-exact, fields against the
    oracle's scatter of the GPU's own model output bit-exact, model output within 1e-5."""
    W = np.load(os.path.join(golden, "zb_nn.npz"))
    Ws, bs = [W["A0"], W["A1"]], [W["b0"], W["b1"]]
    plan = P.mlp_plan(Ws, bs, ["relu", None], 71040, in_norms=W["in_norms"], out_norms=W["out_norms"])
    ST.bind(plan, 71040 * 27, 71040 * 3, verdict="batched", expanded=True, count=71040, gather=True, scatter=True)
    for sx, sy, nz in ((68, 78, 15), (48, 58, 10), (100, 90, 15), (68, 78, 15)):
        gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
        A = configs.zb_arrays(sx, sy, nz)
        count = (sx - 4) * (sy - 4)
        rows = count * nz
        ST.fortis_begin(rows)
        ST.gather_config(S.build_table(gd, lp, kd, "gather"))
        ST.scatter_config(S.build_table(sd, lp, kd, "scatter"))
        garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
        n2, n3 = sx * sy, sx * sy * nz
        Txy_h, Txx, Tyy = np.zeros(n2, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)
        L.fortis_gather(*[a.ctypes.data for a in garr])
        ST.mlp_forward_batched()
        txy = np.zeros((nz, n2), np.float32)
        for k in range(1, nz + 1):
            L.fortis_scatter(k, *[a.ctypes.data for a in (A["norm_h"], A["kappa_h"], Txy_h, Txx, Tyy)])
            txy[k - 1] = Txy_h
        X = np.empty((rows, 27), np.float32)
        Y = np.empty((rows, 3), np.float32)
        L.fortis_d2h(X.ctypes.data, L.fortis_model_input(), X.nbytes)
        L.fortis_d2h(Y.ctypes.data, L.fortis_model_output(), Y.nbytes)
        assert bits_equal(X, O.stencil_gather(gd, garr, count, nz, 3, 3, sx - 4)), (sx, sy, nz)
        assert maxrel(Y, O.mlp_f64(Ws, bs, ["relu", None], X, in_norms=W["in_norms"], out_norms=W["out_norms"])) < TOL
        ref = [A["norm_h"].copy(), A["kappa_h"].copy(), np.zeros(n2, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]
        for kk in range(nz):
            O.stencil_scatter(sd, ref, Y[kk * count:(kk + 1) * count], count, kk, 3, 3, sx - 4)
            assert bits_equal(txy[kk], ref[2]), (sx, sy, nz, kk)
        assert bits_equal(Txx, ref[3]) and bits_equal(Tyy, ref[4]) and np.abs(Txx).max() > 0


def test_plan_buffers_follow_tensor_lifetimes(L, gpu):
    """Temporaries are taken from the pool in front of the kernel that first writes them and handed back behind
    the one that last reads them (compiler/FortisFuse.cpp:512-516), so a deep stack holds a few activations,
    not one per layer; the outputs are what a plan with one buffer per tensor gives."""
    import ctypes as C
    held0, used0 = C.c_int(), C.c_int()
    L.fortis_pool_stats(C.byref(held0), C.byref(used0))
    case = configs.climsim(rows=2048)
    plan = configs.climsim_plan(case)                            # 9 tensors: A, X, five hidden, Y, B
    held, used = C.c_int(), C.c_int()
    L.fortis_pool_stats(C.byref(held), C.byref(used))
    assert used.value - used0.value <= 4                         # in, out and two activations in flight
    B = plan.forward(case["A"].reshape(-1, order="F"), (368, 2048)).T
    X = O.boundary_pre(case["A"], case["mean"], case["vmax"], case["vmin"])
    ref = O.boundary_post(O.mlp_f64(case["Ws"], case["bs"], case["acts"], X, alphas=case["alphas"]), case["scale"])
    assert maxrel(B, ref) < TOL
    B2 = plan.forward(case["A"].reshape(-1, order="F"), (368, 2048)).T
    assert bits_equal(B, B2)
    plan.close()
    L.fortis_pool_stats(C.byref(held), C.byref(used))
    assert used.value == used0.value
    case = configs.tsrgan(D=9, ch=16, nblocks=3)
    plan = configs.tsrgan_plan(case)                             # 13 tensors
    L.fortis_pool_stats(C.byref(held), C.byref(used))
    assert used.value - used0.value <= 6
    y = plan.forward(case["x"], (18, 18, 18, 3))
    y2 = plan.forward(case["x"], (18, 18, 18, 3))
    assert bits_equal(y, y2)
    plan.close()


def _corner_interp(Txy_h, maskBu, sx=68, sy=78):
    """Txy(I,J) = 0.25*((Txy_h(i+1,j+1)+Txy_h(i,j)) + (Txy_h(i+1,j)+Txy_h(i,j+1))) * mask2dBu over
    J=3..75, I=3..65 (mom6_zb/zb_host.f90:102-105), fp32 in the host's operation order."""
    h, m = Txy_h.reshape(sy, sx), maskBu.reshape(sy, sx)
    out = np.zeros((sy, sx), np.float32)
    J, I = slice(2, 75), slice(2, 65)
    J1, I1 = slice(3, 76), slice(3, 66)
    out[J, I] = np.float32(0.25) * ((h[J1, I1] + h[J, I]) + (h[J, I1] + h[J1, I])) * m[J, I]
    return out


def test_zb_host_step_through_gather_batched_scatter(L, gpu, golden, monkeypatch):
    """The fissioned ZB host's step (mom6_zb/host_fissioned.fir:732-740): fortis_gather(4 arrays) ->
    mlp_forward_batched() -> do k: fortis_scatter(k, 5 arrays) + host corner interpolation; results
    against the fixture written by the reference's own CPU build."""
    monkeypatch.setenv("FORTIS_GRAPH_KEEP", "1")                   # exercise the replay path whatever the timing says
    gt, st, gd, sd, lp, kd = S.load_tables(*[os.path.join(golden, f"zb_{n}.json") for n in ("gather", "scatter", "loop", "kdist")])
    W = np.load(os.path.join(golden, "zb_nn.npz"))
    G = np.load(os.path.join(golden, "zb_native_golden.npz"))
    F = O.zb_fields()
    Pp = O.zb_prep(F)
    plan = P.mlp_plan([W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None], 71040, in_norms=W["in_norms"], out_norms=W["out_norms"])
    ST.bind(plan, 71040 * 27, 71040 * 3, verdict="batched", expanded=True, count=71040, gather=True, scatter=True, graph=True)
    ST.gather_config(gt)
    ST.scatter_config(st)
    n3 = 68 * 78 * 15
    for step in range(3):                                            # step 2 captures the graph, step 3 replays
        Txy_h, Txx, Tyy, Txy = np.zeros(68 * 78, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)
        L.fortis_gather(*[a.ctypes.data for a in (Pp["sh_xy_h"], F["sh_xx"], Pp["vort_xy_h"], Pp["norm_h"])])
        ST.mlp_forward_batched()
        for k in range(1, 16):
            L.fortis_scatter(k, *[a.ctypes.data for a in (Pp["norm_h"], F["kappa_h"], Txy_h, Txx, Tyy)])
            Txy.reshape(15, 78, 68)[k - 1] = _corner_interp(Txy_h, F["mask2dBu"])
        lay = G["layers"] - 1
        assert maxrel(Txx.reshape(15, 78, 68)[lay], G["Txx"]) < TOL
        assert maxrel(Tyy.reshape(15, 78, 68)[lay], G["Tyy"]) < TOL
        assert maxrel(Txy.reshape(15, 78, 68)[lay], G["Txy"]) < TOL
        for n, a in enumerate((Txx, Tyy, Txy)):
            assert abs(a.astype(np.float64).sum() - G["checksum"][n]) < 1e-5 * np.abs(a).sum()
        # cells outside the visited rectangle are never written
        assert not Txx.reshape(15, 78, 68)[:, :2].any() and not Txx.reshape(15, 78, 68)[:, :, 66:].any()
    assert ST.graph_active()
    # the gather wrote the model input exactly as the oracle's gather does
    X = np.empty((71040, 27), np.float32)
    L.fortis_d2h(X.ctypes.data, L.fortis_model_input(), X.nbytes)
    assert bits_equal(X, O.stencil_gather(gd, [Pp["sh_xy_h"], F["sh_xx"], Pp["vort_xy_h"], Pp["norm_h"]], 4736, 15, 3, 3, 64))


def test_scatter_reuse_is_verified_against_the_host_arrays(L, gpu, golden):
    """Under loop distribution the first fortis_scatter of a step computes every iteration and later calls
    only copy rows out -- but only while the scalars' planes the host passes are still the bytes read at the
    first call.  A host that changes norm_h(:,:,k) between two scatter calls must get the result for the
    changed values (the one-iteration path), bit for bit what the per-call path gives."""
    gt, st, gd, sd, lp, kd = S.load_tables(*[os.path.join(golden, f"zb_{n}.json") for n in ("gather", "scatter", "loop", "kdist")])
    W = np.load(os.path.join(golden, "zb_nn.npz"))
    F = O.zb_fields()
    Pp = O.zb_prep(F)
    n3 = 68 * 78 * 15
    results = {}
    for mode in ("reuse", "per_call"):
        if mode == "per_call":
            os.environ["FORTIS_SCATTER_PER_CALL"] = "1"
        try:
            ST.reset()
            plan = P.mlp_plan([W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None], 71040, in_norms=W["in_norms"], out_norms=W["out_norms"])
            ST.bind(plan, 71040 * 27, 71040 * 3, verdict="batched", expanded=True, count=71040, gather=True, scatter=True)
            ST.gather_config(gt)
            ST.scatter_config(st)
            norm = Pp["norm_h"].copy()
            Txy_h, Txx, Tyy = np.zeros(68 * 78, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)
            L.fortis_gather(*[a.ctypes.data for a in (Pp["sh_xy_h"], F["sh_xx"], Pp["vort_xy_h"], norm)])
            ST.mlp_forward_batched()
            planes = []
            for k in range(1, 16):
                if k == 7:
                    norm.reshape(15, 78, 68)[6] *= np.float32(1.5)          # the host changes layer 7's scalars
                L.fortis_scatter(k, *[a.ctypes.data for a in (norm, F["kappa_h"], Txy_h, Txx, Tyy)])
                planes.append(Txy_h.copy())
            results[mode] = (Txx.copy(), Tyy.copy(), np.stack(planes))
            plan.close()
        finally:
            os.environ.pop("FORTIS_SCATTER_PER_CALL", None)
    for a, b in zip(results["reuse"], results["per_call"]):
        assert bits_equal(a, b)
    # and layer 7 really was computed from the changed scalars: (y * S0 * S0) * S1 grows by 1.5^2 there
    G = np.load(os.path.join(golden, "zb_native_golden.npz"))
    Txx = results["reuse"][0].reshape(15, 78, 68)
    assert maxrel(Txx[7], G["Txx"][1]) < TOL                       # layer 8 untouched
    assert np.abs(Txx[6]).max() > 0


def test_measurement_aids(L, gpu):
    """fortis_time_parts_ms clocks the parts of a step in order (every part ran once per iteration, every time is
    positive, bad arguments are refused)."""
    n = 1 << 20
    a, b, c = DevBuf(L, np.arange(n, dtype=np.float32)), DevBuf(L, nbytes=4 * n), DevBuf(L, nbytes=4 * n)
    calls = []
    CB = C.CFUNCTYPE(None, C.c_void_p)
    f1 = CB(lambda _: (calls.append(1), L.fortis_d2d(b.ptr, a.ptr, 4 * n)))
    f2 = CB(lambda _: (calls.append(2), L.fortis_d2d(c.ptr, b.ptr, 4 * n)))
    ms = (C.c_float * 2)()
    assert L.fortis_time_parts_ms(2, (CB * 2)(f1, f2), None, 3, ms) == 0
    assert calls == [1, 2] * 3 and ms[0] > 0 and ms[1] > 0
    assert np.array_equal(c.get((n,)), np.arange(n, dtype=np.float32))
    assert L.fortis_time_parts_ms(0, (CB * 2)(f1, f2), None, 3, ms) == -1
    assert L.fortis_time_parts_ms(2, (CB * 2)(f1, f2), None, 0, ms) == -1
    for d in (a, b, c):
        d.free()
