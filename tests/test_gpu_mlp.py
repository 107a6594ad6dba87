"""Column MLPs on the GPU through the C ABI: LDS-resident fused chain (narrow networks), MFMA
GEMM + fused epilogue (wide networks), the memref-expanded fortis_gemm entry, boundary pre/post."""
import ctypes as C
import os

import numpy as np
import pytest

from fortis_amd import configs, plan as P
from oracle import oracle as O
from util import TOL, DevBuf, maxrel

pytestmark = pytest.mark.gpu


def test_config1_toy_mlp(L, gpu):
    case = configs.toy_mlp()
    plan = configs.mlp_case_plan(case)
    assert plan.num_kernels == 1                     # whole 64-256-256-32 stack in one kernel
    Y = plan.forward(case["X"], (1024, 32))
    ref = O.mlp_f64(case["Ws"], case["bs"], case["acts"], case["X"])
    assert maxrel(Y, ref) < TOL
    assert abs(float(Y.astype(np.float64).sum()) - float(ref.astype(np.float64).sum())) < 1e-5 * np.abs(ref).sum()
    plan.close()


def test_reference_toy_model_readme_stamp(L, gpu):
    """The reference's own toy: batch 1, Linear(1024,256) ReLU Linear(256,1024), seed 42, z-scored ramp;
    checksum stamp 7.775037 (README.md:25, frontend/export_mlp.py, benchmarks/toy/bench_fortis.f90)."""
    import torch
    torch.manual_seed(42)
    net = torch.nn.Sequential(torch.nn.Linear(1024, 256), torch.nn.ReLU(), torch.nn.Linear(256, 1024)).eval()
    x = torch.arange(1, 1025, dtype=torch.float32) / 1024
    x = ((x - x.mean()) / x.std(unbiased=False)).numpy()[None]
    Ws = [net[0].weight.detach().numpy(), net[2].weight.detach().numpy()]
    bs = [net[0].bias.detach().numpy(), net[2].bias.detach().numpy()]
    plan = P.mlp_plan(Ws, bs, ["relu", None], 1)
    y = plan.forward(x, (1, 1024))
    assert abs(float(y.astype(np.float64).sum()) - 7.775037) / 7.775037 < 1e-5
    assert maxrel(y, O.mlp_f64(Ws, bs, ["relu", "none"], x)) < TOL
    plan.close()


def test_zb_known_answer_vector(L, gpu, golden):
    W = np.load(os.path.join(golden, "zb_nn.npz"))
    plan = P.mlp_plan([W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None], 100, in_norms=W["in_norms"], out_norms=W["out_norms"])
    y = plan.forward(np.tile(W["x_test"], (100, 1)), (100, 3))
    assert maxrel(y[0], W["y_test"]) < TOL and maxrel(y[99], W["y_test"]) < TOL
    plan.close()


@pytest.mark.parametrize("rows", [1, 63, 64, 65, 1000])
def test_chain_ragged_rows(L, gpu, rows):
    """SAM-shaped 61 -> 128 x4 -> 148 network (benchmarks/sam/fwd_native.f90:5, 34-42), row counts around
    the 64-row tile."""
    rng = np.random.default_rng(0)
    widths = [61, 128, 128, 128, 128, 148]
    Ws = [(rng.standard_normal((widths[i + 1], widths[i])) / np.sqrt(widths[i])).astype(np.float32) for i in range(5)]
    bs = [rng.standard_normal(widths[i + 1]).astype(np.float32) * 0.1 for i in range(5)]
    X = rng.standard_normal((rows, 61)).astype(np.float32)
    plan = P.mlp_plan(Ws, bs, ["relu"] * 4 + [None], rows)
    assert plan.num_kernels == 1
    Y = plan.forward(X, (rows, 148))
    assert maxrel(Y, O.mlp_f64(Ws, bs, ["relu"] * 4 + ["none"], X)) < TOL
    plan.close()


def test_config3_climsim_shape_reduced_rows(L, gpu):
    """556 -> 768 x5 LeakyReLU(0.15) -> 368 with the column-major gather/scatter around it, 1024 rows."""
    case = configs.climsim(rows=1024)
    plan = configs.climsim_plan(case)
    B = plan.forward(case["A"].reshape(-1, order="F"), (368, 1024)).T      # column-major (1024, 368)
    X = O.boundary_pre(case["A"], case["mean"], case["vmax"], case["vmin"])
    Yref = O.mlp_f64(case["Ws"], case["bs"], case["acts"], X, alphas=case["alphas"])
    ref = O.boundary_post(Yref, case["scale"])
    assert maxrel(B, ref) < TOL
    plan.close()


def test_config3_climsim_full_size_row_sample(L, gpu):
    """All 24576 columns on the GPU; rows are independent, so a seeded sample of 192 rows is checked
    against the oracle at full width."""
    case = configs.climsim()
    plan = configs.climsim_plan(case, boundary=False)
    X = np.ascontiguousarray(case["A"])                                   # row-major [24576][556]
    Y = plan.forward(X, (24576, 368))
    idx = np.random.default_rng(5).choice(24576, 192, replace=False)
    ref = O.mlp_f64(case["Ws"], case["bs"], case["acts"], X[idx], alphas=case["alphas"])
    assert maxrel(Y[idx], ref) < TOL
    assert np.isfinite(Y).all()
    plan.close()


def test_config3_climsim_full_size_with_boundary_kernels(L, gpu):
    """Config 3 as the benchmark times it: the host's column-major A(24576, 556) in, column-major B(24576, 368)
    out, the boundary transposes around the six GEMMs.  A seeded sample of 192 columns against
    boundary_pre -> fp64-accumulated MLP -> boundary_post; non-trivial mean / range / scale vectors so that a
    dropped or transposed vector shows."""
    case = configs.climsim()
    rng = np.random.default_rng(8)
    case["mean"] = rng.standard_normal(556).astype(np.float32) * np.float32(0.1)
    case["vmax"] = rng.uniform(1.5, 2.5, 556).astype(np.float32)
    case["vmin"] = rng.uniform(0.0, 0.5, 556).astype(np.float32)
    case["scale"] = rng.uniform(0.5, 2.0, 368).astype(np.float32)
    plan = configs.climsim_plan(case, boundary=True)
    assert plan.kernel_names() == ["boundary_pre"] + ["gemm_bias_act"] * 6 + ["boundary_post"]
    B = plan.forward(case["A"].reshape(-1, order="F"), (368, 24576)).T          # column-major (24576, 368)
    idx = np.sort(np.random.default_rng(5).choice(24576, 192, replace=False))
    X = O.boundary_pre(np.asfortranarray(case["A"][idx]), case["mean"], case["vmax"], case["vmin"])
    Yref = O.mlp_f64(case["Ws"], case["bs"], case["acts"], X, alphas=case["alphas"])
    ref = O.boundary_post(Yref, case["scale"])
    assert maxrel(B[idx], ref) < TOL
    assert np.isfinite(B).all()
    plan.close()
    # the boundary kernels alone at this size are exact arithmetic: bit-equal to the oracle on the sampled columns
    p = P.Plan()
    t0, t1, t2 = p.tensor(24576 * 556), p.tensor(24576 * 556), p.tensor(24576 * 556)
    p.boundary_pre(t0, t1, 24576, 556, case["mean"], case["vmax"], case["vmin"], np.float32)
    sc = rng.uniform(0.5, 2.0, 556).astype(np.float32)
    p.boundary_post(t1, t2, 24576, 556, sc, np.float32)
    p.finalize(t0, t2)
    Bt = p.forward(case["A"].reshape(-1, order="F"), (556, 24576)).T
    assert np.array_equal(p.read(t1, (24576, 556))[idx].view(np.uint32), X.view(np.uint32))
    assert np.array_equal(Bt[idx].view(np.uint32), O.boundary_post(X, sc).view(np.uint32))
    p.close()


def test_masked_relu_head_and_output_scale_fold_into_gemm(L, gpu):
    """124 -> 512 -> 128 with ReLU on the last 8 outputs (benchmarks/climsim/export_wide.py:24-28)."""
    rng = np.random.default_rng(1)
    Ws = [(rng.standard_normal((512, 124)) / 11).astype(np.float32), (rng.standard_normal((128, 512)) / 22).astype(np.float32)]
    bs = [rng.standard_normal(512).astype(np.float32), rng.standard_normal(128).astype(np.float32)]
    X = rng.standard_normal((384, 124)).astype(np.float32)
    plan = P.mlp_plan(Ws, bs, ["leaky", None], 384, alphas=[0.15, 0.0], mask_tail=8)
    assert plan.num_kernels == 2                    # mask head folded into the second GEMM's epilogue
    Y = plan.forward(X, (384, 128))
    assert maxrel(Y, O.mlp_f64(Ws, bs, ["leaky", "none"], X, alphas=[0.15, 0.0], mask_tail=8)) < TOL
    assert (Y[:, 120:] >= 0).all() and (Y[:, :120] < 0).any()
    plan.close()
    out_norms = rng.uniform(0.5, 2, 128).astype(np.float32)
    plan = P.mlp_plan(Ws, bs, ["leaky", None], 384, alphas=[0.15, 0.0], out_norms=out_norms)
    assert plan.num_kernels == 2
    Y = plan.forward(X, (384, 128))
    assert maxrel(Y, O.mlp_f64(Ws, bs, ["leaky", "none"], X, alphas=[0.15, 0.0], out_norms=out_norms)) < TOL
    plan.close()


@pytest.mark.parametrize("B,N,K", [(1, 1, 4), (64, 64, 32), (100, 70, 36), (33, 17, 7), (512, 768, 556), (300, 368, 768)])
def test_fortis_gemm_entry(L, gpu, B, N, K):
    """The memref-expanded entry (runtime/fortis_rt.c:45-48): C = A . W^T, offsets honoured, any shape
    (K = 7 takes the guarded non-vector path)."""
    rng = np.random.default_rng(2)
    pad = 8                                           # elements of offset into each allocation
    A = rng.standard_normal(B * K + pad).astype(np.float32)
    W = rng.standard_normal(N * K + pad).astype(np.float32)
    dA, dW, dC = DevBuf(L, A), DevBuf(L, W), DevBuf(L, nbytes=(B * N + pad) * 4)
    L.fortis_gemm(dA.ptr, dA.ptr, pad, B, K, K, 1, dW.ptr, dW.ptr, pad, N, K, K, 1, dC.ptr, dC.ptr, pad, B, N, N, 1, B, N, K)
    Cc = dC.get((B * N + pad,))[pad:].reshape(B, N)
    assert maxrel(Cc, O.gemm(A[pad:].reshape(B, K), W[pad:].reshape(N, K))) < TOL
    for d in (dA, dW, dC):
        d.free()


def test_fortis_gemm_entry_empty_problems(L, gpu, capfd):
    """B = 0 or N = 0: nothing is written and nothing is printed; K = 0: the empty sum, C = 0 (what the reference's
    SGEMM call with beta = 0 does, runtime/fortis_rt.c:69-74)."""
    Cin = np.full(6 * 5, 7.0, np.float32)
    dA, dW, dC = DevBuf(L, np.ones(64, np.float32)), DevBuf(L, np.ones(64, np.float32)), DevBuf(L, Cin)
    for B, N, K in ((0, 5, 4), (6, 0, 4)):
        L.fortis_gemm(dA.ptr, dA.ptr, 0, B, K, K, 1, dW.ptr, dW.ptr, 0, N, K, K, 1, dC.ptr, dC.ptr, 0, B, N, N, 1, B, N, K)
        assert np.array_equal(dC.get((30,)), Cin)
    L.fortis_gemm(dA.ptr, dA.ptr, 0, 4, 0, 0, 1, dW.ptr, dW.ptr, 0, 5, 0, 0, 1, dC.ptr, dC.ptr, 0, 4, 5, 5, 1, 4, 5, 0)
    got = dC.get((30,))
    assert np.array_equal(got[:20], np.zeros(20, np.float32)) and np.array_equal(got[20:], Cin[20:])
    assert "fortis" not in capfd.readouterr().err
    for d in (dA, dW, dC):
        d.free()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("NI,NK", [(384, 124), (50, 33), (1, 1), (300, 5), (6, 400)])
def test_boundary_pre_post_bit_exact(L, gpu, dtype, NI, NK):
    """E3SM boundary shapes (384 x 124 f64 in, trt_backend/e3sm_boundary.cu:9-20) and ragged ones;
    host-type arithmetic then cast, bit-exact against the oracle."""
    rng = np.random.default_rng(3)
    A = np.asfortranarray(rng.standard_normal((NI, NK)).astype(dtype))
    mean, vmax, vmin = rng.standard_normal(NK).astype(dtype), rng.uniform(2, 3, NK).astype(dtype), rng.uniform(0, 1, NK).astype(dtype)
    scale = rng.uniform(0.5, 2, NK).astype(dtype)
    esz = np.dtype(dtype).itemsize
    p = P.Plan()
    t0, t1, t2 = p.tensor(NI * NK, esz), p.tensor(NI * NK), p.tensor(NI * NK, esz)
    p.boundary_pre(t0, t1, NI, NK, mean, vmax, vmin, dtype)
    p.boundary_post(t1, t2, NI, NK, scale, dtype)
    p.finalize(t0, t2)
    p.write(t0, A.reshape(-1, order="F"))
    p.run()
    X = p.read(t1, (NI, NK))
    Bm = p.read(t2, (NK, NI), dtype).T
    Xref = O.boundary_pre(A, mean, vmax, vmin)
    assert np.array_equal(X.view(np.uint32), Xref.view(np.uint32))
    assert np.array_equal(Bm, O.boundary_post(Xref, scale, dtype))
    p.close()


@pytest.mark.parametrize("B,N,K,act", [
    (8300, 1100, 40, "leaky"),     # 585 tiles: whole rounds + a partial round of quarters; ragged B and N; K tail slab
    (12000, 1100, 36, "relu"),     # 846 tiles: whole rounds + a round of halves + quarters
    (16384, 512, 64, None),        # 512 tiles: whole rounds only, no activation
    (257, 385, 4, "leaky"),        # one row / one column past a tile edge, a single 4-wide k slab
    (70000, 300, 20, "relu"),      # several whole rounds with K below one slab: every tile's only slab runs past K,
                                   # also when it is fetched ahead as the next tile's first slab
    (66000, 264, 32, None),        # K of exactly one slab
    (40000, 384, 76, "leaky"),     # two full slabs and a 12-wide tail, three rounds
])
def test_gemm_schedule_phases(L, gpu, B, N, K, act):
    """The persistent GEMM hands out whole 128 x 128 tiles round by round and cuts the remainder into
    halves and quarters; every phase, ragged edges and the slab that runs past K against numpy float64
    (fortis_gemm + epilogue: runtime/fortis_rt.c:45-75, compiler/FortisFuse.cpp:685-760)."""
    rng = np.random.default_rng(7)
    W = (rng.standard_normal((N, K)) / np.sqrt(K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    X = rng.standard_normal((B, K)).astype(np.float32)
    p = P.Plan()
    t0, t1 = p.tensor(B * K), p.tensor(B * N)
    p.linear(t0, t1, W, b, B, act, 0.15)
    plan = p.finalize(t0, t1)
    assert plan.kernel_names() == ["gemm_bias_act"]
    Y = plan.forward(X, (B, N))
    ref = O.mlp_f64([W], [b], [act or "none"], X, alphas=[0.15])
    assert maxrel(Y, ref) < TOL
    plan.close()


@pytest.mark.parametrize("rows,widths", [
    (20000, [200, 256, 17]),       # 13 k groups in, 16 n-tiles: the wide register-resident variant, ragged tail tile
    (16400, [61, 128, 128, 148]),  # SAM-shaped widths, input not a multiple of 4 (scalar loads), 148 outputs
    (16385, [64, 64, 8]),          # 16-byte input loads and output stores, one row past a tile
    (16391, [27, 64, 3]),          # thin outputs leave a tile in one store after a change of lanes; ragged last tile
    (16397, [20, 32, 2]),
    (16387, [12, 48, 1]),
])
def test_chain_wave_kernel_plain_shapes(L, gpu, rows, widths):
    """Many rows take the wave-per-16-rows chain kernel; widths up to 256, vector and scalar row access."""
    rng = np.random.default_rng(11)
    n = len(widths) - 1
    Ws = [(rng.standard_normal((widths[i + 1], widths[i])) / np.sqrt(widths[i])).astype(np.float32) for i in range(n)]
    bs = [rng.standard_normal(widths[i + 1]).astype(np.float32) * 0.1 for i in range(n)]
    acts = ["relu"] * (n - 1) + [None]
    X = rng.standard_normal((rows, widths[0])).astype(np.float32)
    plan = P.mlp_plan(Ws, bs, acts, rows)
    assert plan.num_kernels == 1
    Y = plan.forward(X, (rows, widths[-1]))
    idx = np.r_[0:64, rows - 64:rows, np.random.default_rng(3).choice(rows, 256, replace=False)]
    ref = O.mlp_f64(Ws, bs, ["relu"] * (n - 1) + ["none"], X[idx])
    assert maxrel(Y[idx], ref) < TOL
    assert np.isfinite(Y).all()
    if widths[-1] < 4:     # every row once (a row stored twice or not at all would pass the sample above)
        assert maxrel(Y, O.mlp_f64(Ws, bs, ["relu"] * (n - 1) + ["none"], X)) < TOL
    plan.close()
