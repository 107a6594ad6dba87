"""Pins the oracle's MLP / GEMM / conv / pool / boundary functions: README stamps of the reference,
library routines (torch.nn.functional on CPU, numpy float64) and closed-form invariants."""
import numpy as np
import pytest
import torch
import torch.nn.functional as TF

from oracle import oracle as O
from util import maxrel


def _zscore_arange(n):
    # benchmarks/toy/bench_fortis.f90:13-16: y = i/n, then (y - mean)/std (population)
    x = torch.arange(1, n + 1, dtype=torch.float32) / n
    return (x - x.mean()) / x.std(unbiased=False)


def test_toy_mlp_readme_stamp():
    """README.md:25 'toy MLP checksum 7.775037': Linear(1024,256) ReLU Linear(256,1024), seed 42
    (frontend/export_mlp.py:3-12), input the z-scored ramp.  The stamp was printed by an fp32 GPU run
    summed in fp32 by the Fortran host; agreement to 1e-5 relative is what it can pin."""
    torch.manual_seed(42)
    net = torch.nn.Sequential(torch.nn.Linear(1024, 256), torch.nn.ReLU(), torch.nn.Linear(256, 1024)).eval()
    x = _zscore_arange(1024).numpy()[None]
    Ws = [net[0].weight.detach().numpy(), net[2].weight.detach().numpy()]
    bs = [net[0].bias.detach().numpy(), net[2].bias.detach().numpy()]
    z = O.mlp_f64(Ws, bs, ["relu", "none"], x)
    assert abs(float(z.astype(np.float64).sum()) - 7.775037) / 7.775037 < 1e-5
    zn = O.mlp_native(Ws, bs, x)
    assert abs(float(zn.astype(np.float64).sum()) - 7.775037) / 7.775037 < 1e-5


def test_conv_probe_readme_stamp():
    """README.md:25 'conv probe 9617.28': Conv3d(3,8,3,pad 1) + LeakyReLU(0.1), seed 3, z-scored ramp as
    1x3x16^3 (frontend/export_conv.py:3-9).  The stamp is the reference host's fp32 sum of 32768 outputs as printed
    to six digits; the exact sum of the correct outputs is 9617.4091 (this oracle and torch agree on it to 3e-9), i.e. the
    stamp itself sits 1.34e-5 away, hence the 3e-5 bound here; element-wise agreement with torch is asserted below."""
    torch.manual_seed(3)
    m = torch.nn.Sequential(torch.nn.Conv3d(3, 8, 3, padding=1), torch.nn.LeakyReLU(0.1)).eval()
    x = _zscore_arange(3 * 16 ** 3).view(1, 3, 16, 16, 16)
    y = O.conv3d(x.numpy(), m[0].weight.detach().numpy(), pad=(1, 1, 1)) + m[0].bias.detach().numpy()[None, :, None, None, None]
    y = np.where(y > 0, y, np.float32(0.1) * y)
    assert abs(float(y.astype(np.float64).sum()) - 9617.28) / 9617.28 < 3e-5
    with torch.no_grad():
        assert maxrel(y, m(x).numpy()) < 1e-6


@pytest.mark.parametrize("stride,pad,k", [(1, 1, 3), (2, 1, 3), (1, 0, 1), (1, 2, 5)])
def test_conv2d_vs_torch(stride, pad, k):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((1, 5, 17, 13)).astype(np.float32)
    w = rng.standard_normal((7, 5, k, k)).astype(np.float32)
    y = O.conv2d(x, w, (stride, stride), (pad, pad))
    ref = TF.conv2d(torch.tensor(x), torch.tensor(w), stride=stride, padding=pad).numpy()
    assert y.shape == ref.shape and maxrel(y, ref) < 2e-6


def test_conv3d_vs_torch():
    rng = np.random.default_rng(6)
    x = rng.standard_normal((1, 4, 9, 8, 7)).astype(np.float32)
    w = rng.standard_normal((6, 4, 3, 3, 3)).astype(np.float32)
    y = O.conv3d(x, w, pad=(1, 1, 1))
    ref = TF.conv3d(torch.tensor(x), torch.tensor(w), padding=1).numpy()
    assert maxrel(y, ref) < 2e-6


@pytest.mark.parametrize("k,stride,pad,opad", [(3, 2, 1, 1), (3, 1, 1, 0), (2, 2, 0, 0)])
def test_convt2d_vs_torch(k, stride, pad, opad):
    # tests/optest.py:9-12: ConvTranspose2d(C, C, 3, stride=2, padding=1, output_padding=1) and stride 1
    rng = np.random.default_rng(7)
    x = rng.standard_normal((4, 16, 16)).astype(np.float32)
    w = rng.standard_normal((4, 6, k, k)).astype(np.float32)
    y = O.convt2d(x, w, stride, pad, opad)
    ref = TF.conv_transpose2d(torch.tensor(x)[None], torch.tensor(w), stride=stride, padding=pad, output_padding=opad)[0].numpy()
    assert y.shape == ref.shape and maxrel(y, ref) < 2e-6


def test_pool_upsample_bn_vs_torch():
    rng = np.random.default_rng(8)
    x = rng.standard_normal((4, 16, 16)).astype(np.float32)
    assert np.array_equal(O.maxpool2d(x, 2), TF.max_pool2d(torch.tensor(x)[None], 2)[0].numpy())
    assert np.array_equal(O.upsample_nearest(x, 2), TF.interpolate(torch.tensor(x)[None], scale_factor=2, mode="nearest")[0].numpy())
    x3 = rng.standard_normal((3, 5, 6, 7)).astype(np.float32)
    assert np.array_equal(O.upsample_nearest(x3, 2), TF.interpolate(torch.tensor(x3)[None], scale_factor=2, mode="nearest")[0].numpy())
    # tests/optest.py:27: mean U(-1,1), var U(0.5,2), weight U(0.5,1.5), bias U(-1,1)
    mean, var = rng.uniform(-1, 1, 4).astype(np.float32), rng.uniform(0.5, 2, 4).astype(np.float32)
    g, b = rng.uniform(0.5, 1.5, 4).astype(np.float32), rng.uniform(-1, 1, 4).astype(np.float32)
    ref = TF.batch_norm(torch.tensor(x)[None], torch.tensor(mean), torch.tensor(var), torch.tensor(g), torch.tensor(b), False, 0.0, 1e-5)[0].numpy()
    assert maxrel(O.bn_eval(x, mean, var, g, b), ref) < 1e-6


def test_gemm_vs_numpy():
    rng = np.random.default_rng(9)
    A = rng.standard_normal((37, 53)).astype(np.float32)
    W = rng.standard_normal((29, 53)).astype(np.float32)
    assert maxrel(O.gemm(A, W), A.astype(np.float64) @ W.astype(np.float64).T) < 1e-6


def test_mlp_f64_vs_torch_leaky_and_mask():
    rng = np.random.default_rng(10)
    Ws = [rng.standard_normal((16, 12)).astype(np.float32), rng.standard_normal((8, 16)).astype(np.float32)]
    bs = [rng.standard_normal(16).astype(np.float32), rng.standard_normal(8).astype(np.float32)]
    X = rng.standard_normal((9, 12)).astype(np.float32)
    h = TF.leaky_relu(torch.tensor(X) @ torch.tensor(Ws[0]).T + torch.tensor(bs[0]), 0.15)
    y = h @ torch.tensor(Ws[1]).T + torch.tensor(bs[1])
    mask = torch.zeros(8)
    mask[5:] = 1.0
    y = y + mask * (torch.relu(y) - y)            # benchmarks/climsim/export_wide.py:28
    got = O.mlp_f64(Ws, bs, ["leaky", "none"], X, alphas=[0.15, 0.0], mask_tail=3)
    assert maxrel(got, y.numpy()) < 1e-6


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_boundary_closed_form_and_round_trip(dtype):
    """pre: X[i][k] = (float)((A[i + NI k] - mean[k]) / (max[k] - min[k])); post: B[i + NI k] = (H)Y[i][k] / scale[k]
    (trt_backend/e3sm_boundary.cu:11-13, 17-19).  With mean 0, range 1, scale 1 the pair is a transpose round trip."""
    rng = np.random.default_rng(11)
    NI, NK = 19, 7
    A = np.asfortranarray(rng.standard_normal((NI, NK)).astype(dtype))
    mean, vmax, vmin = [rng.uniform(0.5, 1.5, NK).astype(dtype) * s for s in (0.1, 3.0, 1.0)]
    X = O.boundary_pre(A, mean, vmax, vmin)
    assert np.array_equal(X, ((A - mean[None]) / (vmax - vmin)[None]).astype(np.float32))
    scale = rng.uniform(0.5, 2, NK).astype(dtype)
    B = O.boundary_post(X, scale, dtype)
    assert B.flags.f_contiguous and np.array_equal(B, X.astype(dtype) / scale[None])
    ident = O.boundary_post(O.boundary_pre(A, np.zeros(NK, dtype), np.ones(NK, dtype), np.zeros(NK, dtype)), np.ones(NK, dtype), dtype)
    assert np.array_equal(ident, A.astype(np.float32).astype(dtype))
