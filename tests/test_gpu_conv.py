"""Convolution family on the GPU through the C ABI: conv2d / conv3d / transposed conv / maxpool /
upsample / concat / folded BatchNorm against the CPU oracle, the reference's op micro-suite models
(tests/optest.py) against PyTorch CPU eval, the memref-expanded entries, and configs 4 and 5."""
import ctypes as C

import numpy as np
import pytest
import torch

from fortis_amd import configs, plan as P
from oracle import oracle as O
from refmodels import tsrgan_ref, unet_ref
from util import TOL, DevBuf, bits_equal, maxrel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("C_,H,W,F,k,stride,pad", [(1, 16, 16, 4, 3, 1, 1), (5, 17, 13, 7, 3, 1, 1), (8, 32, 32, 16, 3, 2, 1),
                                                    (32, 20, 24, 4, 1, 1, 0), (3, 9, 9, 9, 5, 1, 2), (64, 16, 16, 64, 3, 1, 1),
                                                    # matrix-core path: channel counts that end in a partial staged chunk, a partial
                                                    # output-channel group, ragged image sizes, an image wide enough for the
                                                    # 16-round staging variant, and the single-tap form with its 16-channel chunks
                                                    (6, 40, 36, 48, 3, 1, 1), (37, 70, 50, 16, 3, 1, 1), (20, 300, 260, 32, 3, 1, 1),
                                                    (50, 33, 47, 40, 1, 1, 0), (130, 12, 12, 70, 3, 1, 1),
                                                    # the 32-column tiling of wide images: ragged height, widths of one tile, of
                                                    # whole tiles and with a mostly filled last tile, both channel-group widths
                                                    (9, 45, 32, 24, 3, 1, 1), (16, 37, 96, 64, 3, 1, 1), (5, 130, 124, 33, 3, 1, 1),
                                                    # few output tiles and at least 32 input channels: 32 x 32 tiles whose four waves
                                                    # share the input channels (sums meet in LDS); partial last chunk of 16 (3 x 3) and
                                                    # of 64 (1 x 1) channels, partial channel group, ragged height, a single tile
                                                    (40, 33, 64, 72, 3, 1, 1), (96, 20, 60, 32, 3, 1, 1), (32, 32, 32, 256, 3, 1, 1),
                                                    (100, 16, 16, 48, 1, 1, 0), (64, 1, 32, 32, 1, 1, 0),
                                                    # between one and five 64 x 64 tiles per CU: 64 x 32 tiles whose waves share the input
                                                    # channels in two groups; two groups of output channels with a partial one, a
                                                    # partial last chunk of 8 channels, ragged width and height
                                                    (44, 130, 126, 72, 3, 1, 1), (32, 128, 128, 64, 3, 1, 1),
                                                    # the same form on a single tap (chunks of 32 channels, a partial last one)
                                                    (48, 130, 127, 40, 1, 1, 0)])
def test_conv2d_bias_act_vs_oracle(L, gpu, C_, H, W, F, k, stride, pad):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((C_, H, W)).astype(np.float32)
    w = (rng.standard_normal((F, C_, k, k)) / np.sqrt(C_ * k * k)).astype(np.float32)
    b = rng.standard_normal(F).astype(np.float32)
    ref = O.conv2d(x[None], w, (stride, stride), (pad, pad))[0] + b[:, None, None]
    ref = np.where(ref > 0, ref, np.float32(0.1) * ref)
    p = P.Plan()
    t0, t1 = p.tensor(x.size), p.tensor(ref.size)
    p.conv2d(t0, t1, w, b, C_, H, W, stride, pad, "leaky", 0.1)
    p.finalize(t0, t1)
    assert maxrel(p.forward(x, ref.shape), ref) < TOL
    p.close()


@pytest.mark.parametrize("C_,H,W,F", [(16, 38, 64, 24), (8, 130, 96, 40), (48, 12, 32, 64), (44, 130, 126, 72), (32, 128, 160, 32)])
def test_conv2d_with_max_pool_behind(L, gpu, C_, H, W, F):
    """3 x 3 conv + bias + ReLU followed by a 2 x 2 max pool: the conv pools its own tiles (32-column tiling, even tile
    height; ragged last tile rows; the last two shapes in the form whose waves share the input channels in two groups), or
    its channel-split reduce kernel does (the small, deep case).  Both outputs checked."""
    rng = np.random.default_rng(11)
    x = rng.standard_normal((C_, H, W)).astype(np.float32)
    w = (rng.standard_normal((F, C_, 3, 3)) / np.sqrt(C_ * 9)).astype(np.float32)
    b = rng.standard_normal(F).astype(np.float32)
    ref = np.maximum(O.conv2d(x[None], w, (1, 1), (1, 1))[0] + b[:, None, None], 0)
    pooled = ref.reshape(F, H // 2, 2, W // 2, 2).max(axis=(2, 4))
    p = P.Plan()
    t0, t1, t2 = p.tensor(x.size), p.tensor(ref.size), p.tensor(pooled.size)
    p.conv2d(t0, t1, w, b, C_, H, W, 1, 1, "relu", 0.0)
    p.maxpool2d(t1, t2, F, H, W, 2)
    p.finalize(t0, t2)
    got_pool = p.forward(x, pooled.shape)
    got_full = p.read(t1, ref.shape)
    assert maxrel(got_full, ref) < TOL
    # the pool of the kernel's own full-resolution output, bit for bit
    assert np.array_equal(got_pool, got_full.reshape(F, H // 2, 2, W // 2, 2).max(axis=(2, 4)))
    p.close()


@pytest.mark.parametrize("C_,H,W,F", [(72, 12, 20, 24), (40, 127, 130, 24)])
def test_convt2d_channel_groups_vs_oracle(L, gpu, C_, H, W, F):
    """2 x 2 stride-2 transposed conv on a small, deep image (the UNet's first up-convolution in small) and on a mid-sized
    one: the kernel forms whose waves share the input channels in four and in two groups, with bias and ReLU, written
    into a channel range of a wider tensor."""
    rng = np.random.default_rng(4)
    x = rng.standard_normal((C_, H, W)).astype(np.float32)
    w = (rng.standard_normal((C_, F, 2, 2)) / np.sqrt(C_)).astype(np.float32)
    b = rng.standard_normal(F).astype(np.float32)
    ref = np.maximum(O.convt2d(x, w, 2, 0) + b[:, None, None], 0)
    p = P.Plan()
    t0, t1 = p.tensor(x.size), p.tensor(2 * ref.size)
    p.convt2d(t0, t1, w, b, C_, H, W, 2, 0, 0, "relu", 0.0, coff=F, ctot=2 * F)
    p.finalize(t0, t1)
    got = p.forward(x, (2 * F, 2 * H, 2 * W))
    assert maxrel(got[F:], ref) < TOL
    p.close()


def _zramp(n):
    x = torch.arange(1, n + 1, dtype=torch.float32) / n
    return (x - x.mean()) / x.std(unbiased=False)


def test_op_micro_suite(L, gpu):
    """The models of tests/optest.py:6-24 (C=4, H=16, seed 5, z-scored ramp input): maxpool, upsample,
    convT (stride 2, pad 1, output_padding 1), convT_s1, convT_only, bn, two_convs, concat, cat_only."""
    torch.manual_seed(5)
    Cc, H = 4, 16
    nn = torch.nn
    models = {
        "maxpool": nn.Sequential(nn.Conv2d(1, Cc, 3, padding=1), nn.MaxPool2d(2)),
        "upsample": nn.Sequential(nn.Conv2d(1, Cc, 3, padding=1), nn.Upsample(scale_factor=2, mode="nearest")),
        "convT": nn.Sequential(nn.Conv2d(1, Cc, 3, padding=1), nn.ConvTranspose2d(Cc, Cc, 3, stride=2, padding=1, output_padding=1)),
        "bn": nn.Sequential(nn.Conv2d(1, Cc, 3, padding=1), nn.BatchNorm2d(Cc)),
        "convT_s1": nn.Sequential(nn.Conv2d(1, Cc, 3, padding=1), nn.ConvTranspose2d(Cc, Cc, 3, padding=1)),
        "convT_only": nn.Sequential(nn.ConvTranspose2d(1, Cc, 3, padding=1)),
        "two_convs": nn.Sequential(nn.Conv2d(1, Cc, 3, padding=1), nn.Conv2d(Cc, Cc, 3, padding=1)),
    }
    a, b, c = nn.Conv2d(1, Cc, 3, padding=1), nn.Conv2d(1, Cc, 3, padding=1), nn.Conv2d(2 * Cc, Cc, 1)
    bn = models["bn"][1]
    bn.running_mean.uniform_(-1, 1); bn.running_var.uniform_(0.5, 2); bn.weight.data.uniform_(0.5, 1.5); bn.bias.data.uniform_(-1, 1)
    x = _zramp(H * H).view(1, 1, H, H)
    xn = x.numpy()[0]
    g = lambda t: t.detach().numpy()
    for name, m in models.items():
        m.eval()
        with torch.no_grad():
            ref = m(x)[0].numpy()
        p = P.Plan()
        t0 = p.tensor(H * H)
        if name == "convT_only":
            t1 = p.tensor(ref.size)
            p.convt2d(t0, t1, g(m[0].weight), g(m[0].bias), 1, H, H, 1, 1, 0)
        else:
            t1 = p.tensor(Cc * H * H)
            if name == "bn":
                p.conv2d(t0, t1, g(m[0].weight), g(m[0].bias), 1, H, H, 1, 1, None, 0.0,
                         (g(bn.weight), g(bn.bias), g(bn.running_mean), g(bn.running_var)), bn.eps)
            else:
                p.conv2d(t0, t1, g(m[0].weight), g(m[0].bias), 1, H, H, 1, 1)
            if name != "bn":
                t2 = p.tensor(ref.size)
                if name == "maxpool":
                    p.maxpool2d(t1, t2, Cc, H, H, 2)
                elif name == "upsample":
                    p.upsample(t1, t2, Cc, 1, H, H, 2, 2)
                elif name == "convT":
                    p.convt2d(t1, t2, g(m[1].weight), g(m[1].bias), Cc, H, H, 2, 1, 1)
                elif name == "convT_s1":
                    p.convt2d(t1, t2, g(m[1].weight), g(m[1].bias), Cc, H, H, 1, 1, 0)
                elif name == "two_convs":
                    p.conv2d(t1, t2, g(m[1].weight), g(m[1].bias), Cc, H, H, 1, 1)
                t1 = t2
        p.finalize(t0, t1)
        y = p.forward(xn, ref.shape)
        assert maxrel(y, ref) < TOL, name
        assert abs(float(y.sum(dtype=np.float64)) - float(ref.sum(dtype=np.float64))) < 1e-5 * np.abs(ref).sum(), name
        p.close()
    # concat: cat([a(x), b(x)]) -> 1x1 conv, both as channel-offset writes and as concat-by-copy; cat_only
    with torch.no_grad():
        cat_ref = torch.cat([a(x), b(x)], dim=1)
        ref = c(cat_ref)[0].numpy()
    for mode in ("offset", "view", "copy"):
        p = P.Plan()
        t0, tcat, tout = p.tensor(H * H), p.tensor(2 * Cc * H * H), p.tensor(Cc * H * H)
        if mode == "offset":
            p.conv2d(t0, tcat, g(a.weight), g(a.bias), 1, H, H, 1, 1, coff=0, ctot=2 * Cc)
            p.conv2d(t0, tcat, g(b.weight), g(b.bias), 1, H, H, 1, 1, coff=Cc, ctot=2 * Cc)
        elif mode == "view":
            p.conv2d(t0, p.view(tcat, 0, Cc * H * H), g(a.weight), g(a.bias), 1, H, H, 1, 1)
            p.conv2d(t0, p.view(tcat, Cc * H * H, Cc * H * H), g(b.weight), g(b.bias), 1, H, H, 1, 1)
        else:
            ta, tb = p.tensor(Cc * H * H), p.tensor(Cc * H * H)
            p.conv2d(t0, ta, g(a.weight), g(a.bias), 1, H, H, 1, 1)
            p.conv2d(t0, tb, g(b.weight), g(b.bias), 1, H, H, 1, 1)
            p.concat_copy(ta, tcat, Cc, H * H, 0, 2 * Cc)
            p.concat_copy(tb, tcat, Cc, H * H, Cc, 2 * Cc)
        p.conv2d(tcat, tout, g(c.weight), g(c.bias), 2 * Cc, H, H, 1, 0)
        p.finalize(t0, tout)
        assert maxrel(p.forward(xn, ref.shape), ref) < TOL, mode
        assert maxrel(p.read(tcat, (2 * Cc, H, H)), cat_ref[0].numpy()) < TOL, mode      # cat_only
        p.close()


@pytest.mark.parametrize("C_,D,H,W,F,k,pad", [(3, 16, 16, 16, 8, 3, 1), (4, 9, 8, 7, 6, 3, 1), (2, 7, 7, 7, 3, 5, 2),
                                               (64, 9, 9, 9, 64, 3, 1), (5, 6, 6, 6, 10, 1, 0), (3, 8, 8, 8, 4, 3, 0),
                                               # matrix-core path: odd channel count (partial 2-channel chunk), ragged extents,
                                               # a partial output-channel group; a volume whose rows need the 16-round staging
                                               (7, 12, 11, 10, 20, 3, 1), (6, 5, 90, 70, 80, 3, 1),
                                               # image-space heads (at most 4 output channels) whose input channels are split
                                               # over workgroups: even slices, and an odd channel count with a shorter last slice
                                               (32, 8, 20, 20, 3, 3, 1), (17, 6, 10, 12, 4, 3, 1), (64, 5, 30, 33, 1, 3, 1),
                                               # streamed split (equal runs of (tile, chunk) items, partial sums per tile and run):
                                               # two groups of output channels and ragged tiles; an odd chunk count
                                               (64, 12, 20, 19, 128, 3, 1), (46, 10, 17, 23, 64, 3, 1),
                                               # more tiles than are resident at once: whole rounds in one launch, the 26 tiles
                                               # of the last round streamed
                                               (32, 21, 80, 79, 64, 3, 1)])
def test_conv3d_bias_act_residual_vs_oracle(L, gpu, C_, D, H, W, F, k, pad):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((C_, D, H, W)).astype(np.float32)
    w = (rng.standard_normal((F, C_, k, k, k)) / np.sqrt(C_ * k ** 3)).astype(np.float32)
    b = rng.standard_normal(F).astype(np.float32)
    ref = O.conv3d(x[None], w, pad=(pad,) * 3)[0] + b[:, None, None, None]
    ref = np.maximum(ref, 0)
    res = rng.standard_normal(ref.shape).astype(np.float32)
    p = P.Plan()
    t0, t1, tr = p.tensor(x.size), p.tensor(ref.size), p.tensor(ref.size)
    p.conv3d(t0, t1, w, b, C_, D, H, W, pad, "relu", 0.0, res=tr)
    p.finalize(t0, t1)
    p.write(tr, res)
    assert maxrel(p.forward(x, ref.shape), ref + res) < TOL
    p.close()


def test_conv_probe_readme_stamp_through_plan(L, gpu):
    """README.md:25 conv probe 9617.28: Conv3d(3,8,3,pad 1) + LeakyReLU(0.1), seed 3, z-scored ramp
    (frontend/export_conv.py:3-9, benchmarks/toy/bench_fortis_conv.f90).  The exact sum of the correct outputs is
    9617.4091: the six-digit stamp itself is 1.34e-5 away from it (observed here: 1.34e-5), hence the 3e-5 bound on the
    stamp; the outputs themselves are held to torch element-wise below."""
    torch.manual_seed(3)
    m = torch.nn.Sequential(torch.nn.Conv3d(3, 8, 3, padding=1), torch.nn.LeakyReLU(0.1)).eval()
    x = _zramp(3 * 16 ** 3).view(1, 3, 16, 16, 16)
    p = P.Plan()
    t0, t1 = p.tensor(3 * 16 ** 3), p.tensor(8 * 16 ** 3)
    p.conv3d(t0, t1, m[0].weight.detach().numpy(), m[0].bias.detach().numpy(), 3, 16, 16, 16, 1, "leaky", 0.1)
    p.finalize(t0, t1)
    y = p.forward(x.numpy()[0], (8, 16, 16, 16))
    assert abs(float(y.sum(dtype=np.float64)) - 9617.28) / 9617.28 < 3e-5
    with torch.no_grad():
        assert maxrel(y, m(x)[0].numpy()) < TOL
    p.close()


def _memref(buf, shape):
    strides = [1]
    for d in reversed(shape[1:]):
        strides.insert(0, strides[0] * d)
    return [buf.ptr, buf.ptr, 0] + list(shape) + strides


def test_memref_conv_entries(L, gpu, capfd):
    """fortis_conv2d / fortis_conv3d / fortis_conv3d_direct / fortis_conv3d_fft with the argument order of
    compiler/FortisFuse.cpp:642-648 (N, C, in-spatial, F, kernel, out-spatial, strides, pads)."""
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 3, 10, 12)).astype(np.float32)
    w = rng.standard_normal((5, 3, 3, 3)).astype(np.float32)
    ref = O.conv2d(x, w, (2, 1), (1, 1))
    dx, dw, dy = DevBuf(L, x), DevBuf(L, w), DevBuf(L, nbytes=ref.nbytes)
    L.fortis_conv2d(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy, ref.shape),
                    2, 3, 10, 12, 5, 3, 3, ref.shape[2], ref.shape[3], 2, 1, 1, 1)
    assert maxrel(dy.get(ref.shape), ref) < TOL
    x3 = rng.standard_normal((1, 3, 8, 9, 10)).astype(np.float32)
    w3 = rng.standard_normal((4, 3, 3, 3, 3)).astype(np.float32)
    ref3 = O.conv3d(x3, w3, pad=(1, 1, 1))
    dx3, dw3, dy3 = DevBuf(L, x3), DevBuf(L, w3), DevBuf(L, nbytes=ref3.nbytes)
    tail = [1, 3, 8, 9, 10, 4, 3, 3, 3, 8, 9, 10, 1, 1, 1, 1, 1, 1]
    for fn in (L.fortis_conv3d, L.fortis_conv3d_direct):
        L.fortis_d2d(dy3.ptr, dx3.ptr, 16)                                       # dirty the output first
        fn(*_memref(dx3, x3.shape), *_memref(dw3, w3.shape), *_memref(dy3, ref3.shape), *tail)
        assert maxrel(dy3.get(ref3.shape), ref3) < TOL
    # large-kernel entry: 5^3 kernel, pad 0 (the shape class fortis-fuse routes there, FortisFuse.cpp:651-652)
    w5 = rng.standard_normal((2, 3, 5, 5, 5)).astype(np.float32)
    ref5 = O.conv3d(x3, w5)
    dw5, dy5 = DevBuf(L, w5), DevBuf(L, nbytes=ref5.nbytes)
    L.fortis_conv3d_fft(*_memref(dx3, x3.shape), *_memref(dw5, w5.shape), *_memref(dy5, ref5.shape),
                        1, 3, 8, 9, 10, 2, 5, 5, 5, 4, 5, 6, 1, 1, 1, 0, 0, 0)
    assert maxrel(dy5.get(ref5.shape), ref5) < TOL
    capfd.readouterr()
    # shapes the reference rejects print "unsupported shape" and compute nothing (fortis_fft.cu:70, 135)
    L.fortis_conv3d_direct(*_memref(dx3, x3.shape), *_memref(dw3, w3.shape), *_memref(dy3, ref3.shape),
                           *(tail[:12] + [2, 1, 1, 1, 1, 1]))
    L.fortis_conv3d_fft(*_memref(dx3, x3.shape), *_memref(dw3, w3.shape), *_memref(dy3, ref3.shape), *tail)
    L.fortis_sync()
    assert capfd.readouterr().err.count("unsupported shape") == 2
    for d in (dx, dw, dy, dx3, dw3, dy3, dw5, dy5):
        d.free()


def test_memref_conv_entries_wide_shapes(L, gpu):
    """The runtime-tier entries on shapes the matrix-core kernel takes (raw weights packed on the device per call):
    a batch of two 3x3 images, a 1x1 conv, a 3x3x3 volume; a second call with other weights in the same buffer
    must use them (nothing is cached by pointer)."""
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 24, 40, 36)).astype(np.float32)
    for k in (3, 1):
        w = (rng.standard_normal((48, 24, k, k)) / np.sqrt(24 * k * k)).astype(np.float32)
        ref = O.conv2d(x, w, (1, 1), (k // 2, k // 2))
        dx, dw, dy = DevBuf(L, x), DevBuf(L, w), DevBuf(L, nbytes=ref.nbytes)
        args = [2, 24, 40, 36, 48, k, k, 40, 36, 1, 1, k // 2, k // 2]
        L.fortis_conv2d(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy, ref.shape), *args)
        assert maxrel(dy.get(ref.shape), ref) < TOL
        w2 = (rng.standard_normal(w.shape) / np.sqrt(24 * k * k)).astype(np.float32)
        L.fortis_h2d(dw.ptr, w2.ctypes.data, w2.nbytes)
        L.fortis_conv2d(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy, ref.shape), *args)
        assert maxrel(dy.get(ref.shape), O.conv2d(x, w2, (1, 1), (k // 2, k // 2))) < TOL
        for d in (dx, dw, dy):
            d.free()
    # few output tiles, 40 input channels: the form whose waves share the input channels, weights packed for it per call
    x = rng.standard_normal((1, 40, 20, 64)).astype(np.float32)
    for k in (3, 1):
        w = (rng.standard_normal((48, 40, k, k)) / np.sqrt(40 * k * k)).astype(np.float32)
        ref = O.conv2d(x, w, (1, 1), (k // 2, k // 2))
        dx, dw, dy = DevBuf(L, x), DevBuf(L, w), DevBuf(L, nbytes=ref.nbytes)
        L.fortis_conv2d(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy, ref.shape), 1, 40, 20, 64, 48, k, k, 20, 64, 1, 1, k // 2, k // 2)
        assert maxrel(dy.get(ref.shape), ref) < TOL
        for d in (dx, dw, dy):
            d.free()
    x3 = rng.standard_normal((1, 10, 9, 14, 11)).astype(np.float32)
    w3 = (rng.standard_normal((20, 10, 3, 3, 3)) / np.sqrt(270)).astype(np.float32)
    ref3 = O.conv3d(x3, w3, pad=(1, 1, 1))
    dx3, dw3, dy3 = DevBuf(L, x3), DevBuf(L, w3), DevBuf(L, nbytes=ref3.nbytes)
    tail = [1, 10, 9, 14, 11, 20, 3, 3, 3, 9, 14, 11, 1, 1, 1, 1, 1, 1]
    for fn in (L.fortis_conv3d, L.fortis_conv3d_direct):
        L.fortis_d2d(dy3.ptr, dx3.ptr, 16)
        fn(*_memref(dx3, x3.shape), *_memref(dw3, w3.shape), *_memref(dy3, ref3.shape), *tail)
        assert maxrel(dy3.get(ref3.shape), ref3) < TOL
    for d in (dx3, dw3, dy3):
        d.free()


@pytest.mark.parametrize("stride,pad,F,K", [((2, 1, 2), (1, 1, 1), 20, 3), ((2, 2, 2), (0, 1, 0), 5, 3), ((1, 3, 2), (1, 0, 1), 4, (3, 1, 2))])
def test_fortis_conv3d_strided_batches(L, gpu, stride, pad, F, K):
    """fortis_conv3d takes what the reference's library path takes (runtime/fortis_rt.c:137-155: the Nd descriptor
    carries any stride and batch): N = 2 with strides other than 1, wide and thin outputs, against the oracle."""
    rng = np.random.default_rng(31)
    K = (K, K, K) if isinstance(K, int) else K
    x = rng.standard_normal((2, 6, 9, 11, 12)).astype(np.float32)
    w = (rng.standard_normal((F, 6) + K) / np.sqrt(6 * K[0] * K[1] * K[2])).astype(np.float32)
    ref = O.conv3d(x, w, stride=stride, pad=pad)
    assert ref.shape[0] == 2 and min(ref.shape) > 0
    dx, dw, dy = DevBuf(L, x), DevBuf(L, w), DevBuf(L, np.full(ref.shape, 9, np.float32))
    L.fortis_conv3d(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy, ref.shape),
                    2, 6, 9, 11, 12, F, *K, *ref.shape[2:], *stride, *pad)
    assert maxrel(dy.get(ref.shape), ref) < TOL
    for d in (dx, dw, dy):
        d.free()


@pytest.mark.parametrize("H,chans", [(32, (8, 16, 24, 32)), (256, (32, 64, 128, 256))])
def test_config4_unet(L, gpu, H, chans):
    case = configs.unet(H=H, chans=chans)
    plan = configs.unet_plan(case)
    y = plan.forward(case["x"], (case["cout"], H, H))
    assert maxrel(y, unet_ref(case)) < TOL
    plan.close()


@pytest.mark.parametrize("D,ch,nblocks", [(9, 16, 2), (33, 64, 8)])
def test_config5_tsrgan(L, gpu, D, ch, nblocks):
    case = configs.tsrgan(D=D, ch=ch, nblocks=nblocks)
    plan = configs.tsrgan_plan(case)
    y = plan.forward(case["x"], (2 * D, 2 * D, 2 * D, case["cout"]))
    assert maxrel(y, tsrgan_ref(case)) < TOL
    plan.close()


@pytest.mark.parametrize("C_,S", [(3, 35937), (3, 100), (5, 1000), (8, 256), (12, 4096), (64, 7)])
def test_permute_channels_last_and_back_bit_exact(L, gpu, C_, S):
    """Channels-last <-> channels-first copies (the TSRGAN step's first and last operation: NDHWC <-> NCDHW), with few
    channels (a thread per position), few positions and the tiled form: a permutation of the same bits."""
    x = np.random.default_rng(C_ * 1000 + S).standard_normal((S, C_)).astype(np.float32)
    for first in (True, False):
        src = x if first else np.ascontiguousarray(x.T)          # [S][C] -> [C][S], or back
        p = P.Plan()
        t0, t1 = p.tensor(src.size), p.tensor(src.size)
        p.permute(t0, t1, C_, S, first)
        p.finalize(t0, t1)
        got = p.forward(src, src.T.shape)
        p.close()
        assert np.array_equal(got.view(np.uint32), np.ascontiguousarray(src.T).view(np.uint32))


@pytest.mark.parametrize("H,W,C_,F,NH", [(128, 128, 64, 32, 4), (128, 160, 48, 24, 3), (256, 256, 32, 32, 1)])
def test_thin_1x1_head_folded_into_the_conv_before_it(L, gpu, monkeypatch, H, W, C_, F, NH):
    """conv 3 x 3 + BN + ReLU followed by a 1 x 1 conv to a few channels (the UNet's last two layers): the plan lets the
    3 x 3 kernel write the head from its finished tiles (one kernel, the wide tensor never stored); same result as the
    two launches (FORTIS_NO_HEAD_FOLD) within the tolerance, and against the oracle."""
    rng = np.random.default_rng(41)
    x = rng.standard_normal((C_, H, W)).astype(np.float32)
    w1 = (rng.standard_normal((F, C_, 3, 3)) / np.sqrt(9 * C_)).astype(np.float32)
    b1 = rng.standard_normal(F).astype(np.float32)
    bn = [rng.uniform(0.5, 1.5, F).astype(np.float32), rng.standard_normal(F).astype(np.float32) * np.float32(0.1),
          rng.standard_normal(F).astype(np.float32) * np.float32(0.1), rng.uniform(0.5, 1.5, F).astype(np.float32)]
    w2 = (rng.standard_normal((NH, F, 1, 1)) / np.sqrt(F)).astype(np.float32)
    b2 = rng.standard_normal(NH).astype(np.float32)
    outs = []
    for fold in (True, False):
        if not fold:
            monkeypatch.setenv("FORTIS_NO_HEAD_FOLD", "1")
        p = P.Plan()
        t0, t1, t2 = p.tensor(C_ * H * W), p.tensor(F * H * W), p.tensor(NH * H * W)
        p.conv2d(t0, t1, w1, b1, C_, H, W, 1, 1, "relu", 0.0, bn, 1e-5)
        p.conv2d(t1, t2, w2, b2, F, H, W, 1, 0, None, 0.0)
        p.finalize(t0, t2)
        assert p.num_kernels == (1 if fold else 2)
        outs.append(p.forward(x, (NH, H, W)))
        outs.append(p.forward(x, (NH, H, W)))
        assert bits_equal(outs[-1], outs[-2])
        p.close()
    mid = O.conv2d(x[None], w1, (1, 1), (1, 1))[0]
    sc = (bn[0].astype(np.float64) / np.sqrt(bn[3].astype(np.float64) + 1e-5))
    mid = np.maximum((mid.astype(np.float64) + b1[:, None, None] - bn[2][:, None, None]) * sc[:, None, None] + bn[1][:, None, None], 0).astype(np.float32)
    ref = O.conv2d(mid[None], w2, (1, 1), (0, 0))[0] + b2[:, None, None]
    assert maxrel(outs[0], ref) < TOL and maxrel(outs[2], ref) < TOL and maxrel(outs[0], outs[2]) < TOL
