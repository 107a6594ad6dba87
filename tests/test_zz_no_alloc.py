"""fortis_conv3d_noalloc: the conv3d entry for callers that cannot allocate (its packed weights and partial sums
live in a fixed device array of the library), through the C ABI against fortis_conv3d on the same inputs."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O
from util import TOL, DevBuf, bits_equal, maxrel

pytestmark = pytest.mark.gpu


def _memref(buf, shape):
    strides = [1]
    for d in reversed(shape[1:]):
        strides.insert(0, strides[0] * d)
    return [buf.ptr, buf.ptr, 0] + list(shape) + strides


def _both(L, x, w, check_oracle):
    N, Cc, D, H, W = x.shape
    F = w.shape[0]
    dx, dw = DevBuf(L, x), DevBuf(L, w)
    dy0, dy1 = DevBuf(L, np.full((N, F, D, H, W), 7, np.float32)), DevBuf(L, np.full((N, F, D, H, W), -7, np.float32))
    tail = [N, Cc, D, H, W, F, 3, 3, 3, D, H, W, 1, 1, 1, 1, 1, 1]
    L.fortis_conv3d(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy0, (N, F, D, H, W)), *tail)
    rc = L.fortis_conv3d_noalloc(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy1, (N, F, D, H, W)), *tail)
    L.fortis_sync()
    y0, y1 = dy0.get((N, F, D, H, W)), dy1.get((N, F, D, H, W))
    for d in (dx, dw, dy0, dy1):
        d.free()
    assert rc == 0
    assert bits_equal(y0, y1)
    if check_oracle:
        assert maxrel(y1, O.conv3d(x, w, pad=(1, 1, 1))) < TOL
    return y1


def test_noalloc_entry_equals_the_allocating_entry_on_two_calls_in_a_row(L, gpu):
    """Two calls in a row, the second on a smaller input, so that the second finds the first call's packed
    weights and partial sums in the scratch array: 64 -> 64 channels on small volumes splits its input channels
    over workgroups (partial sums in scratch), and both calls pack their weights into it."""
    rng = np.random.default_rng(21)
    shapes = [((1, 64, 16, 18, 20), 64), ((1, 64, 9, 10, 11), 64),      # matrix-core launches with partial sums in scratch
              ((2, 32, 8, 20, 20), 3), ((1, 17, 6, 10, 12), 4),           # thin heads: split on the vector kernel, batch of 2
              ((1, 10, 9, 14, 11), 20)]                                   # no split: only the packed weights use scratch
    for (xs, F) in shapes:
        x = rng.standard_normal(xs).astype(np.float32)
        w = (rng.standard_normal((F, xs[1], 3, 3, 3)) / np.sqrt(27 * xs[1])).astype(np.float32)
        _both(L, x, w, check_oracle=True)


def test_noalloc_entry_asks_the_device_for_no_memory(L, gpu):
    """The entry's defining property: on shapes this process has not run before (larger than any above, so the
    allocating twins would have to grow their buffers when this file runs alone), called before the allocating entry,
    the count of raw device allocations the library has made does not move."""
    rng = np.random.default_rng(23)
    for (xs, F) in [((1, 64, 17, 19, 21), 64), ((1, 48, 10, 22, 26), 3), ((1, 12, 11, 15, 13), 24)]:
        x = rng.standard_normal(xs).astype(np.float32)
        w = (rng.standard_normal((F, xs[1], 3, 3, 3)) / np.sqrt(27 * xs[1])).astype(np.float32)
        N, Cc, D, H, W = xs
        ys = (N, F, D, H, W)
        dx, dw, dy = DevBuf(L, x), DevBuf(L, w), DevBuf(L, np.zeros(ys, np.float32))
        tail = [N, Cc, D, H, W, F, 3, 3, 3, D, H, W, 1, 1, 1, 1, 1, 1]
        L.fortis_sync()
        before = L.fortis_dev_alloc_calls()
        rc = L.fortis_conv3d_noalloc(*_memref(dx, xs), *_memref(dw, w.shape), *_memref(dy, ys), *tail)
        L.fortis_sync()
        assert rc == 0 and L.fortis_dev_alloc_calls() == before, (xs, F)
        assert maxrel(dy.get(ys), O.conv3d(x, w, pad=(1, 1, 1))) < TOL
        for d in (dx, dw, dy):
            d.free()
    # the counter is live: every raw allocation of the library (pool, weights, the convolution path's own buffers)
    # goes through the one counted function; a pool request larger than any buffer the pool can hold released (6 GiB)
    # must move it
    before = L.fortis_dev_alloc_calls()
    p = L.fortis_alloc(6 << 30)
    assert p and L.fortis_dev_alloc_calls() == before + 1
    L.fortis_free(p)


def test_noalloc_entry_refuses_what_does_not_fit_its_scratch(L, gpu, capfd):
    """64 -> 64 channels on 27 x 40 x 40 is streamed over the chip in runs of 22 chunks: up to three partial sums for
    each of its 351 tiles of 128 positions x 64 channels are 34.5 MB behind 0.44 MB of packed weights, more than the
    32 MiB array.  The call says so, returns -1 and computes nothing; the allocating entry takes the shape, and the
    next no-alloc call works."""
    rng = np.random.default_rng(22)
    x = rng.standard_normal((1, 64, 27, 40, 40)).astype(np.float32)
    w = (rng.standard_normal((64, 64, 3, 3, 3)) / np.sqrt(27 * 64)).astype(np.float32)
    dx, dw = DevBuf(L, x), DevBuf(L, w)
    ys = (1, 64, 27, 40, 40)
    dy = DevBuf(L, np.full(ys, 3, np.float32))
    tail = [1, 64, 27, 40, 40, 64, 3, 3, 3, 27, 40, 40, 1, 1, 1, 1, 1, 1]
    capfd.readouterr()
    rc = L.fortis_conv3d_noalloc(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy, ys), *tail)
    L.fortis_sync()
    assert rc == -1 and "more than the fixed" in capfd.readouterr().err
    assert (dy.get(ys) == 3).all()
    L.fortis_conv3d(*_memref(dx, x.shape), *_memref(dw, w.shape), *_memref(dy, ys), *tail)
    y = dy.get(ys)
    idx = (0, slice(0, 64, 9), slice(0, 27, 5), slice(0, 40, 7), slice(None))
    assert maxrel(y[idx], O.conv3d(x, w, pad=(1, 1, 1))[idx]) < TOL
    for d in (dx, dw, dy):
        d.free()
    xs = rng.standard_normal((1, 64, 9, 10, 11)).astype(np.float32)
    _both(L, xs, w, check_oracle=True)
