"""Ground-truth evaluations of the conv configurations with torch.nn.functional on the CPU in
float64 (a library routine, not the reference), from the same seeded case dictionaries the GPU
plans are built from."""
import numpy as np
import torch
import torch.nn.functional as TF


_DT = [torch.float64]


def _t(a):
    return torch.tensor(np.asarray(a), dtype=_DT[0])


def _with_dtype(fn):
    def wrapped(case, dtype=torch.float64):
        _DT[0] = dtype
        try:
            with torch.no_grad():
                return fn(case)
        finally:
            _DT[0] = torch.float64
    return wrapped


def _conv_bn_relu(x, cv):
    y = TF.conv2d(x, _t(cv["W"]), _t(cv["b"]), padding=1)
    g, b, m, v = [_t(t) for t in cv["bn"]]
    return torch.relu(TF.batch_norm(y, m, v, g, b, False, 0.0, 1e-5))


@_with_dtype
def unet_ref(case):
    x = _t(case["x"])[None]
    skips = []
    for blk in case["enc"]:
        x = _conv_bn_relu(_conv_bn_relu(x, blk[0]), blk[1])
        skips.append(x)
        x = TF.max_pool2d(x, 2)
    x = _conv_bn_relu(_conv_bn_relu(x, case["bott"][0]), case["bott"][1])
    for d, skip in zip(case["dec"], reversed(skips)):
        up = TF.conv_transpose2d(x, _t(d["up"]["W"]), _t(d["up"]["b"]), stride=2)
        x = torch.cat([skip, up], dim=1)
        x = _conv_bn_relu(_conv_bn_relu(x, d["convs"][0]), d["convs"][1])
    return TF.conv2d(x, _t(case["final"]["W"]), _t(case["final"]["b"]))[0].numpy()


@_with_dtype
def tsrgan_ref(case):
    a = case["alpha"]
    x = _t(case["x"]).permute(3, 0, 1, 2)[None]                      # NDHWC -> NCDHW
    x = TF.leaky_relu(TF.conv3d(x, _t(case["head"]["W"]), _t(case["head"]["b"]), padding=1), a)
    for blk in case["blocks"]:
        h = torch.relu(TF.conv3d(x, _t(blk["W1"]), _t(blk["b1"]), padding=1))
        x = x + TF.conv3d(h, _t(blk["W2"]), _t(blk["b2"]), padding=1)
    x = TF.interpolate(x, scale_factor=2, mode="nearest")
    x = TF.leaky_relu(TF.conv3d(x, _t(case["upc"]["W"]), _t(case["upc"]["b"]), padding=1), a)
    x = TF.conv3d(x, _t(case["tail"]["W"]), _t(case["tail"]["b"]), padding=1)
    return x[0].permute(1, 2, 3, 0).contiguous().numpy()              # back to NDHWC
