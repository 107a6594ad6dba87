"""The five benchmark configurations as seeded synthetic cases (weights, inputs, and the plan).

Seeds follow one convention everywhere (numpy default_rng): weights 0, inputs 1, masks 2, BatchNorm
statistics 3, so the CPU checker, the GPU run and any other implementation see identical bits.
Weights are N(0, 1/fan_in); biases are zero unless stated.  These play the role of the reference's
exporters (frontend/export_mlp.py, mom6_zb/export_zb.py, benchmarks/climsim/export_wide.py) for
shapes no checked-in weight file covers.
"""
import numpy as np

from . import plan as P


def _w(rng, fan_out, fan_in, *k):
    fi = fan_in * int(np.prod(k)) if k else fan_in
    return (rng.standard_normal((fan_out, fan_in) + tuple(k)) / np.sqrt(fi)).astype(np.float32)


# ---------------------------------------------------------------------------------------------
def toy_mlp(rows=1024, widths=(64, 256, 256, 32)):
    """Config 1: X[rows][64] ~ U(-1,1); Linear 64->256 ReLU -> 256->256 ReLU -> 256->32; bias 0."""
    rw, ri = np.random.default_rng(0), np.random.default_rng(1)
    Ws = [_w(rw, widths[i + 1], widths[i]) for i in range(len(widths) - 1)]
    bs = [np.zeros(w.shape[0], np.float32) for w in Ws]
    acts = ["relu"] * (len(Ws) - 1) + [None]
    X = ri.uniform(-1, 1, (rows, widths[0])).astype(np.float32)
    flops = 2 * rows * sum(widths[i] * widths[i + 1] for i in range(len(Ws)))
    nbytes = 4 * (rows * widths[0] + rows * widths[-1] + sum(w.size + b.size for w, b in zip(Ws, bs)))
    return dict(name="toy_mlp", Ws=Ws, bs=bs, acts=acts, X=X, rows=rows, widths=list(widths), flops=flops, bytes=nbytes)


def mlp_case_plan(case):
    return P.mlp_plan(case["Ws"], case["bs"], case["acts"], case["rows"], alphas=case.get("alphas"),
                      in_norms=case.get("in_norms"), out_norms=case.get("out_norms"), mask_tail=case.get("mask_tail", 0))


# ---------------------------------------------------------------------------------------------
def zb_arrays(sx=68, sy=78, nz=15, mask_land=0.0):
    """Three N(0,1) fp32 fields on an (sx, sy, nz) column-major grid, the 3x3 stencil norm, and the
    kappa plane, in Fortran element order (flat).  mask_land > 0 draws a seeded land mask."""
    ri, rm = np.random.default_rng(1), np.random.default_rng(2)
    f = [ri.standard_normal(sx * sy * nz).astype(np.float32) for _ in range(3)]
    mask = np.ones((sy, sx), np.float32)
    mask[0, :] = mask[-1, :] = 0
    mask[:, 0] = mask[:, -1] = 0
    if mask_land > 0:
        mask = mask * (rm.uniform(0, 1, (sy, sx)) >= mask_land).astype(np.float32)
    sq = sum((a.reshape(nz, sy, sx).astype(np.float64)) ** 2 for a in f) * mask[None]
    box = np.zeros_like(sq)
    for dj in (-1, 0, 1):
        for di in (-1, 0, 1):
            box[:, 1:-1, 1:-1] += sq[:, 1 + dj:sy - 1 + dj, 1 + di:sx - 1 + di]
    norm = np.sqrt(box).astype(np.float32).reshape(-1)
    kappa = (-6.25e8 * mask).astype(np.float32).reshape(-1)
    return dict(sh_xy_h=f[0], sh_xx=f[1], vort_xy_h=f[2], norm_h=norm, kappa_h=kappa, mask=mask.reshape(-1))


def zb_descriptors(sx, sy, nz):
    """gather.json / scatter.json / loop.json / kdist.json content for an (sx, sy, nz) grid, in the
    schema of the reference's checked-in ZB descriptors (mom6_zb/gather.json, scatter.json,
    zb_loop_verdict.json, kdist.json), halo 2 around the visited rectangle i=3..sx-2, j=3..sy-2."""
    sh3 = [sx, sy, nz]
    names = ["sh_xy_h", "sh_xx", "vort_xy_h", "norm_h"]
    g = dict(ok=True, n=27, args=[{"name": "k"}],
             arrays=[dict(name=n, shape=sh3, elt="f32") for n in names],
             scalars=[dict(name="S0", array=3, idx=[["i", 0], ["j", 0], ["v", 0]])],
             exprs=["(tv / (S0 + 1.000000e-30f))"],
             slots=[dict(array=a, idx=[["i", di], ["j", dj], ["v", 0]]) for a in range(3) for dj in (-1, 0, 1) for di in (-1, 0, 1)])
    s = dict(ok=True, n=3, args=[{"name": "k"}],
             arrays=[dict(name="norm_h", shape=sh3, elt="f32"), dict(name="kappa_h", shape=[sx, sy], elt="f32"),
                     dict(name="txy_h", shape=[sx, sy], elt="f32"), dict(name="txx", shape=sh3, elt="f32"),
                     dict(name="tyy", shape=sh3, elt="f32")],
             scalars=[dict(name="S0", array=0, idx=[["i", 0], ["j", 0], ["v", 0]]), dict(name="S1", array=1, idx=[["i", 0], ["j", 0]])],
             exprs=["(((tv * S0) * S0) * S1)"],
             stores=[dict(slot=0, array=2, idx=[["i", 0], ["j", 0]]), dict(slot=1, array=3, idx=[["i", 0], ["j", 0], ["v", 0]]),
                     dict(slot=2, array=4, idx=[["i", 0], ["j", 0], ["v", 0]])])
    ni, nj = sx - 4, sy - 4
    loop = dict(verdict="batched", mode="expanded", batch=ni * nj, lo=1, step=1, minc=1,
                inner=dict(lo=3, hi=sx - 2, n=ni), outer=dict(lo=3, hi=sy - 2), in_shape=[27], out_shape=[3])
    kd = dict(ok=True, nk=nz, loop=dict(lo=1, hi=nz))
    return g, s, loop, kd


def zb_mlp(hidden=(64, 64)):
    """Config 2 network: 27 -> 64 -> 64 -> 3, ReLU between, bias 0."""
    rw = np.random.default_rng(0)
    widths = (27,) + tuple(hidden) + (3,)
    Ws = [_w(rw, widths[i + 1], widths[i]) for i in range(len(widths) - 1)]
    bs = [np.zeros(w.shape[0], np.float32) for w in Ws]
    return dict(Ws=Ws, bs=bs, acts=["relu"] * (len(Ws) - 1) + [None], widths=list(widths))


def zb_cells_from_mask(mask, sx, sy, n):
    """The first n ocean cells (column-major order) that have a full 3x3 neighbourhood inside the
    grid: the index list form of config 2's "seeded land mask giving 4736 active points"."""
    m = mask.reshape(sy, sx)
    ok = np.zeros_like(m, dtype=bool)
    ok[1:-1, 1:-1] = m[1:-1, 1:-1] > 0
    cells = np.flatnonzero(ok.reshape(-1)).astype(np.int32)
    if len(cells) < n:
        raise ValueError(f"mask has only {len(cells)} usable ocean cells, {n} wanted")
    return cells[:n]


# ---------------------------------------------------------------------------------------------
def climsim(rows=24576, n_in=556, hidden=768, nhidden=5, n_out=368, alpha=0.15):
    """Config 3: A(rows, n_in) column-major ~ N(0,1) -> X[rows][n_in] (mean 0 / range 1 vectors still
    applied) -> 556 -> 768 x5 LeakyReLU(0.15) -> 368 linear head -> B(rows, n_out) column-major."""
    rw, ri = np.random.default_rng(0), np.random.default_rng(1)
    widths = [n_in] + [hidden] * nhidden + [n_out]
    Ws = [_w(rw, widths[i + 1], widths[i]) for i in range(len(widths) - 1)]
    bs = [np.zeros(w.shape[0], np.float32) for w in Ws]
    acts = ["leaky"] * nhidden + [None]
    alphas = [alpha] * nhidden + [0.0]
    A = np.asfortranarray(ri.standard_normal((rows, n_in)).astype(np.float32))
    mean = np.zeros(n_in, np.float32)
    vmax = np.ones(n_in, np.float32)
    vmin = np.zeros(n_in, np.float32)
    scale = np.ones(n_out, np.float32)
    flops = 2 * rows * sum(widths[i] * widths[i + 1] for i in range(len(Ws)))
    nbytes = 4 * (rows * n_in + rows * n_out + sum(w.size + b.size for w, b in zip(Ws, bs)))
    return dict(name="climsim", Ws=Ws, bs=bs, acts=acts, alphas=alphas, A=A, mean=mean, vmax=vmax, vmin=vmin, scale=scale,
                rows=rows, widths=widths, flops=flops, bytes=nbytes)


def climsim_plan(case, boundary=True):
    """gather (boundary pre) -> GEMM chain -> scatter (boundary post), or the bare chain."""
    rows, widths = case["rows"], case["widths"]
    p = P.Plan()
    if boundary:
        t_in = p.tensor(rows * widths[0])
        cur = p.tensor(rows * widths[0])
        p.boundary_pre(t_in, cur, rows, widths[0], case["mean"], case["vmax"], case["vmin"], np.float32)
    else:
        t_in = cur = p.tensor(rows * widths[0])
    for l, (W, b) in enumerate(zip(case["Ws"], case["bs"])):
        t = p.tensor(rows * widths[l + 1])
        p.linear(cur, t, W, b, rows, case["acts"][l], case["alphas"][l])
        cur = t
    if boundary:
        t = p.tensor(rows * widths[-1])
        p.boundary_post(cur, t, rows, widths[-1], case["scale"], np.float32)
        cur = t
    return p.finalize(t_in, cur)


