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


def climsim_plan(case, boundary=True, plan_cls=None):
    """gather (boundary pre) -> GEMM chain -> scatter (boundary post), or the bare chain.  plan_cls: a class with
    Plan's interface to fill instead (the op-list recorder of fortis_amd.shim_hip)."""
    rows, widths = case["rows"], case["widths"]
    p = (plan_cls or P.Plan)()
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




# ---------------------------------------------------------------------------------------------
def _conv_bn(rw, rb, ci, co):
    return dict(W=_w(rw, co, ci, 3, 3), b=np.zeros(co, np.float32),
                bn=(np.ones(co, np.float32), np.zeros(co, np.float32), (0.1 * rb.standard_normal(co)).astype(np.float32),
                    rb.uniform(0.5, 1.5, co).astype(np.float32)))


def unet(H=256, cin=4, chans=(32, 64, 128, 256), cout=4):
    """Config 4: x 1 x cin x H x H ~ N(0,1).  Encoder: (conv3x3 + BN + ReLU) x2 at chans[:-1], 2x2 maxpool
    after each; bottleneck (conv3x3 + BN + ReLU) x2 at chans[-1]; decoder: 2x2 stride-2 transposed conv,
    concat [skip, up], (conv3x3 + BN + ReLU) x2; final 1x1 conv to cout.  BN eval: running mean N(0, 0.1),
    var U(0.5, 1.5), gamma 1, beta 0, eps 1e-5; conv biases 0."""
    rw, ri, rb = np.random.default_rng(0), np.random.default_rng(1), np.random.default_rng(3)
    x = ri.standard_normal((cin, H, H)).astype(np.float32)
    enc, ci = [], cin
    for c in chans[:-1]:
        enc.append([_conv_bn(rw, rb, ci, c), _conv_bn(rw, rb, c, c)])
        ci = c
    bott = [_conv_bn(rw, rb, ci, chans[-1]), _conv_bn(rw, rb, chans[-1], chans[-1])]
    dec, ci = [], chans[-1]
    for c in reversed(chans[:-1]):
        up = dict(W=(rw.standard_normal((ci, c, 2, 2)) / np.sqrt(ci)).astype(np.float32), b=np.zeros(c, np.float32))
        dec.append(dict(up=up, convs=[_conv_bn(rw, rb, 2 * c, c), _conv_bn(rw, rb, c, c)]))
        ci = c
    final = dict(W=_w(rw, cout, ci, 1, 1), b=np.zeros(cout, np.float32))
    macs, h, cp = 0, H, cin
    for c in chans[:-1]:
        macs += h * h * 9 * (cp * c + c * c)
        cp, h = c, h // 2
    macs += h * h * 9 * (cp * chans[-1] + chans[-1] ** 2)
    cp = chans[-1]
    for c in reversed(chans[:-1]):
        h *= 2
        macs += h * h * cp * c + h * h * 9 * (2 * c * c + c * c)
        cp = c
    macs += h * h * cp * cout
    return dict(name="unet", x=x, enc=enc, bott=bott, dec=dec, final=final, H=H, cin=cin, chans=list(chans), cout=cout,
                flops=2 * macs, voxels=H * H)


def unet_plan(case, plan_cls=None):
    H, chans = case["H"], case["chans"]
    p = (plan_cls or P.Plan)()
    t_in = p.tensor(case["cin"] * H * H)
    # one buffer per decoder level holds [skip | up]; the encoder's last conv of the level writes the
    # first window, the transposed conv writes the second: the concatenation costs no copy
    cat, skip_v, up_v = {}, {}, {}
    for lvl, c in enumerate(chans[:-1]):
        hh = H >> lvl
        cat[lvl] = p.tensor(2 * c * hh * hh)
        skip_v[lvl] = p.view(cat[lvl], 0, c * hh * hh)
        up_v[lvl] = p.view(cat[lvl], c * hh * hh, c * hh * hh)

    def conv(src, dst, cv, ci, h):
        p.conv2d(src, dst, cv["W"], cv["b"], ci, h, h, 1, 1, "relu", 0.0, cv["bn"], 1e-5)

    cur, ci, h = t_in, case["cin"], H
    for lvl, (blk, c) in enumerate(zip(case["enc"], chans[:-1])):
        t = p.tensor(c * h * h)
        conv(cur, t, blk[0], ci, h)
        conv(t, skip_v[lvl], blk[1], c, h)
        t = p.tensor(c * (h // 2) * (h // 2))
        p.maxpool2d(skip_v[lvl], t, c, h, h, 2)
        cur, ci, h = t, c, h // 2
    cb = chans[-1]
    t1, t2 = p.tensor(cb * h * h), p.tensor(cb * h * h)
    conv(cur, t1, case["bott"][0], ci, h)
    conv(t1, t2, case["bott"][1], cb, h)
    cur, ci = t2, cb
    for lvl, d in zip(reversed(range(len(chans) - 1)), case["dec"]):
        c = chans[lvl]
        p.convt2d(cur, up_v[lvl], d["up"]["W"], d["up"]["b"], ci, h, h, 2, 0, 0, None, 0.0)
        h *= 2
        t1, t2 = p.tensor(c * h * h), p.tensor(c * h * h)
        conv(cat[lvl], t1, d["convs"][0], 2 * c, h)
        conv(t1, t2, d["convs"][1], c, h)
        cur, ci = t2, c
    t_out = p.tensor(case["cout"] * h * h)
    p.conv2d(cur, t_out, case["final"]["W"], case["final"]["b"], ci, h, h, 1, 0, None, 0.0)
    return p.finalize(t_in, t_out)


def tsrgan(D=33, cin=3, ch=64, nblocks=8, cout=3, alpha=0.2):
    """Config 5: x NDHWC 1 x D^3 x 3 ~ U(0,1), permuted to NCDHW inside the step; conv3d 3^3 3->64 +
    LeakyReLU(0.2); 8 residual blocks (conv 64->64, ReLU, conv 64->64, + skip); nearest x2 upsample;
    conv 64->64 + LeakyReLU(0.2); conv 64->3; output permuted back to NDHWC.  All pad 1, stride 1, bias 0."""
    rw, ri = np.random.default_rng(0), np.random.default_rng(1)
    x = ri.uniform(0, 1, (D, D, D, cin)).astype(np.float32)
    z = lambda n: np.zeros(n, np.float32)
    head = dict(W=_w(rw, ch, cin, 3, 3, 3), b=z(ch))
    blocks = [dict(W1=_w(rw, ch, ch, 3, 3, 3), b1=z(ch), W2=_w(rw, ch, ch, 3, 3, 3), b2=z(ch)) for _ in range(nblocks)]
    upc = dict(W=_w(rw, ch, ch, 3, 3, 3), b=z(ch))
    tail = dict(W=_w(rw, cout, ch, 3, 3, 3), b=z(cout))
    v1, v2 = D ** 3, (2 * D) ** 3
    macs = v1 * 27 * (cin * ch + 2 * nblocks * ch * ch) + v2 * 27 * (ch * ch + ch * cout)
    return dict(name="tsrgan", x=x, head=head, blocks=blocks, upc=upc, tail=tail, D=D, cin=cin, ch=ch, cout=cout,
                alpha=alpha, flops=2 * macs, voxels=v2)


def tsrgan_plan(case, plan_cls=None):
    D, ch, cin, cout, a = case["D"], case["ch"], case["cin"], case["cout"], case["alpha"]
    v1, D2 = D ** 3, 2 * D
    v2 = D2 ** 3
    p = (plan_cls or P.Plan)()
    t_in = p.tensor(v1 * cin)
    t = p.tensor(v1 * cin)
    p.permute(t_in, t, cin, v1, True)
    cur = p.tensor(ch * v1)
    p.conv3d(t, cur, case["head"]["W"], case["head"]["b"], cin, D, D, D, 1, "leaky", a)
    for blk in case["blocks"]:
        h1, out = p.tensor(ch * v1), p.tensor(ch * v1)
        p.conv3d(cur, h1, blk["W1"], blk["b1"], ch, D, D, D, 1, "relu", 0.0)
        p.conv3d(h1, out, blk["W2"], blk["b2"], ch, D, D, D, 1, None, 0.0, res=cur)
        cur = out
    up = p.tensor(ch * v2)
    p.upsample(cur, up, ch, D, D, D, 2, 3)
    c1 = p.tensor(ch * v2)
    p.conv3d(up, c1, case["upc"]["W"], case["upc"]["b"], ch, D2, D2, D2, 1, "leaky", a)
    c2 = p.tensor(cout * v2)
    p.conv3d(c1, c2, case["tail"]["W"], case["tail"]["b"], ch, D2, D2, D2, 1, None, 0.0)
    t_out = p.tensor(cout * v2)
    p.permute(c2, t_out, cout, v2, False)
    return p.finalize(t_in, t_out)
