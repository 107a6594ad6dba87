"""Host programs linked against this library with step files from the FORTIS_BACKEND=hip generator
(fortis_amd/hosts/build_hosts.py): the reference's own Fortran hosts compiled from its sources, which call the
entry points by bind(c) name exactly as they do in a FORTIS build (their printed checksums and written fields are
compared with the reference-held numbers), and plain C hosts for every verdict the generator handles."""
import os
import re
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFBIN = os.path.join(ROOT, "build", "hosts")


def run_host(name, cwd, env=None, args=()):
    exe = os.path.join(REFBIN, name)
    if not os.path.exists(exe):
        if name.endswith("_hip"):
            pytest.skip(f"{exe} not built (needs the reference sources and flang at build time)")
        raise AssertionError(f"{exe} is not built: run __graft_entry__.build()")
    e = dict(os.environ)
    e.update(env or {})
    r = subprocess.run([exe] + [str(a) for a in args], cwd=cwd, capture_output=True, text=True, timeout=120, env=e)
    assert r.returncode == 0, r.stdout + r.stderr
    return r.stdout


def test_toy_host_upload_forward_dev_download(gpu, tmp_path):
    """benchmarks/toy/bench_dev.f90: upload once, 1000 x mlp_forward_dev (captured as a graph on the
    second call and replayed), download; README.md:25 stamps the checksum 7.775037."""
    out = run_host("toy_dev_hip", tmp_path)
    chk = float(re.search(r"checksum:\s*([-0-9.Ee+]+)", out).group(1))
    assert abs(chk - 7.775037) / 7.775037 < 1e-5, out
    per_call = float(re.search(r"per-call us:\s*([-0-9.Ee+]+)", out).group(1))
    print("toy host per-call us:", per_call)
    assert 0 < per_call < 1000


def test_toy_host_per_call(gpu, tmp_path):
    """benchmarks/toy/bench_fortis.f90: mlp_forward(x, y) with upload and download inside every call."""
    out = run_host("toy_call_hip", tmp_path)
    chk = float(re.search(r"checksum:\s*([-0-9.Ee+]+)", out).group(1))
    assert abs(chk - 7.775037) / 7.775037 < 1e-5, out
    print("toy host per-call (upload + step + download) us:", float(re.search(r"per-call us:\s*([-0-9.Ee+]+)", out).group(1)))


@pytest.mark.parametrize("exe", ["conv_dev_hip", "conv_call_hip"])
def test_conv_probe_hosts(gpu, tmp_path, exe):
    """benchmarks/toy/bench_dev_conv.f90 / bench_fortis_conv.f90 on the conv probe; README.md:25 stamps the
    checksum 9617.28 (an fp32 sum of 32768 terms whose exact value is 9617.4091: the stamp is 1.34e-5 off; bound 3e-5)."""
    out = run_host(exe, tmp_path)
    chk = float(re.search(r"checksum:\s*([-0-9.Ee+]+)", out).group(1))
    assert abs(chk - 9617.28) / 9617.28 < 3e-5, out
    print(exe, "per-call us:", float(re.search(r"per-call us:\s*([-0-9.Ee+]+)", out).group(1)))


def test_zb_expert_host_matches_native_golden(gpu, tmp_path, golden):
    """mom6_zb/zb_host_expert.f90: the host packs 4736 stencils per layer itself and calls
    mlp_forward(xb, yb) 15 x 11 times; its Txx/Tyy/Txy must agree with the reference's native CPU build
    (golden checksums and layers 1, 8, 15) within the reference's own difftest tolerance of 5e-6 of the
    field maximum (mom6_zb/README.md:16)."""
    out = run_host("zb_expert_hip", tmp_path)
    m = re.search(r"checksum Txx:\s*([-0-9.Ee+]+)\s+Tyy:\s*([-0-9.Ee+]+)\s+Txy:\s*([-0-9.Ee+]+)", out)
    chk = np.array([float(m.group(i)) for i in (1, 2, 3)])
    G = np.load(os.path.join(golden, "zb_native_golden.npz"))
    assert np.all(np.abs(chk - G["checksum"]) < 1e-5 * np.abs(G["checksum"])), (chk, G["checksum"])
    raw = np.fromfile(os.path.join(tmp_path, "zb_out.bin"), dtype=np.float64).reshape(3, 15, 78, 68)
    for f, name in enumerate(("Txx", "Tyy", "Txy")):
        for n, layer in enumerate(G["layers"]):
            ref = G[name][n].astype(np.float64)
            got = raw[f, layer - 1]
            assert np.abs(got - ref).max() <= 5e-6 * np.abs(ref).max(), (name, layer)


_LIFTED_CHILD = r"""
import ctypes as C, os, sys
import numpy as np
root, golden = sys.argv[1], sys.argv[2]
sys.path.insert(0, root)
from oracle import oracle as O          # checker: field synthesis of the reference host only
so = C.CDLL(os.path.join(root, "build", "hosts", "zb_lifted_step.so"))   # constructors: plan bound, tables configured
G = np.load(os.path.join(golden, "zb_native_golden.npz"))
F = O.zb_fields(); P = O.zb_prep(F)
p = lambda a: a.ctypes.data_as(C.c_void_p)
n3 = 68 * 78 * 15
for step in range(2):
    Txy_h, Txx, Tyy, Txy = np.zeros(68 * 78, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)
    so.fortis_gather(p(P["sh_xy_h"]), p(F["sh_xx"]), p(P["vort_xy_h"]), p(P["norm_h"]))
    so.mlp_forward_batched(None, None)
    for k in range(1, 16):
        so.fortis_scatter(C.c_int(k), p(P["norm_h"]), p(F["kappa_h"]), p(Txy_h), p(Txx), p(Tyy))
        h, m = Txy_h.reshape(78, 68), F["mask2dBu"].reshape(78, 68)
        Txy.reshape(15, 78, 68)[k - 1][2:75, 2:65] = np.float32(0.25) * ((h[3:76, 3:66] + h[2:75, 2:65]) + (h[2:75, 3:66] + h[3:76, 2:65])) * m[2:75, 2:65]
    lay = G["layers"] - 1
    for got, key in ((Txx, "Txx"), (Tyy, "Tyy"), (Txy, "Txy")):
        ref = G[key].astype(np.float64)
        err = np.abs(got.reshape(15, 78, 68)[lay] - ref).max() / np.abs(ref).max()
        assert err < 1e-5, (key, err)
    for n, a in enumerate((Txx, Tyy, Txy)):
        assert abs(a.astype(np.float64).sum() - G["checksum"][n]) < 1e-5 * np.abs(a).sum()
print("lifted step ok")
"""


def test_emitted_step_and_tables_drive_the_lifted_zb_step(gpu, golden, tmp_path):
    """The files the generator writes for the lifted ZB host -- the step (plan + host facts) and the stencil
    tables with their generated fortis_gather / fortis_scatter entries -- built into one shared object at build
    time and driven in the lifted host's call order (mom6_zb/host_fissioned.fir:732-740), in a process of its
    own because loading the object binds the step; results against the reference's native CPU build."""
    assert os.path.exists(os.path.join(REFBIN, "zb_lifted_step.so")), "zb_lifted_step.so is not built: run __graft_entry__.build()"
    r = subprocess.run([os.sys.executable, "-c", _LIFTED_CHILD, ROOT, golden], capture_output=True, text=True, timeout=180)
    assert r.returncode == 0 and "lifted step ok" in r.stdout, r.stdout + r.stderr


# ---- C hosts on generated step files: one per verdict of the fortis.host attribute ------------------------
def _io(tmp_path, x):
    fin, fout = os.path.join(tmp_path, "in.bin"), os.path.join(tmp_path, "out.bin")
    np.ascontiguousarray(x).tofile(fin)
    return fin, fout


@pytest.mark.parametrize("mode", ["call", "dev"])
def test_generated_unet_step_from_a_c_host(gpu, tmp_path, mode):
    """Config 4 through the whole generator chain: fortis.host attribute text + outline.json + op list ->
    step_tables.c -> C host calling mlp_forward (and the resident triple, whose graph is captured on call 2:
    fortis.graph is set and the step has more kernels than the replay threshold)."""
    import sys
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from fortis_amd import configs
    from refmodels import unet_ref
    from util import TOL, maxrel
    case = configs.unet()
    fin, fout = _io(tmp_path, case["x"])
    out = run_host("unet_host", tmp_path, args=[mode, fin, fout, case["x"].nbytes, 4 * 256 * 256 * 4, 3])
    y = np.fromfile(fout, np.float32).reshape(4, 256, 256)
    assert maxrel(y, unet_ref(case)) < TOL, out


def test_generated_tsrgan_step_from_a_c_host(gpu, tmp_path):
    import sys
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from fortis_amd import configs
    from refmodels import tsrgan_ref
    from util import TOL, maxrel
    case = configs.tsrgan()
    fin, fout = _io(tmp_path, case["x"])
    run_host("tsrgan_host", tmp_path, args=["call", fin, fout, case["x"].nbytes, 66 ** 3 * 3 * 4, 2])
    y = np.fromfile(fout, np.float32).reshape(66, 66, 66, 3)
    assert maxrel(y, tsrgan_ref(case)) < TOL


def test_generated_batched_steps_from_a_c_host(gpu, tmp_path):
    """Batched verdict in both forms: expanded (fortis_pack / mlp_forward_batched() / fortis_unpack) and the slice
    form with a strided loop (step 2 from column 3: rows 2, 4, ... of the host's arrays, the others untouched)."""
    from fortis_amd import configs
    from oracle import oracle as O
    from util import TOL, maxrel
    case = configs.toy_mlp(200)
    ref = O.mlp_f64(case["Ws"], case["bs"], case["acts"], case["X"])
    fin, fout = _io(tmp_path, case["X"])
    run_host("packed_host", tmp_path, args=["packed", fin, fout, case["X"].nbytes, 200 * 32 * 4, 2, 200])
    assert maxrel(np.fromfile(fout, np.float32).reshape(200, 32), ref) < TOL
    big = np.random.default_rng(9).uniform(-1, 1, (210, 64)).astype(np.float32)
    fin, fout = _io(tmp_path, big)
    run_host("strided_host", tmp_path, args=["slice", fin, fout, big.nbytes, 210 * 32 * 4])
    out = np.fromfile(fout, np.float32).reshape(210, 32)
    rows = np.arange(100) * 2 + 2
    c100 = configs.toy_mlp(100)
    assert maxrel(out[rows], O.mlp_f64(c100["Ws"], c100["bs"], c100["acts"], big[rows])) < TOL
    assert not out[np.setdiff1d(np.arange(210), rows)].any()


def test_generated_boundary_step_reads_host_globals_at_first_use(gpu, tmp_path):
    """Boundary verdict: the host passes its own f64 column-major arrays, and the normalisation vectors are
    arrays of the host object that it fills at run time -- the step binds at the first mlp_forward, as the
    reference's setup() does, so it sees the filled values (zeros at load time would divide by zero)."""
    from oracle import oracle as O
    from util import TOL, maxrel
    NI, NIN, NH, NOUT = 384, 124, 128, 128
    rng = np.random.default_rng(4)                                  # the seeds of build_hosts.py
    Ws = [(rng.standard_normal((NH, NIN)) / 11).astype(np.float32), (rng.standard_normal((NOUT, NH)) / 11).astype(np.float32)]
    bs = [rng.standard_normal(NH).astype(np.float32), rng.standard_normal(NOUT).astype(np.float32)]
    r2 = np.random.default_rng(14)
    A = np.asfortranarray(r2.standard_normal((NI, NIN)))
    mean, vmax, vmin, scale = r2.standard_normal(NIN), r2.uniform(2, 3, NIN), r2.uniform(0, 1, NIN), r2.uniform(0.5, 2, NOUT)
    fin, fvec, fout = [os.path.join(tmp_path, n) for n in ("in.bin", "vec.bin", "out.bin")]
    A.reshape(-1, order="F").tofile(fin)
    np.concatenate([mean, vmax, vmin, scale]).tofile(fvec)
    out = run_host("boundary_host", tmp_path, args=[fin, fvec, fout])
    assert "boundary host ok" in out
    B = np.fromfile(fout, np.float64).reshape(NOUT, NI).T
    X = O.boundary_pre(A, mean, vmax, vmin)
    ref = O.boundary_post(O.mlp_f64(Ws, bs, ["leaky", "none"], X, alphas=[0.15, 0]), scale, np.float64)
    assert maxrel(B, ref) < TOL
