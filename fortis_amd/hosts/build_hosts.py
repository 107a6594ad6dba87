"""Builds host programs against libfortis_rt.so with step files from the FORTIS_BACKEND=hip generator
(fortis_amd/shim_hip.py): the drop-in check of the entry tier.  Outputs go to build/hosts/ (git-ignored);
built by __graft_entry__.build(), run by tests/test_gpu_hosts.py.

From the reference's own Fortran sources, where they lie under /root/reference (skipped when that tree or
flang is absent):
  toy_dev_hip     benchmarks/toy/bench_dev.f90  (mlp_upload / mlp_forward_dev x1000 / mlp_download; the
                  model is frontend/export_mlp.py's: seed 42, Linear(1024,256) ReLU Linear(256,1024))
  toy_call_hip    benchmarks/toy/bench_fortis.f90  (mlp_forward(x, y) x1000: upload, step, download per call)
  conv_dev_hip    benchmarks/toy/bench_dev_conv.f90, conv_call_hip  benchmarks/toy/bench_fortis_conv.f90
                  (the same two call patterns on frontend/export_conv.py's model: seed 3, Conv3d(3,8,3,pad 1)
                  LeakyReLU(0.1) on 1x3x16^3)
  zb_expert_hip   mom6_zb/zb_host_expert.f90    (per-layer hand-batched mlp_forward(xb(27,4736), yb(3,4736));
                  the model is mom6_zb/zb_nn.npz with its input and output norms)
  zb_lifted_step.so   no host: the step file and the stencil tables + fortis_gather / fortis_scatter entries
                  for mom6_zb/gather.json, scatter.json, zb_loop_verdict.json, kdist.json (what links beside the
                  lifted host mom6_zb/host_fissioned.fir; that FIR text is of a newer dialect than this flang
                  parses, so the test drives the entries itself in the host's call order, :732-740)
From this repository's C hosts (fortis_amd/hosts/step_host.c, boundary_host.c), one per verdict:
  unet_host, tsrgan_host   whole-array call on the UNet and TSRGAN configurations (conv2d / convT / pool / concat
                  windows / conv3d / upsample / permute stacks)
  packed_host     batched verdict, expanded: fortis_pack / mlp_forward_batched() / fortis_unpack
  strided_host    batched verdict, slice form with step 2 from column 3
  boundary_host   boundary verdict: f64 column-major host arrays, normalisation vectors as host globals

Each links: host.o + step_tables.o + weights.o + libfortis_rt.so."""
import json
import os
import shutil
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
REF = os.environ.get("FORTIS_REFERENCE", "/root/reference")
FLANG = os.environ.get("FLANG", "/opt/rocm/lib/llvm/bin/flang")
OUT = os.path.join(ROOT, "build", "hosts")
INC = os.path.join(ROOT, "include")
LIBDIR = os.path.join(ROOT, "fortis_amd")
RPATH = "-Wl,-rpath,$ORIGIN/../../fortis_amd"


def run(cmd):
    r = subprocess.run(cmd, cwd=OUT, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("build_hosts: %s\n%s\n%s" % (" ".join(cmd), r.stdout, r.stderr))


def step_objects(work, cfiles):
    objs = []
    for c in cfiles:
        o = c[:-2] + ".o"
        run(["gcc", "-O2", "-fPIC", "-c", "-I", INC, c, "-o", o])
        objs.append(o)
    return objs


def link(host_src, cfiles, exe, work, fortran=True, defs=()):
    hobj = os.path.join(work, "host.o")
    if fortran:
        run([FLANG, "-O2", "-c", host_src, "-o", hobj])
    else:
        run(["gcc", "-O2", "-c"] + list(defs) + [host_src, "-o", hobj])
    objs = step_objects(work, cfiles)
    run([FLANG if fortran else "gcc", hobj] + objs + ["-L", LIBDIR, "-lfortis_rt", RPATH, "-o", os.path.join(OUT, exe)])
    shutil.rmtree(work)        # the weights are inside the executable now


def main():
    sys.path.insert(0, ROOT)
    from fortis_amd import configs, emit, shim_hip
    os.makedirs(OUT, exist_ok=True)
    built = []
    W = np.load(os.path.join(ROOT, "tests", "golden", "zb_nn.npz"))
    if os.path.isdir(os.path.join(REF, "mom6_zb")) and os.access(FLANG, os.X_OK):
        # toy: the exporter's model, reproduced from its seed (frontend/export_mlp.py:3-15)
        import torch
        torch.manual_seed(42)
        net = torch.nn.Sequential(torch.nn.Linear(1024, 256), torch.nn.ReLU(), torch.nn.Linear(256, 1024)).eval()
        Ws = [net[0].weight.detach().numpy(), net[2].weight.detach().numpy()]
        bs = [net[0].bias.detach().numpy(), net[2].bias.detach().numpy()]
        for exe, src, graph in (("toy_dev_hip", "benchmarks/toy/bench_dev.f90", True), ("toy_call_hip", "benchmarks/toy/bench_fortis.f90", False)):
            work = os.path.join(OUT, exe + "_work")
            link(os.path.join(REF, src), emit.emit_mlp_step(work, Ws, bs, ["relu", None], rows=1, graph=graph), exe, work)
            built.append(exe)
        # conv probe: the exporter's model from its seed (frontend/export_conv.py:3-4)
        torch.manual_seed(3)
        conv = torch.nn.Conv3d(3, 8, 3, padding=1)
        cw, cb = conv.weight.detach().numpy(), conv.bias.detach().numpy()
        for exe, src, graph in (("conv_dev_hip", "benchmarks/toy/bench_dev_conv.f90", True), ("conv_call_hip", "benchmarks/toy/bench_fortis_conv.f90", False)):
            work = os.path.join(OUT, exe + "_work")
            link(os.path.join(REF, src), emit.emit_conv3d_step(work, cw, cb, (3, 16, 16, 16), act="leaky", alpha=0.1, graph=graph), exe, work)
            built.append(exe)
        # ZB expert host: one call per layer on 4736 cells
        work = os.path.join(OUT, "zb_expert_work")
        cs = emit.emit_mlp_step(work, [W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None], rows=4736, in_norms=W["in_norms"], out_norms=W["out_norms"])
        link(os.path.join(REF, "mom6_zb/zb_host_expert.f90"), cs, "zb_expert_hip", work)
        built.append("zb_expert_hip")
    else:
        print("build_hosts: reference sources or flang not present, skipping the reference's Fortran hosts")
    # the lifted ZB step: plan + tables + generated entries in one shared object
    g = os.path.join(ROOT, "tests", "golden")
    desc = [json.load(open(os.path.join(g, "zb_%s.json" % n))) for n in ("gather", "scatter", "loop", "kdist")]
    work = os.path.join(OUT, "zb_lifted_work")
    cs = emit.emit_mlp_step(work, [W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None], rows=71040, in_norms=W["in_norms"],
                            out_norms=W["out_norms"], verdict="batched", expanded=True, count=71040, gather=True, scatter=True)
    cs.append(emit.emit_stencil_tables(os.path.join(work, "zb_lifted_tables.c"), *desc))
    run(["gcc", "-shared"] + step_objects(work, cs) + ["-L", LIBDIR, "-lfortis_rt", RPATH, "-o", os.path.join(OUT, "zb_lifted_step.so")])
    shutil.rmtree(work)
    built.append("zb_lifted_step.so")
    # C hosts on generated step files, one per verdict
    host_c = os.path.join(HERE, "step_host.c")
    case = configs.unet()
    work = os.path.join(OUT, "unet_work")
    cs = emit.step_files(work, configs.unet_plan(case, plan_cls=shim_hip.OpList), emit.host_attr("whole", shape=(1, 4, 256, 256), graph=True),
                         "tensor<1x4x256x256xf32>", "tensor<1x4x256x256xf32>")
    link(host_c, cs, "unet_host", work, fortran=False)
    case = configs.tsrgan()
    work = os.path.join(OUT, "tsrgan_work")
    cs = emit.step_files(work, configs.tsrgan_plan(case, plan_cls=shim_hip.OpList), emit.host_attr("whole", shape=(1, 33, 33, 33, 3)),
                         "tensor<1x33x33x33x3xf32>", "tensor<1x66x66x66x3xf32>")
    link(host_c, cs, "tsrgan_host", work, fortran=False)
    toy = configs.toy_mlp(200)
    work = os.path.join(OUT, "packed_work")
    link(host_c, emit.emit_mlp_step(work, toy["Ws"], toy["bs"], toy["acts"], 200, verdict="batched", expanded=True, count=200), "packed_host", work, fortran=False)
    toy = configs.toy_mlp(100)
    work = os.path.join(OUT, "strided_work")
    link(host_c, emit.emit_mlp_step(work, toy["Ws"], toy["bs"], toy["acts"], 100, verdict="batched", count=100, lo=3, step=2, minc=3), "strided_host", work, fortran=False)
    # boundary verdict: f64 host arrays, the four normalisation vectors are globals of the host object
    NI, NIN, NH, NOUT = 384, 124, 128, 128
    rng = np.random.default_rng(4)
    Ws = [(rng.standard_normal((NH, NIN)) / 11).astype(np.float32), (rng.standard_normal((NOUT, NH)) / 11).astype(np.float32)]
    bs = [rng.standard_normal(NH).astype(np.float32), rng.standard_normal(NOUT).astype(np.float32)]
    ol = shim_hip.OpList()
    t0, t1, t2, t3, t4 = ol.tensor(NI * NIN, 8), ol.tensor(NI * NIN), ol.tensor(NI * NH), ol.tensor(NI * NOUT), ol.tensor(NI * NOUT, 8)
    ol.boundary_pre(t0, t1, NI, NIN, "g0", "g1", "g2", np.float64)
    ol.linear(t1, t2, Ws[0], bs[0], NI, "leaky", 0.15)
    ol.linear(t2, t3, Ws[1], bs[1], NI, None)
    ol.boundary_post(t3, t4, NI, NOUT, "g3", np.float64)
    ol.finalize(t0, t4)
    attr = emit.host_attr("boundary", shape=(NI, NIN), boundary=dict(**{"in": "colmajor", "in_elt": "f64", "out": "colmajor", "out_elt": "f64"},
                                                                      pre=["cam_mean", "cam_max", "cam_min"], post=["cam_oscale"]))
    work = os.path.join(OUT, "boundary_work")
    cs = emit.step_files(work, ol, attr, "tensor<%dx%dxf64>" % (NI, NIN), "tensor<%dx%dxf64>" % (NI, NOUT),
                         extra_inputs=["tensor<%dxf64>" % NIN] * 3 + ["tensor<%dxf64>" % NOUT])
    link(os.path.join(HERE, "boundary_host.c"), cs, "boundary_host", work, fortran=False, defs=["-DNI=%d" % NI, "-DNIN=%d" % NIN, "-DNOUT=%d" % NOUT])
    built += ["unet_host", "tsrgan_host", "packed_host", "strided_host", "boundary_host"]
    print("build_hosts: built", ", ".join(built), "in", OUT)
    return 0


if __name__ == "__main__":
    sys.exit(main())
