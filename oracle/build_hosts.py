"""Builds the reference's own Fortran host programs, from their sources where they lie under
/root/reference, against this library: the drop-in check of the entry tier.  Outputs go to oracle/_ref/
only (git-ignored).  Test infrastructure: run by tests/test_gpu_hosts.py, built by __graft_entry__.build().

  toy_dev_hip     benchmarks/toy/bench_dev.f90  (mlp_upload / mlp_forward_dev x1000 / mlp_download; the
                  model is frontend/export_mlp.py's: seed 42, Linear(1024,256) ReLU Linear(256,1024))
  toy_call_hip    benchmarks/toy/bench_fortis.f90  (mlp_forward(x, y) x1000: upload, step, download per call)
  conv_dev_hip    benchmarks/toy/bench_dev_conv.f90, conv_call_hip  benchmarks/toy/bench_fortis_conv.f90
                  (the same two call patterns on frontend/export_conv.py's model: seed 3, Conv3d(3,8,3,pad 1)
                  LeakyReLU(0.1) on 1x3x16^3)
  zb_expert_hip   mom6_zb/zb_host_expert.f90    (per-layer hand-batched mlp_forward(xb(27,4736), yb(3,4736));
                  the model is mom6_zb/zb_nn.npz with its input and output norms)
  zb_lifted_step.so   no host: the step file and the stencil tables + fortis_gather / fortis_scatter entries that
                  the emitter writes for mom6_zb/gather.json, scatter.json, zb_loop_verdict.json, kdist.json (what
                  links beside the lifted host mom6_zb/host_fissioned.fir; that FIR text is of a newer dialect than
                  this flang parses, so the test drives the entries itself in the host's call order, :732-740)

Each links: host.o + step file emitted by fortis_amd/emit.py + libfortis_rt.so."""
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
REF = os.environ.get("FORTIS_REFERENCE", "/root/reference")
FLANG = os.environ.get("FLANG", "/opt/rocm/lib/llvm/bin/flang")
OUT = os.path.join(HERE, "_ref")


def run(cmd):
    r = subprocess.run(cmd, cwd=OUT, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("build_hosts: %s\n%s\n%s" % (" ".join(cmd), r.stdout, r.stderr))


def link(host_f90, step_c, exe):
    obj = os.path.join(OUT, exe + "_host.o")
    run([FLANG, "-O2", "-c", host_f90, "-o", obj])
    sobj = os.path.join(OUT, exe + "_step.o")
    run(["gcc", "-O2", "-c", "-I", os.path.join(ROOT, "include"), step_c, "-o", sobj])
    run([FLANG, obj, sobj, "-L", os.path.join(ROOT, "fortis_amd"), "-lfortis_rt", "-Wl,-rpath,$ORIGIN/../../fortis_amd",
         "-o", os.path.join(OUT, exe)])
    for f in (obj, sobj, step_c[:-2] + ".bin"):      # the weights are inside the object now
        os.remove(f)


def main():
    if not os.path.isdir(os.path.join(REF, "mom6_zb")) or not os.access(FLANG, os.X_OK):
        print("build_hosts: reference sources or flang not present, skipping")
        return 0
    sys.path.insert(0, ROOT)
    from fortis_amd import emit
    os.makedirs(OUT, exist_ok=True)
    # toy: the exporter's model, reproduced from its seed (frontend/export_mlp.py:3-15)
    import torch
    torch.manual_seed(42)
    net = torch.nn.Sequential(torch.nn.Linear(1024, 256), torch.nn.ReLU(), torch.nn.Linear(256, 1024)).eval()
    Ws = [net[0].weight.detach().numpy(), net[2].weight.detach().numpy()]
    bs = [net[0].bias.detach().numpy(), net[2].bias.detach().numpy()]
    c, _ = emit.emit_mlp_step(os.path.join(OUT, "toy_dev_step"), Ws, bs, ["relu", None], rows=1, graph=True)
    link(os.path.join(REF, "benchmarks/toy/bench_dev.f90"), c, "toy_dev_hip")
    c, _ = emit.emit_mlp_step(os.path.join(OUT, "toy_call_step"), Ws, bs, ["relu", None], rows=1)
    link(os.path.join(REF, "benchmarks/toy/bench_fortis.f90"), c, "toy_call_hip")
    # conv probe: the exporter's model from its seed (frontend/export_conv.py:3-4)
    torch.manual_seed(3)
    conv = torch.nn.Conv3d(3, 8, 3, padding=1)
    cw, cb = conv.weight.detach().numpy(), conv.bias.detach().numpy()
    c, _ = emit.emit_conv3d_step(os.path.join(OUT, "conv_dev_step"), cw, cb, (3, 16, 16, 16), act="leaky", alpha=0.1, graph=True)
    link(os.path.join(REF, "benchmarks/toy/bench_dev_conv.f90"), c, "conv_dev_hip")
    c, _ = emit.emit_conv3d_step(os.path.join(OUT, "conv_call_step"), cw, cb, (3, 16, 16, 16), act="leaky", alpha=0.1)
    link(os.path.join(REF, "benchmarks/toy/bench_fortis_conv.f90"), c, "conv_call_hip")
    # ZB expert host: one call per layer on 4736 cells
    W = np.load(os.path.join(ROOT, "tests", "golden", "zb_nn.npz"))
    c, _ = emit.emit_mlp_step(os.path.join(OUT, "zb_expert_step"), [W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None],
                              rows=4736, in_norms=W["in_norms"], out_norms=W["out_norms"])
    link(os.path.join(REF, "mom6_zb/zb_host_expert.f90"), c, "zb_expert_hip")
    # the lifted ZB step: plan + tables + generated entries in one shared object
    import json
    g = os.path.join(ROOT, "tests", "golden")
    desc = [json.load(open(os.path.join(g, "zb_%s.json" % n))) for n in ("gather", "scatter", "loop", "kdist")]
    c, b = emit.emit_mlp_step(os.path.join(OUT, "zb_lifted_step"), [W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None],
                              rows=71040, in_norms=W["in_norms"], out_norms=W["out_norms"], verdict="batched", expanded=True,
                              count=71040, gather=True, scatter=True)
    tc = emit.emit_stencil_tables(os.path.join(OUT, "zb_lifted_tables.c"), *desc)
    run(["gcc", "-O2", "-shared", "-fPIC", "-I", os.path.join(ROOT, "include"), c, tc, "-L", os.path.join(ROOT, "fortis_amd"),
         "-lfortis_rt", "-Wl,-rpath,$ORIGIN/../../fortis_amd", "-o", os.path.join(OUT, "zb_lifted_step.so")])
    for f in (c, b, tc):
        os.remove(f)
    print("build_hosts: built toy_dev_hip, toy_call_hip, conv_dev_hip, conv_call_hip, zb_expert_hip, zb_lifted_step.so in", OUT)
    return 0


if __name__ == "__main__":
    sys.exit(main())
