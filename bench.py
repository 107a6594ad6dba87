#!/usr/bin/env python3
"""Benchmark of the fused inference step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload climsim|zb|zb_ref|zb_unfused|toy|unet|tsrgan|copy|climsim_host|zb_host] [--no-cpu]

One "step" is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  Prints ONE JSON line: columns/s for the whole job, the roofline figure of the dominant
kernel (duration measured with HIP events on the library's own stream inside the timed region) and
a CPU baseline (PyTorch CPU eval of the same network, the reference's CPU path for the column MLPs, with the oracle's
port of the reference's native Fortran forward beside it, both timed on this host on a bounded sample of the same
workload).  Only the cpu_baseline leg touches oracle/.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_F32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this
# same command (see profiles/), or None where no counter run has been made for the workload.
MEASURED_TRAFFIC = {"climsim": int((61642.6 * 2 + 68419.7) * 1024), "zb": int((1059.5 * 2 + 885.2) * 1024),
                    "zb_ref": int((990.4 * 2 + 885.2) * 1024), "zb_1028x1028x15": int((200382.1 * 2 + 192014.2) * 1024),
                    "zb_ref_1028x1028x15": int((196559.2 * 2 + 192937.5) * 1024), "toy": int((1638.8 * 2 + 128.0) * 1024),
                    "zb_unfused_1028x1028x15": int((242206.1 * 2 + 1659097.0) * 1024),
                    "zb_unfused_1028x1028x15_f64": int((247395.1 * 2 + 1659004.2) * 1024),
                    # conv workloads: every dispatch of a step summed, divided by the step's conv operations (18 and 19),
                    # like flop_per_launch
                    "unet": int((1084771.1 * 2 + 491007.3) * 1024 / 7 / 18), "tsrgan": int((3426949.4 * 2 + 4994724.7) * 1024 / 7 / 19)}


TRAFFIC_SOURCE = {"climsim": "profiles/gemm_bias_act_climsim.txt", "zb": "profiles/mlp_chain_stencil_zb.txt", "toy": "profiles/mlp_chain_stencil_zb.txt",
                  "zb_ref": "profiles/mlp_chain_stencil_zb.txt", "zb_1028x1028x15": "profiles/mlp_chain_stencil_zb.txt",
                  "zb_ref_1028x1028x15": "profiles/mlp_chain_stencil_zb.txt",
                  "zb_unfused_1028x1028x15": "profiles/stencil_gather_scatter_zb_1028x1028x15.txt",
                  "zb_unfused_1028x1028x15_f64": "profiles/stencil_gather_scatter_zb_1028x1028x15.txt",
                  "unet": "profiles/conv_mfma_unet_tsrgan.txt", "tsrgan": "profiles/conv_mfma_unet_tsrgan.txt"}


def traffic(key):
    """roofline.traffic and where it comes from: a constant from a rocprofv3 --pmc run of this command recorded under
    profiles/ (counters cannot be read from inside this process), never a figure of the present run."""
    t = MEASURED_TRAFFIC.get(key)
    return dict(traffic=t, traffic_source=None if t is None else
                "constant from %s (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE passes of this command); not measured in this run" % TRAFFIC_SOURCE[key])


def omp_threads():
    try:
        return int(os.environ.get("OMP_NUM_THREADS", "")) or os.cpu_count()
    except ValueError:
        return os.cpu_count()


def cpu_baseline_mlp(case, sample_rows, X, min_seconds=8.0, **kw):
    """Times oracle.mlp_native_t (native Fortran loop nest, OpenMP over columns) on `sample_rows` rows."""
    from oracle import oracle as O   # checker / baseline only
    Xs = np.ascontiguousarray(X[:sample_rows])
    O.mlp_native_t(case["Ws"], case["bs"], case["acts"], Xs[:64], alphas=case.get("alphas"), **kw)   # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        O.mlp_native_t(case["Ws"], case["bs"], case["acts"], Xs, alphas=case.get("alphas"), **kw)
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds or reps >= 100000:
            break
    return dict(value=sample_rows * reps / dt, unit="columns/s", cores=omp_threads(), kind="port",
                sample=f"{sample_rows} of {case['rows']} rows x {reps} passes of oracle mlp_native_t "
                       f"(native Fortran loop order, fp32, OpenMP over columns), {dt:.1f} s")


def cpu_torch_mlp(case, sample_rows, X, min_seconds=4.0, in_norms=None, out_norms=None):
    """PyTorch CPU eval (fp32, torch.no_grad, all host threads) of the same seeded network on the same sample:
    the reference's other CPU path (its exporters' nn.Module in eval mode)."""
    import torch
    torch.set_num_threads(omp_threads())
    acts, alphas = case["acts"], case.get("alphas") or [0.0] * len(case["Ws"])
    Ws = [torch.from_numpy(np.ascontiguousarray(w)) for w in case["Ws"]]
    bs = [torch.from_numpy(np.ascontiguousarray(b)) for b in case["bs"]]
    x = torch.from_numpy(np.ascontiguousarray(X[:sample_rows]))
    inn = None if in_norms is None else torch.from_numpy(np.ascontiguousarray(in_norms, dtype=np.float32))
    outn = None if out_norms is None else torch.from_numpy(np.ascontiguousarray(out_norms, dtype=np.float32))

    def fwd():
        with torch.no_grad():
            h = x if inn is None else x / inn
            for W, b, a, al in zip(Ws, bs, acts, alphas):
                h = torch.nn.functional.linear(h, W, b)
                if a == "relu":
                    h = torch.relu(h)
                elif a == "leaky":
                    h = torch.nn.functional.leaky_relu(h, float(al))
            return h if outn is None else h * outn
    fwd()
    reps, t0 = 0, time.perf_counter()
    while True:
        fwd()
        reps += 1
        dt = time.perf_counter() - t0
        if dt >= min_seconds or reps >= 100000:
            break
    return dict(value=sample_rows * reps / dt, unit="columns/s", threads=omp_threads(),
                sample=f"PyTorch {torch.__version__} CPU eval fp32 of the same network, {sample_rows} rows x {reps} passes, {dt:.1f} s")


def cpu_baseline_both(case, sample_rows, X, port_seconds, torch_seconds, **norms):
    """The stated CPU baseline is the reference's own CPU path for the column MLPs, PyTorch CPU eval of the exporter's
    module (benchmarks/climsim/export_climsim.py:32-34 writes its reference output that way); the oracle's port of
    the native Fortran loop nest (mom6_zb/fwd_native_zb.f90:30-48) on the same sample rides inside it."""
    t = cpu_torch_mlp(case, sample_rows, X, min_seconds=torch_seconds, **norms)
    port = cpu_baseline_mlp(case, sample_rows, X, min_seconds=port_seconds, **norms)
    return dict(value=t["value"], unit=t["unit"], cores=t["threads"], kind="port", path="pytorch_cpu_eval",
                sample=t["sample"] + " (a restated nn.Module with the same seeded weights; the reference's exporter is not imported)",
                native_loop_port=port)


def timed_steps(L, plan, steps):
    """Two passes of `steps` steps each: the first, with nothing but the step's own launches on the stream,
    is the clocked one (-> value, ms_per_step); the second records a HIP event on the library's stream
    before and after every kernel (-> per-kernel durations for the roofline figure).  Events between
    kernels cost a few microseconds of idle stream each, which is why the clocked pass carries none."""
    t0 = time.perf_counter()
    for _ in range(steps):
        plan.run()
    L.fortis_sync()
    dt = time.perf_counter() - t0
    plan.profile(True)
    for _ in range(steps):
        plan.run()
    L.fortis_sync()
    passes, per = plan.profile_read()
    plan.profile(False)
    assert passes == steps
    return dt, passes, per


def run_climsim(L, args):
    from fortis_amd import configs
    case = configs.climsim()
    plan = configs.climsim_plan(case, boundary=True)
    plan.write(plan.in_tensor, case["A"].reshape(-1, order="F"))
    for _ in range(args.warmup):
        plan.run()
    L.fortis_sync()
    dt, passes, per = timed_steps(L, plan, args.steps)
    gemm_ms = sum(ms for name, ms in per if name == "gemm_bias_act")
    ngemm = sum(1 for name, _ in per if name == "gemm_bias_act")
    avg_launch_ms = gemm_ms / (ngemm * passes)
    flops_per_launch = case["flops"] / ngemm
    achieved = flops_per_launch / (avg_launch_ms * 1e-3) / 1e12
    kern = {name: 0.0 for name, _ in per}
    for name, ms in per:
        kern[name] += ms / passes
    out = dict(rows=case["rows"], dt=dt, dtype="f32",
               config={"workload": "climsim_mlp_24576x556_768x5_368", "columns": case["rows"],
                       "widths": case["widths"], "step": "colmajor gather -> 6 fused GEMM+bias+LeakyReLU -> colmajor scatter",
                       "launches_per_step": plan.num_kernels, "ms_per_step_by_kernel": {k: round(v, 4) for k, v in kern.items()}},
               roofline=dict(bound="mfma", kernel="gemm_bias_act (fp32 MFMA 32x32x2)", achieved=round(achieved, 3),
                             peak=PEAK_F32_MFMA_TFLOPS, unit="TFLOP/s", frac=round(achieved / PEAK_F32_MFMA_TFLOPS, 4),
                             avg_launch_ms=round(avg_launch_ms, 5), flop_per_launch=flops_per_launch,
                             **traffic("climsim")))
    if not args.no_cpu:
        X = np.ascontiguousarray(case["A"][:2048])
        out["cpu_baseline"] = cpu_baseline_both(case, 2048, X, 8.0, 6.0)
    plan.close()
    return out


def run_copy(L, args):
    """Plain device copy of 256 MiB (concat-by-copy kernel): the known-size kernel the HBM counters are
    calibrated against, and the achievable-bandwidth yardstick for the memory-bound kernels."""
    from fortis_amd import plan as P
    n = 64 * 1024 * 1024
    p = P.Plan()
    a, b = p.tensor(n), p.tensor(n)
    p.concat_copy(a, b, 1, n, 0, 1)
    p.finalize(a, b)
    p.write(a, np.ones(n, np.float32))
    p.time_ms(max(1, args.warmup))
    L.fortis_sync()
    t0 = time.perf_counter()
    ms = p.time_ms(args.steps)
    L.fortis_sync()
    dt = time.perf_counter() - t0
    avg = ms / args.steps
    gbs = 2 * n * 4 / (avg * 1e-3) / 1e9
    out = dict(rows=n, dt=dt, dtype="f32", config={"workload": "device_copy_256MiB", "columns": n, "launches_per_step": 1},
               roofline=dict(bound="hbm", kernel="copy_kernel", achieved=round(gbs, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                             frac=round(gbs / PEAK_HBM_GBS, 4), avg_launch_ms=round(avg, 5), bytes_per_launch=2 * n * 4, traffic=None))
    p.close()
    return out


def run_zb_unfused(L, args):
    """The reference's structure of the ZB step: gather kernel -> X in HBM -> MLP -> Y in HBM -> scatter
    (mom6_zb/gather.cu:50-57, 82-91; all layers scattered by one launch, as fortis_scatter does under loop
    distribution), every part timed with HIP events on the library's stream.  The gather is the memory-bound kernel
    of the path: the roofline block is its."""
    from fortis_amd import configs, plan as P, stencil as S
    sx, sy, nz = (int(v) for v in (args.grid or "1028x1028x15").lower().split("x"))
    gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
    # --f64: every host array is double precision (an E3SM-style host), which takes the general stencil
    # kernels (typed expression evaluation) instead of the fp32 form
    esz, ft = (8, np.float64) if args.f64 else (4, np.float32)
    if args.f64:
        for d in (gd, sd):
            for a in d["arrays"]:
                a["elt"] = "f64"
    gt, st = S.build_table(gd, lp, kd, "gather"), S.build_table(sd, lp, kd, "scatter")
    A = {k: np.ascontiguousarray(v, dtype=ft) for k, v in configs.zb_arrays(sx, sy, nz).items()}
    rows, count, n3 = gt.count * gt.nk, int(gt.count), sx * sy * nz
    net = configs.zb_mlp()

    held = []

    def dev(a):
        d = L.fortis_alloc(a.nbytes)
        L.fortis_h2d(d, a.ctypes.data, a.nbytes)
        held.append(d)
        return d
    # The gather's four planes live in ONE device allocation, one behind the other: together they just fit the chip's 256 MB
    # memory-side cache and stay in it from step to step only if their lines spread evenly over its sets, which
    # consecutive addresses do and four buffers placed wherever the pool has room do not (0.31 against 0.37 ms per gather).
    # They are allocated before the plan's gigabytes of X and Y for the same reason (behind them, in a process that had run
    # other large workloads, the gather read 0.325 ms).
    garr = [A[k] for k in ("sh_xy_h", "sh_xx", "vort_xy_h", "norm_h")]
    goff = np.cumsum([0] + [(a.nbytes + 255) // 256 * 256 for a in garr])
    gblock = L.fortis_alloc(int(goff[-1]))
    held.append(gblock)
    for a, o in zip(garr, goff):
        L.fortis_h2d(gblock + int(o), a.ctypes.data, a.nbytes)
    dG = (C.c_void_p * 4)(*[gblock + int(o) for o in goff[:4]])
    dS = (C.c_void_p * 5)(dG[3], dev(A["kappa_h"]), dev(np.zeros(n3, ft)), dev(np.zeros(n3, ft)), dev(np.zeros(n3, ft)))   # Txy_h: a plane per layer
    plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows)
    dX = L.fortis_plan_tensor_ptr(plan.handle, plan.in_tensor)
    dY = L.fortis_plan_tensor_ptr(plan.handle, plan.out_tensor)
    CB = C.CFUNCTYPE(None, C.c_void_p)
    gather_cb = CB(lambda _: L.fortis_stencil_gather_dev(C.byref(gt), dG, dX))

    def scatter_all(_):
        assert L.fortis_stencil_scatter_all_dev(C.byref(st), dS, C.c_void_p(dY)) == 0
    scatter_cb = CB(scatter_all)
    mlp_cb = CB(lambda _: plan.run())
    parts = (CB * 3)(gather_cb, mlp_cb, scatter_cb)

    def step():
        gather_cb(None)
        plan.run()
        scatter_all(None)
    for _ in range(max(1, args.warmup)):
        step()
    L.fortis_sync()
    # clocked pass: the step's own launches only, in the step's order; then the same steps with an event
    # between the parts (gather / MLP / the scatter launches), each part right behind the one before it
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    L.fortis_sync()
    dt = time.perf_counter() - t0
    ms = (C.c_float * 3)()
    assert L.fortis_time_parts_ms(3, parts, None, args.steps, ms) == 0
    g_ms, m_ms, s_ms = (v / args.steps for v in ms)
    # the gather alone, launched back to back (what a kernel trace of a gather-only loop shows): reported beside the
    # in-step figure, which is the one the roofline block is priced on
    alone = (C.c_float * 1)()
    assert L.fortis_time_parts_ms(1, (CB * 1)(gather_cb), None, max(10, args.steps), alone) == 0
    ga_ms = alone[0] / max(10, args.steps)
    g_bytes = esz * 4 * n3 + 4 * 27 * rows                 # 4 planes read once, X written
    s_bytes = 4 * 3 * rows + esz * (n3 + sx * sy + 3 * rows)       # Y read, norm's planes and the one kappa plane read once, 3 outputs written
    gbs = g_bytes / (g_ms * 1e-3) / 1e9
    kname = "gather_generic_kernel (typed stencil gather, fp64 host arrays)" if args.f64 else "gather_kernel (stencil gather with lifted expressions)"
    roof = dict(bound="hbm", kernel=kname, achieved=round(gbs, 1), peak=PEAK_HBM_GBS,
                unit="GB/s", frac=round(gbs / PEAK_HBM_GBS, 4), avg_launch_ms=round(g_ms, 5), bytes_per_launch=g_bytes,
                back_to_back_ms=round(ga_ms, 5), back_to_back_frac=round(g_bytes / (ga_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                scatter_GBs=round(s_bytes / (s_ms * 1e-3) / 1e9, 1), scatter_frac=round(s_bytes / (s_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), scatter_ms_all_layers=round(s_ms, 5), mlp_ms=round(m_ms, 5),
                **traffic("zb_unfused_%dx%dx%d%s" % (sx, sy, nz, "_f64" if args.f64 else "")))
    out = dict(rows=rows, dt=dt, dtype="f32",
               config={"workload": "zb_unfused_gather_mlp_scatter_27_64_64_3_%dx%dx%d%s" % (sx, sy, nz, "_f64_arrays" if args.f64 else ""), "columns": rows,
                       "cells_per_layer": count, "layers": nz, "launches_per_step": 2 + (nz - 1 if args.f64 else 0) + plan.num_kernels},
               roofline=roof)
    plan.close()
    for d in held:
        L.fortis_free(d)
    return out


def run_conv(L, args, which):
    """Configs 4 and 5: voxels/s = output spatial positions per second."""
    from fortis_amd import configs
    if which == "unet":
        case = configs.unet()
        plan = configs.unet_plan(case)
        name, dom = "unet2d_1x4x256x256_32_64_128_256", "conv2d"
    else:
        case = configs.tsrgan()
        plan = configs.tsrgan_plan(case)
        name, dom = "tsrgan3d_33cubed_to_66cubed_64ch_8blocks", "conv3d"
    plan.write(plan.in_tensor, case["x"])
    for _ in range(args.warmup):
        plan.run()
    L.fortis_sync()
    dt, passes, per = timed_steps(L, plan, args.steps)
    kern, count = {}, {}
    for n, ms in per:
        kern[n] = kern.get(n, 0.0) + ms / passes
        count[n] = count.get(n, 0) + 1
    dom_ms = kern[dom]
    # every flop of these models is in the convolutions (transposed convs are counted with them; they
    # are under 2 % of the UNet's work), so the conv kernels' share of the clock prices them
    # The per-kernel clock (an event after every kernel) leaves a few microseconds of idle stream per launch that the
    # clocked pass does not have, so its sum exceeds the clocked step.  The convolutions are therefore priced at
    # their SHARE of the event pass applied to the clocked step time: conv time <= step time by construction.
    ev_total = sum(kern.values())
    step_ms = dt / passes * 1e3
    conv_ms = step_ms * sum(v for k, v in kern.items() if k in ("conv2d", "conv3d", "convt2d")) / ev_total
    raw = dict(kern)                                   # as clocked by the events, idle stream per launch included
    kern = {k: v * step_ms / ev_total for k, v in kern.items()}
    nconv = sum(v for k, v in count.items() if k in ("conv2d", "conv3d", "convt2d"))
    achieved = case["flops"] / (conv_ms * 1e-3) / 1e12
    out = dict(rows=case["voxels"], dt=dt, dtype="f32", unit="voxels/s",
               config={"workload": name, "voxels": case["voxels"], "launches_per_step": plan.num_kernels,
                       "ms_per_step_by_kernel": {k: round(v, 4) for k, v in kern.items()}},
               roofline=dict(bound="mfma", kernel=dom + " (+ fused BN/bias/activation/residual epilogue)", achieved=round(achieved, 3),
                             peak=PEAK_F32_MFMA_TFLOPS, unit="TFLOP/s", frac=round(achieved / PEAK_F32_MFMA_TFLOPS, 4),
                             avg_launch_ms=round(conv_ms / nconv, 5), flop_per_launch=case["flops"] / nconv,
                             conv_share_of_step=round(conv_ms / step_ms, 4), event_pass_ms_per_step=round(ev_total, 4),
                             frac_basis="estimate: the convolutions' share of the event pass (event_pass_ms_by_kernel) applied to the clocked step",
                             event_pass_ms_by_kernel={k: round(v, 4) for k, v in raw.items()},
                             **traffic(which)))
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_conv(case, which)
    plan.close()
    return out


def cpu_baseline_conv(case, which):
    """PyTorch CPU eval (fp32, all host threads) of the whole model: the reference's CPU path for the
    conv configurations; beside it the oracle's own direct loop nest on one representative layer."""
    import torch
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from refmodels import tsrgan_ref, unet_ref
    from oracle import oracle as O
    torch.set_num_threads(omp_threads())
    fn = unet_ref if which == "unet" else tsrgan_ref
    fn(case, dtype=torch.float32)
    reps, t0 = 0, time.perf_counter()
    while True:
        fn(case, dtype=torch.float32)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > 8.0:
            break
    # oracle direct loops on one layer, extrapolated by MAC count
    if which == "unet":
        cv = case["dec"][-1]["convs"][1]
        x = np.random.default_rng(1).standard_normal((1, 32, 256, 256)).astype(np.float32)
        t1 = time.perf_counter(); O.conv2d(x, cv["W"], (1, 1), (1, 1)); t_layer = time.perf_counter() - t1
        share = 2 * 256 * 256 * 9 * 32 * 32 / case["flops"]
    else:
        blk = case["blocks"][0]
        x = np.random.default_rng(1).standard_normal((1, 64, 33, 33, 33)).astype(np.float32)
        t1 = time.perf_counter(); O.conv3d(x, blk["W1"], pad=(1, 1, 1)); t_layer = time.perf_counter() - t1
        share = 2 * 33 ** 3 * 27 * 64 * 64 / case["flops"]
    return dict(value=case["voxels"] * reps / dt, unit="voxels/s", cores=omp_threads(), kind="port",
                sample=f"PyTorch CPU eval fp32 of the whole model, {reps} passes in {dt:.1f} s; "
                       f"oracle direct loop nest (fp64 accumulate, OpenMP) on one layer = {share * 100:.1f} % of the MACs "
                       f"took {t_layer:.2f} s -> {case['voxels'] * share / t_layer:.3g} voxels/s extrapolated")


def run_climsim_host(L, args):
    """PCIe-inclusive: the boundary verdict's whole-array call, mlp_forward(host column-major A, host column-major B)
    (driver/fortis_shim.py:126-133), on pageable host arrays as a Fortran host owns them.  Never the headline value."""
    from fortis_amd import configs, step as ST
    case = configs.climsim()
    plan = configs.climsim_plan(case, boundary=True)
    A = np.ascontiguousarray(case["A"].reshape(-1, order="F"))
    rows = case["rows"]
    nout = rows * case["widths"][-1]
    ST.bind(plan, A.size, nout, verdict="boundary")
    out = np.empty(nout, np.float32)
    for _ in range(max(2, args.warmup)):
        ST.mlp_forward(A, out)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        ST.mlp_forward(A, out)
    dt = time.perf_counter() - t0
    nk = plan.num_kernels
    ST.reset()
    plan.close()
    nbytes = A.nbytes + out.nbytes
    ms = dt / args.steps * 1e3
    return dict(rows=rows, dt=dt, dtype="f32",
                config={"workload": "climsim_host_arrays_mlp_forward_24576x556_to_24576x368", "columns": rows, "launches_per_step": nk,
                        "host_bytes_per_call": nbytes, "note": "host arrays pageable; in row bands through page-locked staging, copies under the computation"},
                roofline=dict(bound="pcie", kernel="whole-array entry (host -> device -> host)", achieved=round(nbytes / (ms * 1e-3) / 1e9, 2), peak=None,
                              unit="GB/s over the bus, both directions summed", frac=None, avg_launch_ms=round(ms, 4), traffic=None))


def run_zb_host_step(L, args):
    """PCIe-inclusive: the fissioned ZB host's step through the entries, fortis_gather(4 host arrays) ->
    mlp_forward_batched() -> 15 x fortis_scatter(k, 5 host arrays) (mom6_zb/host_fissioned.fir:732-740), reference
    geometry and network, pageable host arrays."""
    from fortis_amd import configs, plan as P, stencil as S, step as ST
    g = os.path.join(ROOT, "tests", "golden")
    gt, st, gd, sd, lp, kd = S.load_tables(f"{g}/zb_gather.json", f"{g}/zb_scatter.json", f"{g}/zb_loop.json", f"{g}/zb_kdist.json")
    W = np.load(f"{g}/zb_nn.npz")
    A = configs.zb_arrays(68, 78, 15)
    rows = 71040
    plan = P.mlp_plan([W["A0"], W["A1"]], [W["b0"], W["b1"]], ["relu", None], rows, in_norms=W["in_norms"], out_norms=W["out_norms"])
    ST.bind(plan, rows * 27, rows * 3, verdict="batched", expanded=True, count=rows, gather=True, scatter=True)
    ST.gather_config(gt)
    ST.scatter_config(st)
    n3 = 68 * 78 * 15
    Txy_h, Txx, Tyy = np.zeros(68 * 78, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)
    ga = [a.ctypes.data for a in (A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"])]
    sa = [a.ctypes.data for a in (A["norm_h"], A["kappa_h"], Txy_h, Txx, Tyy)]

    def step():
        L.fortis_gather(*ga)
        ST.mlp_forward_batched()
        for k in range(1, 16):
            L.fortis_scatter(k, *sa)
    for _ in range(max(3, args.warmup)):
        step()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    dt = time.perf_counter() - t0
    ST.reset()
    plan.close()
    ms = dt / args.steps * 1e3
    return dict(rows=rows, dt=dt, dtype="f32",
                config={"workload": "zb_host_step_gather_batched_15_scatters_68x78x15", "columns": rows, "launches_per_step": 3,
                        "note": "host arrays pageable; includes the Python call overhead of 17 entry calls per step"},
                roofline=dict(bound="pcie", kernel="fortis_gather + mlp_forward_batched + 15 fortis_scatter", achieved=None, peak=None,
                              unit="", frac=None, avg_launch_ms=round(ms, 5), traffic=None))


def run_toy(L, args):
    from fortis_amd import configs
    case = configs.toy_mlp()
    plan = configs.mlp_case_plan(case)
    plan.write(plan.in_tensor, case["X"])
    plan.time_ms(max(1, args.warmup))
    L.fortis_sync()
    t0 = time.perf_counter()
    ms = plan.time_ms(args.steps, graph=False)
    L.fortis_sync()
    dt = time.perf_counter() - t0
    avg = ms / args.steps
    achieved = case["flops"] / (avg * 1e-3) / 1e12
    out = dict(rows=case["rows"], dt=dt, dtype="f32",
               config={"workload": "toy_mlp_1024x64_256_256_32", "columns": case["rows"], "launches_per_step": plan.num_kernels},
               roofline=dict(bound="mfma", kernel="mlp_chain (LDS-resident, fp32 MFMA)", achieved=round(achieved, 4),
                             peak=PEAK_F32_MFMA_TFLOPS, unit="TFLOP/s", frac=round(achieved / PEAK_F32_MFMA_TFLOPS, 5),
                             avg_launch_ms=round(avg, 5), flop_per_launch=case["flops"], **traffic("toy")))
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_both(case, case["rows"], case["X"], 3.0, 2.0)
    plan.close()
    return out


def run_zb(L, args, reference_net=False):
    """gather -> MLP -> scatter for all 15 layers of the reference geometry in one kernel."""
    from fortis_amd import configs, plan as P, stencil as S
    g = os.path.join(ROOT, "tests", "golden")
    if args.grid:
        # the same step on a larger synthetic grid (descriptors in the reference's schema)
        sx, sy, nz = (int(v) for v in args.grid.lower().split("x"))
        gd, sd, lp, kd = configs.zb_descriptors(sx, sy, nz)
        gt, st = S.build_table(gd, lp, kd, "gather"), S.build_table(sd, lp, kd, "scatter")
    else:
        sx, sy, nz = 68, 78, 15
        gt, st, gd, sd, lp, kd = S.load_tables(f"{g}/zb_gather.json", f"{g}/zb_scatter.json", f"{g}/zb_loop.json", f"{g}/zb_kdist.json")
    A = configs.zb_arrays(sx, sy, nz)
    rows = gt.count * gt.nk
    if reference_net:
        W = np.load(f"{g}/zb_nn.npz")
        net = dict(Ws=[W["A0"], W["A1"]], bs=[W["b0"], W["b1"]], acts=["relu", None], widths=[27, 20, 3])
        plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows, in_norms=W["in_norms"], out_norms=W["out_norms"])
        extra = dict(in_norms=W["in_norms"], out_norms=W["out_norms"])
    else:
        net = configs.zb_mlp()
        plan = P.mlp_plan(net["Ws"], net["bs"], net["acts"], rows)
        extra = {}
    garr = [A["sh_xy_h"], A["sh_xx"], A["vort_xy_h"], A["norm_h"]]
    n3 = sx * sy * nz
    sarr = [A["norm_h"], A["kappa_h"], np.zeros(n3, np.float32), np.zeros(n3, np.float32), np.zeros(n3, np.float32)]

    held = []

    def dev(a):
        d = L.fortis_alloc(a.nbytes)
        L.fortis_h2d(d, a.ctypes.data, a.nbytes)
        held.append(d)
        return d
    dG = (C.c_void_p * 4)(*[dev(a) for a in garr])
    dS = (C.c_void_p * 5)(*[dev(a) for a in sarr])
    L.fortis_stencil_step_fused_time_ms(C.byref(gt), C.byref(st), plan.handle, dG, dS, None, max(1, args.warmup))
    L.fortis_sync()
    t0 = time.perf_counter()
    ms = L.fortis_stencil_step_fused_time_ms(C.byref(gt), C.byref(st), plan.handle, dG, dS, None, args.steps)
    L.fortis_sync()
    dt = time.perf_counter() - t0
    avg = ms / args.steps          # the helper runs one validating launch before the clocked ones
    widths = net["widths"]
    flops = 2 * rows * sum(widths[i] * widths[i + 1] for i in range(len(widths) - 1))
    # algorithmic bytes: 4 input planes + kappa read once, 3 output values per cell written, weights once
    nbytes = 4 * (4 * n3 + sx * sy + 3 * rows + sum(w.size + b.size for w, b in zip(net["Ws"], net["bs"])))
    tf, gbs = flops / (avg * 1e-3) / 1e12, nbytes / (avg * 1e-3) / 1e9
    # the fused kernel's arithmetic intensity decides the bound: flop/byte against 157.3e12 / 8e12 = 19.7
    bound = "mfma" if flops / nbytes > PEAK_F32_MFMA_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9) else "hbm"
    roof = dict(bound=bound, kernel="mlp_chain<stencil> (gather -> MLP -> scatter, one launch)",
                achieved=round(tf if bound == "mfma" else gbs, 3), peak=PEAK_F32_MFMA_TFLOPS if bound == "mfma" else PEAK_HBM_GBS,
                unit="TFLOP/s" if bound == "mfma" else "GB/s",
                frac=round((tf / PEAK_F32_MFMA_TFLOPS) if bound == "mfma" else (gbs / PEAK_HBM_GBS), 5),
                avg_launch_ms=round(avg, 5), flop_per_launch=flops, bytes_per_launch=nbytes,
                hbm_GBs=round(gbs, 2), mfma_TFLOPs=round(tf, 3), **traffic(("zb_ref" if reference_net else "zb") + ("_%dx%dx%d" % (sx, sy, nz) if args.grid else "")))
    # dt covers the validating launch too; whole-job throughput uses the clocked launches only
    out = dict(rows=rows, dt=ms * 1e-3, wall_dt=dt, dtype="f32",
               config={"workload": "zb_gather_mlp_scatter_%s_%dx%dx%d" % ("27_20_3" if reference_net else "27_64_64_3", sx, sy, nz),
                       "columns": rows, "cells_per_layer": int(gt.count), "layers": int(gt.nk), "widths": widths,
                       "launches_per_step": 1},
               roofline=roof)
    if not args.no_cpu:
        ref = cpu_baseline_zb_reference() if (reference_net and not args.grid) else None
        if ref:
            out["cpu_baseline"] = ref
        else:
            from oracle import oracle as O
            X = O.stencil_gather(gd, garr, int(gt.count), int(gt.nk), 3, 3, 64)
            case = dict(net, rows=rows)
            out["cpu_baseline"] = cpu_baseline_both(case, rows, X, 5.0, 3.0, **extra)
            out["cpu_baseline"]["sample"] += " (MLP part only; the gather and scatter loops of the host are not included)"
    plan.close()
    for d in held:
        L.fortis_free(d)
    return out


def cpu_baseline_zb_reference(min_seconds=10.0):
    """The reference's own CPU path for this very step: its native Fortran host (mom6_zb/zb_host.f90 with
    fwd_native_zb.f90, compiled unchanged by oracle/build_ref.sh) on the reference geometry and network,
    which times 10 steps itself ('per-step ms').  Single-threaded, as the reference runs it.  None if the
    binary was not built."""
    import re
    import subprocess
    import tempfile
    exe = os.path.join(ROOT, "oracle", "_ref", "zb_native4")
    if not os.path.exists(exe):
        return None
    W = np.load(os.path.join(ROOT, "tests", "golden", "zb_nn.npz"))
    ms, runs, t0 = [], 0, time.perf_counter()
    with tempfile.TemporaryDirectory() as td:
        with open(os.path.join(td, "zb_nn.bin"), "wb") as o:      # layout of mom6_zb/make_zb_weights.py:12-17
            for a in (W["A0"].T, W["b0"], W["A1"].T, W["b1"], W["in_norms"], W["out_norms"]):
                o.write(np.ascontiguousarray(a, dtype=np.float32).tobytes())
        while time.perf_counter() - t0 < min_seconds:
            r = subprocess.run([exe], cwd=td, capture_output=True, text=True, timeout=120)
            m = re.search(r"per-step ms:\s*([-0-9.Ee+]+)", r.stdout)
            if r.returncode != 0 or not m:
                return None
            ms.append(float(m.group(1)))
            runs += 1
    per_step = float(np.median(ms))
    return {"value": 71040 / (per_step * 1e-3), "unit": "columns/s", "cores": 1, "kind": "reference",
            "sample": "%d runs of the reference's native Fortran ZB host (zb_host.f90 + fwd_native_zb.f90, flang -O2), each timing 10 whole "
                      "steps (stencil packing, 27->20->3 forward, de-scaling and stores on 71040 cells); median %.2f ms per step" % (runs, per_step)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20, help="untimed steps first; the clocks need about ten steps of this size to settle")
    ap.add_argument("--workload", default=None, help="default: climsim, followed by short runs of the other configurations (others)", choices=["climsim", "zb", "zb_ref", "zb_unfused", "toy", "copy", "unet", "tsrgan", "climsim_host", "zb_host"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-others", action="store_true", help="skip the short runs of the other configurations that follow the default workload")
    ap.add_argument("--f64", action="store_true", help="zb_unfused only: double-precision host arrays (the general stencil kernels)")
    ap.add_argument("--grid", default=None, help="zb / zb_ref / zb_unfused only: SXxSYxNZ grid instead of the reference's 68x78x15 (zb_unfused: 1028x1028x15)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the fused step on ONE GPU; --gpus %d is not supported "
              "(the path has no inter-GPU exchange to measure)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import fortis_amd
    L = fortis_amd.load()
    name = C.create_string_buffer(64)
    if L.fortis_device_info(name, 64, None) != 0:
        print("bench.py: no GPU visible; the HIP path has no CPU fallback", file=sys.stderr)
        sys.exit(3)
    with_others = args.workload is None and not args.no_others
    args.workload = args.workload or "climsim"
    r = run_workload(L, args, args.workload)
    ms_per_step = r["dt"] / args.steps * 1e3
    unit = r.get("unit", "columns/s")
    line = {"metric": r.get("metric", "%s per fused forward step" % unit.replace("/s", "/sec")), "value": r.get("value", r["rows"] * args.steps / r["dt"]), "unit": unit,
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": r["dtype"], "data": "synthetic", "device": name.value.decode(),
            "config": r["config"], "roofline": r["roofline"]}
    if "cpu_baseline" in r:
        line["cpu_baseline"] = r["cpu_baseline"]
    if with_others:
        line["others"] = run_others(L, args)
    if L.fortis_error_count():
        raise SystemExit("bench.py: %d HIP call(s) failed during the run (see stderr): no figure reported" % L.fortis_error_count())
    print(json.dumps(line))


def run_workload(L, args, workload):
    if workload == "climsim":
        return run_climsim(L, args)
    if workload == "toy":
        return run_toy(L, args)
    if workload == "copy":
        return run_copy(L, args)
    if workload in ("unet", "tsrgan"):
        return run_conv(L, args, workload)
    if workload == "zb_unfused":
        return run_zb_unfused(L, args)
    if workload == "climsim_host":
        return run_climsim_host(L, args)
    if workload == "zb_host":
        return run_zb_host_step(L, args)
    return run_zb(L, args, reference_net=(workload == "zb_ref"))


# The other configurations and kernels of the path, each run for a few steps after the headline so that every
# figure quoted for them is clocked in the same process as the headline: (label, workload, grid, steps, warm-up).
OTHERS = [("toy 1024x(64-256-256-32)", "toy", None, 200, 50),
          ("zb 68x78x15 fused, 27-64-64-3", "zb", None, 200, 50),
          ("zb 68x78x15 fused, reference net 27-20-3", "zb_ref", None, 200, 50),
          ("zb 1028x1028x15 fused, 27-64-64-3", "zb", "1028x1028x15", 40, 20),
          ("zb 1028x1028x15 fused, reference net 27-20-3", "zb_ref", "1028x1028x15", 40, 20),
          ("zb 1028x1028x15 unfused (gather kernel is the roofline)", "zb_unfused", "1028x1028x15", 20, 10),
          ("unet 1x4x256x256", "unet", None, 100, 30),
          ("tsrgan 33^3 -> 66^3", "tsrgan", None, 40, 15),
          ("climsim whole-array call on host arrays (PCIe-inclusive)", "climsim_host", None, 20, 3),
          ("zb host step through the entries (PCIe-inclusive)", "zb_host", None, 100, 10)]


def run_others(L, args):
    out = []
    for label, workload, grid, steps, warmup in OTHERS:
        a = argparse.Namespace(**vars(args))
        a.grid, a.steps, a.warmup, a.no_cpu, a.f64 = grid, steps, warmup, True, False
        L.fortis_sync()
        L.fortis_pool_trim()          # every workload starts on fresh device memory, as when it is run alone
        r = run_workload(L, a, workload)
        roof = r["roofline"]
        out.append({"workload": r["config"]["workload"], "label": label, "steps": steps, "ms_per_step": round(r["dt"] / steps * 1e3, 5),
                    "value": r["rows"] * steps / r["dt"], "unit": r.get("unit", "columns/s"), "bound": roof["bound"],
                    "kernel": roof["kernel"], "achieved": roof["achieved"], "peak": roof["peak"], "roofline_unit": roof["unit"],
                    "frac": roof["frac"], "avg_launch_ms": roof["avg_launch_ms"]})
        for k in ("back_to_back_ms", "back_to_back_frac", "scatter_GBs", "scatter_frac", "scatter_ms_all_layers", "mlp_ms"):     # the unfused step's other parts
            if k in roof:
                out[-1][k] = roof[k]
    return out


if __name__ == "__main__":
    main()
