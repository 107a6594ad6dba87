"""The FORTIS_BACKEND=hip shim generator on the CPU: the attribute grammar of driver/fortis_hostattr.py:11-28
read with the semantics of driver/fortis_shim.py:9-38, the host facts it derives for every verdict
(fortis_shim.py:94-133), and that the emitted step file compiles against the public header."""
import json
import os
import subprocess

import numpy as np
import pytest

from fortis_amd import configs, emit, shim_hip as SH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# hand-written in the syntax fortis_hostattr.py prints (not produced by emit.host_attr)
ZB_ATTR = ('fortis.host = {version = 1 : i64, shape = [27], batch = 71040 : i64, repeat = 0 : i64, verdict = "batched", '
           'provenance = {shape = "proven", repeat = "proven", dependence = "proven", lift = "proven", layout = "proven", scope = "proven", '
           'aliasing = "checked", purity = "checked", fp_order = "assumed"}, '
           'loop = {lo = 1 : i64, step = 1 : i64, count = 71040 : i64, minc = 1 : i64, in = "_QFEx", out = "_QFEy", post_download = false}, '
           'expand = {in = "_QFEx", out = "_QFEy", count = 71040 : i64, nin = 27 : i64, nout = 3 : i64}}, fortis.graph = true')


def _module(attr, sig="%arg0: tensor<71040x27xf32>, %arg1: tensor<20x27xf32>, %arg2: tensor<71040x3xf32>"):
    return "module {\n  func.func @mlp_kernel(%s) attributes {%s} {\n    return\n  }\n}\n" % (sig, attr)


def test_attribute_grammar():
    v, end = SH.parse_attr('{a = 1 : i64, b = [1, 2, -3], c = "x y", d = {e = true, f = false}, g.h = []}')
    assert v == {"a": 1, "b": [1, 2, -3], "c": "x y", "d": {"e": True, "f": False}, "g.h": []} and end == 77
    assert SH.parse_attr("  [ ]")[0] == [] and SH.parse_attr("{}")[0] == {}
    assert SH.parse_attr("-12 : i32, rest")[0] == -12
    for bad in ("{a = }", '{a = "unterminated}', "{a 1}", "[1 2]", "{a = 1.5}", "{a = 1"):
        with pytest.raises((SH.AttrError, IndexError)):
            SH.parse_attr(bad)
    A = SH.func_attrs(_module(ZB_ATTR))
    assert A["fortis.graph"] is True and A["fortis.host"]["loop"]["count"] == 71040 and A["fortis.host"]["expand"]["nout"] == 3
    assert SH.func_attrs("module { func.func @other() { return } }") == {}
    assert SH.func_attrs("func.func @mlp_kernel(%a: tensor<4xf32>) {\n}") == {}


OUTLINE = dict(inputs=["tensor<71040x27xf32>"], weights=["tensor<20x27xf32>"], output="tensor<71040x3xf32>")


def test_host_facts_per_verdict():
    A = SH.func_attrs(_module(ZB_ATTR))
    f, g = SH.host_facts(A, OUTLINE, env={})
    assert g == [] and f == dict(n_in=71040 * 27, n_out=71040 * 3, in_esz=4, out_esz=4, verdict="FORTIS_VERDICT_BATCHED", expanded=1,
                                 count=71040, lo=1, step=1, minc=1, graph=1, gather=0, scatter=0)
    f, _ = SH.host_facts(A, OUTLINE, env={"FORTIS_GATHER": "1", "FORTIS_SCATTER": "1"})          # fortis_shim.py:107-112
    assert (f["gather"], f["scatter"]) == (1, 1)
    # batched, slice form, strided loop (fortis_shim.py:116-121): no expand block
    strided = ('fortis.host = {version = 1 : i64, shape = [64], batch = 100 : i64, repeat = 0 : i64, verdict = "batched", '
               'loop = {lo = 3 : i64, step = -2 : i64, count = 100 : i64, minc = 3 : i64, in = "a", out = "b", post_download = true}}')
    f, _ = SH.host_facts(SH.func_attrs(_module(strided)), dict(inputs=["tensor<100x64xf32>"], weights=[], output="tensor<100x32xf32>"), env={"FORTIS_GATHER": "1"})
    assert (f["verdict"], f["expanded"], f["count"], f["lo"], f["step"], f["minc"], f["graph"], f["gather"]) == ("FORTIS_VERDICT_BATCHED", 0, 100, 3, -2, 3, 0, 0)
    # whole-array call; a rejected / disabled loop verdict is a whole-array call too (fortis_shim.py:123)
    for v in ("whole", "reject", "block", "disabled"):
        whole = 'fortis.host = {version = 1 : i64, shape = [1, 1024], batch = 1 : i64, repeat = 1000 : i64, verdict = "%s"}' % v
        f, _ = SH.host_facts(SH.func_attrs(_module(whole)), dict(inputs=["tensor<1x1024xf32>"], weights=[], output="tensor<1x1024xf32>"), env={})
        assert (f["verdict"], f["n_in"], f["count"]) == ("FORTIS_VERDICT_WHOLE", 1024, 0)
    # boundary: host element types from the tensor types, pre + post globals are the model's extra inputs
    bnd = ('fortis.host = {version = 1 : i64, shape = [384, 124], batch = 1 : i64, repeat = 0 : i64, verdict = "boundary", '
           'boundary = {in = "colmajor", in_elt = "f64", out = "colmajor", out_elt = "f64", pre = ["m", "hi", "lo"], post = ["s"]}}')
    ol = dict(inputs=["tensor<384x124xf64>", "tensor<124xf64>", "tensor<124xf64>", "tensor<124xf64>", "tensor<128xf64>"], weights=[], output="tensor<384x128xf64>")
    f, g = SH.host_facts(SH.func_attrs(_module(bnd)), ol, env={})
    assert g == ["m", "hi", "lo", "s"] and (f["verdict"], f["in_esz"], f["out_esz"], f["n_out"]) == ("FORTIS_VERDICT_BOUNDARY", 8, 8, 384 * 128)
    with pytest.raises(ValueError):                                   # fortis_shim.py:58: globals must match the extra inputs
        SH.host_facts(SH.func_attrs(_module(bnd)), dict(ol, inputs=ol["inputs"][:3]), env={})
    lifted = ZB_ATTR.replace("}, fortis.graph", ', lift = {globals = ["in_n", "out_n"], in = "_QFEx"}}, fortis.graph')
    f, g = SH.host_facts(SH.func_attrs(_module(lifted)), dict(OUTLINE, inputs=OUTLINE["inputs"] + ["tensor<27xf32>", "tensor<3xf32>"]), env={})
    assert g == ["in_n", "out_n"]


def _compile(path, tmp_path):
    r = subprocess.run(["gcc", "-Wall", "-Werror", "-c", "-I", os.path.join(ROOT, "include"), path, "-o", str(tmp_path / "o.o")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_cli_on_hand_written_inputs(tmp_path):
    """python -m fortis_amd.shim_hip m4.mlir outline.json outdir, as fortisc would call it (fortisc.in:53-54)."""
    (tmp_path / "m4.mlir").write_text(_module(ZB_ATTR.replace("}, fortis.graph", ', lift = {globals = ["zb_in_norms", "zb_out_norms"], in = "x"}}, fortis.graph'),
                                              "%a: tensor<71040x27xf32>, %n0: tensor<27xf32>, %n1: tensor<3xf32>, %w0: tensor<20x27xf32>, %w1: tensor<20xf32>, "
                                              "%w2: tensor<3x20xf32>, %w3: tensor<3xf32>, %o: tensor<71040x3xf32>"))
    json.dump(dict(inputs=["tensor<71040x27xf32>", "tensor<27xf32>", "tensor<3xf32>"],
                   weights=["tensor<20x27xf32>", "tensor<20xf32>", "tensor<3x20xf32>", "tensor<3xf32>"], output="tensor<71040x3xf32>"),
              open(tmp_path / "outline.json", "w"))
    rows = 71040
    ops = dict(tensors=[dict(elems=rows * 27), dict(elems=rows * 27), dict(elems=rows * 20), dict(elems=rows * 3), dict(elems=rows * 3)], input=0, output=4,
               ops=[dict(op="scale", src=0, dst=1, vec="g0", rows=rows, n=27, divide=True),
                    dict(op="linear", src=1, dst=2, w="w0", b="w1", B=rows, K=27, N=20, act="relu", alpha=0.0),
                    dict(op="linear", src=2, dst=3, w="w2", b="w3", B=rows, K=20, N=3, act="none"),
                    dict(op="scale", src=3, dst=4, vec="g1", rows=rows, n=3, divide=False)])
    json.dump(ops, open(tmp_path / "ops.json", "w"))
    env = dict(os.environ, FORTIS_GATHER="1", FORTIS_SCATTER="1", PYTHONPATH=ROOT)
    r = subprocess.run([os.sys.executable, "-m", "fortis_amd.shim_hip", str(tmp_path / "m4.mlir"), str(tmp_path / "outline.json"), str(tmp_path)],
                       capture_output=True, text=True, env=env)
    assert r.returncode == 0, r.stderr
    assert r.stdout.startswith("shim[hip]: verdict=batched batch=71040 repeat=0 graph=1 in=tensor<71040x27xf32> out=tensor<71040x3xf32>")
    text = (tmp_path / "step_tables.c").read_text()
    assert "extern float w0[], w1[], w2[], w3[];" in text and "extern float zb_in_norms[];" in text and "extern float zb_out_norms[];" in text
    assert "fortis_plan_scale(p, t[0], t[1], zb_in_norms, 71040L, 27, 1)" in text
    assert "fortis_plan_linear(p, t[1], t[2], w0, w1, 71040L, 27, 20, 1, 0.0f)" in text
    assert ".verdict = FORTIS_VERDICT_BATCHED" in text and ".expanded = 1, .count = 71040L" in text and ".graph = 1, .gather = 1, .scatter = 1" in text
    assert "fortis_step_on_first_use(fortis_bind_step)" in text
    _compile(str(tmp_path / "step_tables.c"), tmp_path)
    assert "-lfortis_rt" in (tmp_path / "link_hip.txt").read_text() and "cudart" not in (tmp_path / "link_hip.txt").read_text()


def test_generator_refuses_inconsistent_inputs(tmp_path):
    A = SH.func_attrs(_module(ZB_ATTR))
    base = dict(tensors=[dict(elems=71040 * 27), dict(elems=71040 * 3)], input=0, output=1,
                ops=[dict(op="linear", src=0, dst=1, w="w0", b=None, B=71040, K=27, N=3, act="none")])
    SH.emit_step(A, OUTLINE, base, env={})
    for edit, msg in ((lambda o: o["ops"][0].update(w="w5"), "lists 1 weights"), (lambda o: o["ops"][0].update(w="g0"), "host globals"),
                      (lambda o: o["ops"][0].update(op="softmax"), "unknown op"), (lambda o: o["ops"][0].update(dst=7), "names tensor"),
                      (lambda o: o["ops"][0].update(act="gelu"), "unknown activation"), (lambda o: o["tensors"][0].update(elems=5), "smaller than"),
                      (lambda o: o.update(ops=[]), "empty model")):
        o = json.loads(json.dumps(base))
        edit(o)
        with pytest.raises(ValueError, match=msg):
            SH.emit_step(A, OUTLINE, o, env={})
    with pytest.raises(ValueError, match="does not divide"):
        SH.emit_step(SH.func_attrs(_module(ZB_ATTR.replace("count = 71040", "count = 71041"))), OUTLINE, base, env={})


@pytest.mark.parametrize("which", ["unet", "tsrgan", "climsim"])
def test_conv_stacks_and_wide_mlp_emit_and_compile(tmp_path, which):
    """Every op kind the plan accepts comes out of the generator: conv2d with BatchNorm vectors, transposed conv,
    max pool, tensor windows (UNet); permute, conv3d with residuals, upsample (TSRGAN); linear stacks (ClimSim)."""
    if which == "unet":
        case = configs.unet(H=32, chans=(8, 16, 24, 32))
        ol = configs.unet_plan(case, plan_cls=SH.OpList)
        tin, tout = "tensor<1x4x32x32xf32>", "tensor<1x4x32x32xf32>"
    elif which == "tsrgan":
        case = configs.tsrgan(D=9, ch=16, nblocks=2)
        ol = configs.tsrgan_plan(case, plan_cls=SH.OpList)
        tin, tout = "tensor<1x9x9x9x3xf32>", "tensor<1x18x18x18x3xf32>"
    else:
        case = configs.climsim(rows=64)
        ol = configs.climsim_plan(case, boundary=False, plan_cls=SH.OpList)
        tin, tout = "tensor<64x556xf32>", "tensor<64x368xf32>"
    cs = emit.step_files(str(tmp_path), ol, emit.host_attr("whole", graph=True), tin, tout)
    text = open(cs[0]).read()
    kinds = {"unet": ("fortis_plan_conv2d", "fortis_plan_convt2d", "fortis_plan_maxpool2d", "fortis_plan_view"),
             "tsrgan": ("fortis_plan_permute", "fortis_plan_conv3d", "fortis_plan_upsample"), "climsim": ("fortis_plan_linear",)}[which]
    for k in kinds:
        assert k + "(" in text
    assert len(ol.weights) == len(json.load(open(tmp_path / "outline.json"))["weights"])
    for c in cs:
        _compile(c, tmp_path)
