"""The reader that names the operations of a model's linalg text (fortis_amd/mlir_ops.py), on hand-written
snippets in the statement forms of the torch-mlir exporter and of driver/fortis_emit2d.py:20-52.  The reference
checks in no .mlir file, so these snippets, not a reference fixture, are what the reader is held to; what it
writes must be the op list that the same model gives through the Plan interface, and the generator must take it."""
import json

import numpy as np
import pytest

from fortis_amd import mlir_ops as M, plan as P, shim_hip as SH

MAPS2 = "affine_map<(d0, d1) -> (d0, d1)>"
BCAST = "affine_map<(d0, d1) -> (d1)>"


def _linear(x, w, b, B, K, N, n, act=None):
    """torch-mlir's nn.Linear (+ activation): transpose, zero fill, matmul, broadcast bias add."""
    t = f"""
    %e{n} = tensor.empty() : tensor<{K}x{N}xf32>
    %wt{n} = linalg.transpose ins({w} : tensor<{N}x{K}xf32>) outs(%e{n} : tensor<{K}x{N}xf32>) permutation = [1, 0]
    %o{n} = tensor.empty() : tensor<{B}x{N}xf32>
    %z{n} = linalg.fill ins(%cst : f32) outs(%o{n} : tensor<{B}x{N}xf32>) -> tensor<{B}x{N}xf32>
    %mm{n} = linalg.matmul ins({x}, %wt{n} : tensor<{B}x{K}xf32>, tensor<{K}x{N}xf32>) outs(%z{n} : tensor<{B}x{N}xf32>) -> tensor<{B}x{N}xf32>
    %l{n} = linalg.generic {{indexing_maps = [{MAPS2}, {BCAST}, {MAPS2}], iterator_types = ["parallel", "parallel"]}} ins(%mm{n}, {b} : tensor<{B}x{N}xf32>, tensor<{N}xf32>) outs(%o{n} : tensor<{B}x{N}xf32>) {{
    ^bb0(%in: f32, %in_0: f32, %out: f32):
      %s = arith.addf %in, %in_0 : f32
      linalg.yield %s : f32
    }} -> tensor<{B}x{N}xf32>"""
    res = f"%l{n}"
    if act == "relu":
        t += f"""
    %a{n} = linalg.generic {{indexing_maps = [{MAPS2}, {MAPS2}], iterator_types = ["parallel", "parallel"]}} ins(%l{n} : tensor<{B}x{N}xf32>) outs(%o{n} : tensor<{B}x{N}xf32>) {{
    ^bb0(%in: f32, %out: f32):
      %c = arith.cmpf ugt, %in, %cst : f32
      %s = arith.select %c, %in, %cst : f32
      linalg.yield %s : f32
    }} -> tensor<{B}x{N}xf32>"""
        res = f"%a{n}"
    elif act == "leaky":
        t += f"""
    %a{n} = linalg.generic {{indexing_maps = [{MAPS2}, {MAPS2}], iterator_types = ["parallel", "parallel"]}} ins(%l{n} : tensor<{B}x{N}xf32>) outs(%o{n} : tensor<{B}x{N}xf32>) {{
    ^bb0(%in: f32, %out: f32):
      %c = arith.cmpf ugt, %in, %cst : f32
      %m = arith.mulf %in, %cst_15 : f32
      %s = arith.select %c, %in, %m : f32
      linalg.yield %s : f32
    }} -> tensor<{B}x{N}xf32>"""
        res = f"%a{n}"
    return t, res


def _scale(x, v, B, N, n, op):
    return f"""
    %se{n} = tensor.empty() : tensor<{B}x{N}xf32>
    %sc{n} = linalg.generic {{indexing_maps = [{MAPS2}, {BCAST}, {MAPS2}], iterator_types = ["parallel", "parallel"]}} ins({x}, {v} : tensor<{B}x{N}xf32>, tensor<{N}xf32>) outs(%se{n} : tensor<{B}x{N}xf32>) {{
    ^bb0(%in: f32, %in_0: f32, %out: f32):
      %s = arith.{op} %in, %in_0 : f32
      linalg.yield %s : f32
    }} -> tensor<{B}x{N}xf32>""", f"%sc{n}"


def test_zb_shaped_mlp_text_gives_the_plan_interface_op_list(tmp_path):
    """x / in_norms -> Linear + ReLU -> Linear -> * out_norms (mom6_zb/export_zb.py:10-16) with outlined weights
    (driver/fortis_outline.py:20-24: constants become trailing arguments in order of appearance)."""
    B = 4736
    body = "\n    %cst = arith.constant 0.000000e+00 : f32"
    t, v = _scale("%arg0", "%w0", B, 27, 0, "divf"); body += t
    t, v = _linear(v, "%w1", "%w2", B, 27, 20, 1, "relu"); body += t
    t, v = _linear(v, "%w3", "%w4", B, 20, 3, 2); body += t
    t, v = _scale(v, "%w5", B, 3, 3, "mulf"); body += t
    src = ("module {\n  func.func @mlp_kernel(%arg0: tensor<4736x27xf32>, %w0: tensor<27xf32>, %w1: tensor<20x27xf32>, %w2: tensor<20xf32>, "
           "%w3: tensor<3x20xf32>, %w4: tensor<3xf32>, %w5: tensor<3xf32>) -> tensor<4736x3xf32> attributes {fortis.host = {version = 1 : i64, verdict = \"whole\"}} {"
           + body + f"\n    return {v} : tensor<4736x3xf32>\n  }}\n}}\n")
    outline = dict(inputs=["tensor<4736x27xf32>"], weights=["tensor<27xf32>", "tensor<20x27xf32>", "tensor<20xf32>", "tensor<3x20xf32>", "tensor<3xf32>", "tensor<3xf32>"],
                   output="tensor<4736x3xf32>")
    got = M.read_ops(src, outline).as_json()
    rng = np.random.default_rng(0)
    Ws, bs = [rng.standard_normal((20, 27)), rng.standard_normal((3, 20))], [rng.standard_normal(20), rng.standard_normal(3)]
    want = P.mlp_plan(Ws, bs, ["relu", None], B, in_norms=rng.standard_normal(27), out_norms=rng.standard_normal(3), plan_cls=SH.OpList).as_json()
    assert [o["op"] for o in got["ops"]] == ["scale", "linear", "linear", "scale"]
    strip = lambda o: {k: v for k, v in o.items() if k not in ("src", "dst")}
    assert [strip(o) for o in got["ops"]] == [strip(o) for o in want["ops"]]
    # same data flow: every op reads what the one before wrote, from the model's input to its output
    assert got["ops"][0]["src"] == got["input"] and got["ops"][-1]["dst"] == got["output"]
    for a, b in zip(got["ops"][:-1], got["ops"][1:]):
        assert a["dst"] == b["src"]
    assert [t["elems"] for t in got["tensors"]] == [B * 27, B * 27, B * 20, B * 3, B * 3]
    # and the generator takes it
    attrs = SH.func_attrs(src)
    text, facts = SH.emit_step(attrs, outline, got)
    assert "fortis_plan_linear(p, t[1], t[2], w1, w2, 4736L, 27, 20, 1, 0.0f)" in text and facts["n_out"] == B * 3
    (tmp_path / "m.mlir").write_text(src)
    (tmp_path / "outline.json").write_text(json.dumps(outline))
    M.generate(str(tmp_path / "m.mlir"), str(tmp_path / "outline.json"), str(tmp_path))
    assert json.load(open(tmp_path / "ops.json")) == got


def test_boundary_wrapper_text_of_the_reference_emitter():
    """@fortis_main in the text driver/fortis_emit2d.py:20-52 prints (transposing generics, lifted expressions over
    the extra arguments, truncf / extf) around a LeakyReLU model: f64 host arrays (384, 124) -> (384, 128)."""
    NI, NIN, NH, NOUT = 384, 124, 128, 128
    inner = "\n    %cst = arith.constant 0.000000e+00 : f32\n    %cst_15 = arith.constant 1.500000e-01 : f32"
    t, v = _linear("%arg0", "%w0", "%w1", NI, NIN, NH, 0, "leaky"); inner += t
    t, v = _linear(v, "%w2", "%w3", NI, NH, NOUT, 1); inner += t
    T2 = "affine_map<(d0, d1) -> (d1, d0)>"
    G1, G0 = "affine_map<(d0, d1) -> (d1)>", "affine_map<(d0, d1) -> (d0)>"
    src = f"""module {{
  func.func private @forward(%arg0: tensor<{NI}x{NIN}xf32>, %w0: tensor<{NH}x{NIN}xf32>, %w1: tensor<{NH}xf32>, %w2: tensor<{NOUT}x{NH}xf32>, %w3: tensor<{NOUT}xf32>) -> tensor<{NI}x{NOUT}xf32> {{{inner}
    return {v} : tensor<{NI}x{NOUT}xf32>
  }}
  func.func @fortis_main(%x: tensor<{NIN}x{NI}xf64>, %preG0: tensor<{NIN}xf64>, %preG1: tensor<{NIN}xf64>, %preG2: tensor<{NIN}xf64>, %postG0: tensor<{NOUT}xf64>) -> tensor<{NOUT}x{NI}xf64> {{
    %pree = tensor.empty() : tensor<{NI}x{NIN}xf32>
    %prer = linalg.generic {{indexing_maps = [{T2}, {G1}, {G1}, {G1}, {MAPS2}], iterator_types = ["parallel", "parallel"]}} ins(%x, %preG0, %preG1, %preG2 : tensor<{NIN}x{NI}xf64>, tensor<{NIN}xf64>, tensor<{NIN}xf64>, tensor<{NIN}xf64>) outs(%pree : tensor<{NI}x{NIN}xf32>) {{
    ^bb0(%a: f64, %g0: f64, %g1: f64, %g2: f64, %o: f32):
      %prev1 = arith.subf %a, %g0 : f64
      %prev2 = arith.subf %g1, %g2 : f64
      %prev3 = arith.divf %prev1, %prev2 : f64
      %preout = arith.truncf %prev3 : f64 to f32
      linalg.yield %preout : f32
    }} -> tensor<{NI}x{NIN}xf32>
    %y0 = call @forward(%prer) : (tensor<{NI}x{NIN}xf32>) -> tensor<{NI}x{NOUT}xf32>
    %poste = tensor.empty() : tensor<{NOUT}x{NI}xf64>
    %postr = linalg.generic {{indexing_maps = [{T2}, {G0}, {MAPS2}], iterator_types = ["parallel", "parallel"]}} ins(%y0, %postG0 : tensor<{NI}x{NOUT}xf32>, tensor<{NOUT}xf64>) outs(%poste : tensor<{NOUT}x{NI}xf64>) {{
    ^bb0(%a: f32, %g0: f64, %o: f64):
      %postin = arith.extf %a : f32 to f64
      %postv1 = arith.divf %postin, %g0 : f64
      linalg.yield %postv1 : f64
    }} -> tensor<{NOUT}x{NI}xf64>
    return %postr : tensor<{NOUT}x{NI}xf64>
  }}
}}
"""
    outline = dict(inputs=[f"tensor<{NIN}x{NI}xf64>"] + [f"tensor<{NIN}xf64>"] * 3 + [f"tensor<{NOUT}xf64>"],
                   weights=[f"tensor<{NH}x{NIN}xf32>", f"tensor<{NH}xf32>", f"tensor<{NOUT}x{NH}xf32>", f"tensor<{NOUT}xf32>"], output=f"tensor<{NOUT}x{NI}xf64>")
    got = M.read_ops(src, outline).as_json()
    assert [o["op"] for o in got["ops"]] == ["boundary_pre", "linear", "linear", "boundary_post"]
    pre, l0, l1, post = got["ops"]
    assert (pre["NI"], pre["NK"], pre["esz"], pre["mean"], pre["vmax"], pre["vmin"]) == (NI, NIN, 8, "g0", "g1", "g2")
    assert (post["NI"], post["NK"], post["esz"], post["scale"]) == (NI, NOUT, 8, "g3")
    assert (l0["act"], l0["alpha"], l0["w"], l0["b"], l1["act"], l1["w"], l1["b"]) == ("leaky", pytest.approx(0.15), "w0", "w1", "none", "w2", "w3")
    assert got["tensors"][got["input"]] == dict(elems=NI * NIN, esz=8) and got["tensors"][got["output"]] == dict(elems=NI * NOUT, esz=8)
    assert pre["dst"] == l0["src"] and l0["dst"] == l1["src"] and l1["dst"] == post["src"]


def test_conv_text_with_pad_bias_and_pool():
    """Conv2d(4 -> 8, 3 x 3, pad 1) with its bias broadcast as the accumulator's start, ReLU, 2 x 2 max pool."""
    src = """module {
  func.func @mlp_kernel(%arg0: tensor<1x4x16x16xf32>, %w0: tensor<8x4x3x3xf32>, %w1: tensor<8xf32>) -> tensor<1x8x8x8xf32> {
    %cst = arith.constant 0.000000e+00 : f32
    %cst_0 = arith.constant 0xFF800000 : f32
    %padded = tensor.pad %arg0 low[0, 0, 1, 1] high[0, 0, 1, 1] {
    ^bb0(%a0: index, %a1: index, %a2: index, %a3: index):
      tensor.yield %cst : f32
    } : tensor<1x4x16x16xf32> to tensor<1x4x18x18xf32>
    %0 = tensor.empty() : tensor<1x8x16x16xf32>
    %1 = linalg.generic {indexing_maps = [affine_map<(d0, d1, d2, d3) -> (d1)>, affine_map<(d0, d1, d2, d3) -> (d0, d1, d2, d3)>], iterator_types = ["parallel", "parallel", "parallel", "parallel"]} ins(%w1 : tensor<8xf32>) outs(%0 : tensor<1x8x16x16xf32>) {
    ^bb0(%in: f32, %out: f32):
      linalg.yield %in : f32
    } -> tensor<1x8x16x16xf32>
    %2 = linalg.conv_2d_nchw_fchw {dilations = dense<1> : tensor<2xi64>, strides = dense<1> : tensor<2xi64>} ins(%padded, %w0 : tensor<1x4x18x18xf32>, tensor<8x4x3x3xf32>) outs(%1 : tensor<1x8x16x16xf32>) -> tensor<1x8x16x16xf32>
    %3 = linalg.generic {indexing_maps = [affine_map<(d0, d1, d2, d3) -> (d0, d1, d2, d3)>, affine_map<(d0, d1, d2, d3) -> (d0, d1, d2, d3)>], iterator_types = ["parallel", "parallel", "parallel", "parallel"]} ins(%2 : tensor<1x8x16x16xf32>) outs(%0 : tensor<1x8x16x16xf32>) {
    ^bb0(%in: f32, %out: f32):
      %c = arith.cmpf ugt, %in, %cst : f32
      %s = arith.select %c, %in, %cst : f32
      linalg.yield %s : f32
    } -> tensor<1x8x16x16xf32>
    %4 = tensor.empty() : tensor<1x8x8x8xf32>
    %5 = linalg.fill ins(%cst_0 : f32) outs(%4 : tensor<1x8x8x8xf32>) -> tensor<1x8x8x8xf32>
    %6 = tensor.empty() : tensor<2x2xf32>
    %7 = linalg.pooling_nchw_max {dilations = dense<1> : tensor<2xi64>, strides = dense<2> : tensor<2xi64>} ins(%3, %6 : tensor<1x8x16x16xf32>, tensor<2x2xf32>) outs(%5 : tensor<1x8x8x8xf32>) -> tensor<1x8x8x8xf32>
    return %7 : tensor<1x8x8x8xf32>
  }
}
"""
    outline = dict(inputs=["tensor<1x4x16x16xf32>"], weights=["tensor<8x4x3x3xf32>", "tensor<8xf32>"], output="tensor<1x8x8x8xf32>")
    got = M.read_ops(src, outline).as_json()
    assert [o["op"] for o in got["ops"]] == ["conv2d", "maxpool2d"]
    cv, mp = got["ops"]
    assert (cv["C"], cv["H"], cv["W"], cv["F"], cv["KH"], cv["KW"], cv["stride"], cv["pad"], cv["act"], cv["w"], cv["b"]) == (4, 16, 16, 8, 3, 3, 1, 1, "relu", "w0", "w1")
    assert (mp["C"], mp["H"], mp["W"], mp["k"]) == (8, 16, 16, 2) and cv["dst"] == mp["src"]
    text, _ = SH.emit_step({}, outline, got)
    assert "fortis_plan_conv2d(" in text and "fortis_plan_maxpool2d(" in text


def test_statements_the_reader_does_not_name_are_reported():
    src = """module {
  func.func @mlp_kernel(%arg0: tensor<8x4xf32>, %w0: tensor<4xf32>) -> tensor<8x4xf32> {
    %0 = tensor.empty() : tensor<8x4xf32>
    %1 = linalg.generic {indexing_maps = [affine_map<(d0, d1) -> (d0, d1)>, affine_map<(d0, d1) -> (d0, d1)>], iterator_types = ["parallel", "parallel"]} ins(%arg0 : tensor<8x4xf32>) outs(%0 : tensor<8x4xf32>) {
    ^bb0(%in: f32, %out: f32):
      %s = math.tanh %in : f32
      linalg.yield %s : f32
    } -> tensor<8x4xf32>
    return %1 : tensor<8x4xf32>
  }
}
"""
    with pytest.raises(M.MlirError, match="does not name"):
        M.read_ops(src, dict(inputs=["tensor<8x4xf32>"], weights=["tensor<4xf32>"], output="tensor<8x4xf32>"))
