"""Writes tests/golden/zb_native_golden.npz from the reference's own CPU path.

Runs oracle/_ref/zb_native4 (mom6_zb/zb_host.f90 + fwd_native_zb.f90 compiled by oracle/build_ref.sh)
in a scratch directory next to a zb_nn.bin derived from the checked-in zb_nn.npz the way
mom6_zb/make_zb_weights.py:12-17 lays it out (A0 as Fortran (20,27), b0, A1 as (3,20), b1,
input_norms, output_norms, all float32), and keeps:
  - the three fp64 checksums the host prints (sum of Txx, Tyy, Txy over the whole (68,78,15) arrays),
  - layers k = 1, 8, 15 of Txx, Tyy, Txy as float32 (the host wrote float32 values widened to fp64).
Only this container has the reference tree; the fixture is what travels.
"""
import os
import subprocess
import sys
import tempfile

import numpy as np

here = os.path.dirname(os.path.abspath(__file__))
root = os.path.dirname(os.path.dirname(here))
exe = os.path.join(root, "oracle", "_ref", "zb_native4")
if not os.path.exists(exe):
    sys.exit("build oracle/_ref first: make -C oracle ref")
W = np.load(os.path.join(here, "zb_nn.npz"))
with tempfile.TemporaryDirectory() as td:
    with open(os.path.join(td, "zb_nn.bin"), "wb") as o:
        for a in (W["A0"].T, W["b0"], W["A1"].T, W["b1"], W["in_norms"], W["out_norms"]):
            o.write(np.ascontiguousarray(a, dtype=np.float32).tobytes())
    out = subprocess.run([exe], cwd=td, check=True, capture_output=True, text=True).stdout
    raw = np.fromfile(os.path.join(td, "zb_out.bin"), dtype=np.float64)
sx, sy, nz = 68, 78, 15
T = raw.reshape(3, nz, sy, sx)           # Fortran (sx,sy,nz) order: k slowest
assert np.array_equal(T.astype(np.float32).astype(np.float64), T)
layers = np.array([1, 8, 15])
np.savez_compressed(os.path.join(here, "zb_native_golden.npz"),
                    checksum=np.array([T[0].sum(), T[1].sum(), T[2].sum()]),
                    layers=layers,
                    Txx=T[0][layers - 1].astype(np.float32),
                    Tyy=T[1][layers - 1].astype(np.float32),
                    Txy=T[2][layers - 1].astype(np.float32))
print(out)
print("checksums", T[0].sum(), T[1].sum(), T[2].sum())
