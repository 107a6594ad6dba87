"""fortis_amd: MI355X (gfx950) backend for the FORTIS fused inference step.

The product is the C-ABI shared library libfortis_rt.so (sources in fortis_amd/csrc, declarations
in include/).  This package is the thin host-side layer over it, mirroring the roles of the
reference's Python generators: plan.py builds the model plan an exporter would emit, stencil.py
turns the reference's gather.json / scatter.json / loop.json / kdist.json descriptors into the
library's tables, step.py binds the `fortis.host` facts and exposes the shim entry points.
There is no CPU fallback: without the built library (or without a GPU) calls fail loudly.
"""
from ._lib import lib, load, LIB_PATH, FortisLibraryMissing  # noqa: F401
