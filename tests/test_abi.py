"""The C-ABI library loads without a GPU and exports every symbol include/*.h declares."""
import ctypes as C
import os
import re

import pytest

from conftest import ROOT


def declared_symbols():
    names = set()
    for h in ("fortis_rt.h", "fortis_step.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"#define FORTIS_CONV3D_ARGS.*?pw\n", "", text, flags=re.S)
        for m in re.finditer(r"^\s*(?:extern\s+)?[\w\s\*]+?\b(\w+)\s*\(", text, flags=re.M):
            n = m.group(1)
            if n not in ("defined",) and not n.isupper():
                names.add(n)
        for m in re.finditer(r"extern\s+int\s+(\w+)\s*;", text):
            names.add(m.group(1))
    return names


def test_headers_declare_the_reference_abi():
    names = declared_symbols()
    # runtime tier (runtime/fortis_rt.c, runtime/fortis_fft.cu) and shim / gather entries
    # (driver/fortis_shim.py, mom6_zb/gather.cu, driver/fortis_stub.c)
    for n in ("mgpuStreamCreate", "mgpuStreamDestroy", "mgpuStreamSynchronize", "fortis_alloc", "fortis_free",
              "fortis_capturing", "fortis_gemm", "fortis_conv2d", "fortis_conv3d", "fortis_conv3d_direct",
              "fortis_conv3d_fft", "mlp_forward", "mlp_forward_batched", "mlp_upload", "mlp_forward_dev", "mlp_download",
              "fortis_pack", "fortis_unpack", "fortis_model_input", "fortis_model_output", "fortis_gather",
              "fortis_scatter", "fortis_begin"):
        assert n in names, n


def test_library_exports_every_declared_symbol(L):
    missing = []
    for n in sorted(declared_symbols()):
        try:
            getattr(L, n)
        except AttributeError:
            missing.append(n)
    assert not missing, missing


def test_python_prototypes_cover_the_headers(L):
    from fortis_amd import _lib
    have = set(_lib.PROTOTYPES) | set(_lib.DATA_SYMBOLS)
    assert declared_symbols() <= have, sorted(declared_symbols() - have)


def test_missing_library_is_loud(tmp_path):
    from fortis_amd import _lib
    saved = _lib._L
    _lib._L = None
    try:
        with pytest.raises(_lib.FortisLibraryMissing):
            _lib.load(str(tmp_path / "nope.so"))
    finally:
        _lib._L = saved


def test_capturing_flag_is_data(L):
    assert C.c_int.in_dll(L, "fortis_capturing").value == 0
