import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; run with -m gpu on the GPU box")


@pytest.fixture(scope="session")
def golden():
    return GOLDEN


@pytest.fixture(scope="session")
def L():
    """The product library, loaded once.  GPU tests fail (not skip) if it is missing."""
    import fortis_amd
    return fortis_amd.load()


@pytest.fixture(scope="session")
def gpu(L):
    import ctypes as C
    name = C.create_string_buffer(64)
    assert L.fortis_device_info(name, 64, None) == 0, "no GPU visible to libfortis_rt"
    return name.value.decode()


@pytest.fixture(autouse=True)
def _announce(request):
    # names the case before it runs, flushed, so a run that dies on the GPU still says where
    print(f"\n[case] {request.node.nodeid}", flush=True)
    lib = request.getfixturevalue("L") if request.node.get_closest_marker("gpu") else None
    before = lib.fortis_error_count() if lib is not None else 0
    yield
    # the library prints a failed runtime call and goes on: a GPU case during which one failed is a failed case
    if lib is not None:
        assert lib.fortis_error_count() == before, "a HIP call failed during this case (see stderr)"
