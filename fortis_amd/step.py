"""Step binding and entry points: what the generated shim.c is in the reference
(driver/fortis_shim.py:54-135), as calls into the library."""
import ctypes as C

import numpy as np

from ._lib import HostFacts, lib

VERDICT = {"whole": 0, "batched": 1, "boundary": 2}


def bind(plan, n_in, n_out, verdict="whole", in_dtype=np.float32, out_dtype=np.float32, expanded=False, count=0,
         lo=1, step=1, minc=1, graph=False, gather=False, scatter=False):
    """Binds `plan` as the process's step with the facts of the fortis.host attribute
    (driver/fortis_hostattr.py:11-28)."""
    h = HostFacts(n_in, n_out, np.dtype(in_dtype).itemsize, np.dtype(out_dtype).itemsize, VERDICT[verdict],
                  1 if expanded else 0, count, lo, step, minc, 1 if graph else 0, 1 if gather else 0, 1 if scatter else 0)
    if lib().fortis_step_bind(plan.handle, C.byref(h)) != 0:
        raise ValueError("fortis_step_bind rejected the host facts (see stderr)")
    return h


def reset():
    lib().fortis_step_reset()


def _vp(a):
    return a.ctypes.data_as(C.c_void_p)


def mlp_forward(x, y):
    lib().mlp_forward(_vp(x), _vp(y))


def mlp_upload(x):
    lib().mlp_upload(_vp(x))


def mlp_forward_dev():
    lib().mlp_forward_dev()


def mlp_download(y):
    lib().mlp_download(_vp(y))


def mlp_forward_batched(x=None, y=None):
    lib().mlp_forward_batched(None if x is None else _vp(x), None if y is None else _vp(y))


def fortis_pack(row, col):
    lib().fortis_pack(_vp(row), col)


def fortis_unpack(row, col):
    lib().fortis_unpack(_vp(row), col)


def fortis_begin(count):
    lib().fortis_begin(count)


def graph_active():
    return bool(lib().fortis_step_graph_active())


def gather_config(table):
    if lib().fortis_gather_config(C.byref(table)) != 0:
        raise ValueError("fortis_gather_config rejected the table (see stderr)")


def scatter_config(table):
    if lib().fortis_scatter_config(C.byref(table)) != 0:
        raise ValueError("fortis_scatter_config rejected the table (see stderr)")


def fortis_gather_v(args, arrays):
    a = (C.c_int * max(1, len(args)))(*args) if args else None
    H = (C.c_void_p * len(arrays))(*[x.ctypes.data for x in arrays])
    lib().fortis_gather_v(a, H)


def fortis_scatter_v(args, arrays):
    a = (C.c_int * max(1, len(args)))(*args) if args else None
    H = (C.c_void_p * len(arrays))(*[x.ctypes.data for x in arrays])
    lib().fortis_scatter_v(a, H)
