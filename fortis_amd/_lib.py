"""ctypes loader and prototypes for libfortis_rt.so (include/fortis_rt.h, include/fortis_step.h)."""
import ctypes as C
import os

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libfortis_rt.so")


class FortisLibraryMissing(RuntimeError):
    pass


MAX_ARRAYS, MAX_REFS, MAX_SCAL, MAX_INS, MAX_CONST = 8, 128, 8, 32, 16


class Ref(C.Structure):
    _fields_ = [("array", C.c_int), ("planar", C.c_int), ("base", C.c_long), ("si", C.c_long), ("sj", C.c_long)]


class Ins(C.Structure):
    _fields_ = [("op", C.c_int), ("a", C.c_int), ("b", C.c_int)]


class Stencil(C.Structure):
    _fields_ = [("narrays", C.c_int), ("total", C.c_long * MAX_ARRAYS), ("plane", C.c_long * MAX_ARRAYS),
                ("nrefs", C.c_int), ("refs", Ref * MAX_REFS), ("nscal", C.c_int), ("scal", Ref * MAX_SCAL),
                ("nins", C.c_int), ("ins", Ins * MAX_INS), ("nconst", C.c_int), ("consts", C.c_float * MAX_CONST),
                ("count", C.c_long), ("nk", C.c_int), ("klo", C.c_int), ("nargs", C.c_int), ("ilo", C.c_int),
                ("jlo", C.c_int), ("ni", C.c_int), ("nj", C.c_int), ("sx", C.c_int), ("cells", C.POINTER(C.c_int)),
                ("elt", C.c_int * MAX_ARRAYS), ("cdouble", C.c_int * MAX_CONST), ("dconsts", C.c_double * MAX_CONST)]


class HostFacts(C.Structure):
    _fields_ = [("n_in", C.c_long), ("n_out", C.c_long), ("in_esz", C.c_int), ("out_esz", C.c_int),
                ("verdict", C.c_int), ("expanded", C.c_int), ("count", C.c_long), ("lo", C.c_long),
                ("step", C.c_long), ("minc", C.c_long), ("graph", C.c_int), ("gather", C.c_int), ("scatter", C.c_int)]


_L = None
vp, l, i, f = C.c_void_p, C.c_long, C.c_int, C.c_float
fp = C.POINTER(C.c_float)

# name -> (restype, argtypes); every symbol include/*.h declares
PROTOTYPES = {
    # fortis_rt.h
    "mgpuStreamCreate": (vp, []), "mgpuStreamDestroy": (None, [vp]), "mgpuStreamSynchronize": (None, [vp]),
    "fortis_alloc": (vp, [l]), "fortis_free": (None, [vp]),
    "fortis_gemm": (None, [vp, vp, l, l, l, l, l] * 3 + [l, l, l]),
    "fortis_conv2d": (None, [vp, vp] + [l] * 9 + [vp, vp] + [l] * 9 + [vp, vp] + [l] * 9 + [l] * 13),
    "fortis_conv3d": (None, ([vp, vp] + [l] * 11) * 3 + [l] * 18),
    "fortis_conv3d_noalloc": (i, ([vp, vp] + [l] * 11) * 3 + [l] * 18),
    "fortis_conv3d_direct": (None, ([vp, vp] + [l] * 11) * 3 + [l] * 18),
    "fortis_conv3d_fft": (None, ([vp, vp] + [l] * 11) * 3 + [l] * 18),
    "fortis_h2d": (None, [vp, vp, l]), "fortis_d2h": (None, [vp, vp, l]), "fortis_d2d": (None, [vp, vp, l]),
    "fortis_gemm_schedule": (i, [C.c_long, C.c_long, C.c_long, C.POINTER(C.c_long)]),
    "fortis_magic_divmod": (None, [C.c_uint, C.c_uint, C.POINTER(C.c_uint), C.POINTER(C.c_uint)]),
    "fortis_sync": (None, []), "fortis_dev_alloc_calls": (l, []), "fortis_error_count": (l, []), "fortis_note_error": (None, []), "fortis_conv_scratch_reserve": (i, [l]), "fortis_pool_stats": (None, [C.POINTER(i), C.POINTER(i)]), "fortis_pool_trim": (i, []),
    "fortis_pool_set_allocator": (None, [vp, vp]), "fortis_device_info": (i, [C.c_char_p, i, C.POINTER(l)]),
    # fortis_step.h: plan
    "fortis_plan_create": (vp, []), "fortis_plan_destroy": (None, [vp]), "fortis_plan_tensor": (i, [vp, l]),
    "fortis_plan_view": (i, [vp, i, l, l]),
    "fortis_plan_linear": (i, [vp, i, i, vp, vp, l, l, l, i, f]),
    "fortis_plan_scale": (i, [vp, i, i, vp, l, l, i]),
    "fortis_plan_mask_relu": (i, [vp, i, i, l, l, l]),
    "fortis_plan_boundary_pre": (i, [vp, i, i, l, l, vp, vp, vp, i]),
    "fortis_plan_boundary_post": (i, [vp, i, i, l, l, vp, i]),
    "fortis_plan_conv2d": (i, [vp, i, i, vp, vp, vp, vp, vp, vp, f, l, l, l, l, l, l, l, l, i, f, l, l]),
    "fortis_plan_convt2d": (i, [vp, i, i, vp, vp, l, l, l, l, l, l, l, l, l, i, f, l, l]),
    "fortis_plan_maxpool2d": (i, [vp, i, i, l, l, l, l]),
    "fortis_plan_upsample": (i, [vp, i, i, l, l, l, l, l, i]),
    "fortis_plan_concat_copy": (i, [vp, i, i, l, l, l, l]),
    "fortis_plan_conv3d": (i, [vp, i, i, i, vp, vp, l, l, l, l, l, l, l, i, f]),
    "fortis_plan_permute": (i, [vp, i, i, l, l, i]),
    "fortis_plan_finalize": (i, [vp, i, i]), "fortis_plan_run": (None, [vp]),
    "fortis_plan_tensor_ptr": (vp, [vp, i]), "fortis_plan_num_kernels": (i, [vp]),
    # step + entries
    "fortis_step_bind": (i, [vp, C.POINTER(HostFacts)]), "fortis_step_reset": (None, []),
    "fortis_step_graph_active": (i, []), "fortis_step_on_first_use": (None, [vp]),
    "mlp_upload": (None, [vp]), "mlp_forward_dev": (None, []), "mlp_download": (None, [vp]),
    "mlp_forward": (None, [vp, vp]), "mlp_forward_batched": (None, [vp, vp]),
    "fortis_pack": (None, [vp, i]), "fortis_unpack": (None, [vp, i]),
    "fortis_model_input": (vp, []), "fortis_model_output": (vp, []), "fortis_begin": (None, [i]),
    # stencil
    "fortis_stencil_check": (i, [C.POINTER(Stencil)]),
    "fortis_stencil_route": (i, [C.POINTER(Stencil)]),
    "fortis_gather_config": (i, [C.POINTER(Stencil)]), "fortis_scatter_config": (i, [C.POINTER(Stencil)]),
    "fortis_gather_v": (None, [C.POINTER(i), C.POINTER(vp)]), "fortis_scatter_v": (None, [C.POINTER(i), C.POINTER(vp)]),
    "fortis_gather": (None, [vp, vp, vp, vp]), "fortis_scatter": (None, [i, vp, vp, vp, vp, vp]),
    "fortis_stencil_gather_dev": (None, [C.POINTER(Stencil), C.POINTER(vp), vp]),
    "fortis_stencil_scatter_dev": (None, [C.POINTER(Stencil), C.POINTER(vp), vp, i]),
    "fortis_stencil_scatter_all_dev": (i, [C.POINTER(Stencil), C.POINTER(vp), vp]),
    "fortis_stencil_step_fused": (i, [C.POINTER(Stencil), C.POINTER(Stencil), vp, C.POINTER(vp), C.POINTER(vp), vp]),
    "fortis_stencil_step_fused_time_ms": (f, [C.POINTER(Stencil), C.POINTER(Stencil), vp, C.POINTER(vp), C.POINTER(vp), vp, i]),
    "fortis_plan_profile": (None, [vp, i]), "fortis_plan_profile_read": (i, [vp, fp]),
    "fortis_plan_kernel_name": (C.c_char_p, [vp, i]),
    "fortis_time_ms": (f, [vp, vp, i]), "fortis_time_parts_ms": (i, [i, vp, vp, i, fp]),
    "fortis_plan_time_ms": (f, [vp, i, i]),
}
DATA_SYMBOLS = ["fortis_capturing"]


def load(path=None):
    """dlopen the library and attach prototypes.  Raises FortisLibraryMissing if it was not built."""
    global _L
    if _L is not None:
        return _L
    path = path or LIB_PATH
    if not os.path.exists(path):
        raise FortisLibraryMissing(
            f"{path} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` or "
            "`make -C fortis_amd/csrc`.  There is no CPU fallback.")
    L = C.CDLL(path, mode=C.RTLD_GLOBAL)
    for name, (res, args) in PROTOTYPES.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args
    _L = L
    return L


def lib():
    return load()
