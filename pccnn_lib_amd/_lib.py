"""ctypes binding of ``libpccnn_hip.so`` (the C ABI declared in include/pccnn_hip.h).

The library is the only compute path of this package: if it is missing, or an entry point
returns an error, a RuntimeError is raised -- there is no CPU or PyTorch fallback.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpccnn_hip.so")

P = ctypes.c_void_p
I64 = ctypes.c_int64
I32 = ctypes.c_int
F32 = ctypes.c_float
SZ = ctypes.c_size_t



class Basis(ctypes.Structure):
    """struct pccnn_basis of include/pccnn_hip.h."""
    _fields_ = [("kind", ctypes.c_int), ("k", ctypes.c_int), ("a", P), ("b", P), ("c", P),
                ("nb0", ctypes.c_int), ("nb1", ctypes.c_int), ("nb2", ctypes.c_int), ("sigma", ctypes.c_float),
                ("pdf", P)]


BP = ctypes.POINTER(Basis)

# name -> (restype, argtypes); mirrors include/pccnn_hip.h declaration by declaration.
SIGNATURES = {
    "pccnn_last_error": (ctypes.c_char_p, []),
    "pccnn_version": (I32, []),
    "pccnn_bounding_box": (I32, [P, P, I64, I32, I32, P, P, P]),
    "pccnn_num_cells": (I32, [P, P, P, I32, I32, P, P]),
    "pccnn_compute_keys": (I32, [P, P, P, P, P, I64, I32, P, P]),
    "pccnn_sort_keys_workspace_bytes": (SZ, [I64]),
    "pccnn_sort_keys": (I32, [P, I64, I32, P, P, P, I32, P, P, SZ, P]),
    "pccnn_sort_keys_static": (I32, [P, I64, I32, P, P, P, I32, P, P]),
    "pccnn_build_grid_ds": (I32, [P, I64, P, I32, I64, P, P]),
    "pccnn_find_neighbors_workspace_bytes": (SZ, [I64, I64]),
    "pccnn_build_cell_table": (I32, [P, I64, I64, P, P]),
    "pccnn_find_neighbors_count": (I32, [P, P, I64, P, P, I64, P, I32, P, I64, P, I64, P, P, I32, I32, P, P, SZ, P]),
    "pccnn_find_neighbors_fill": (I32, [P, P, I64, P, P, I64, P, I32, P, I64, P, I64, P, P, I32, I32, P, P, I64, P, P,
                                        SZ, P]),
    "pccnn_grid_build_workspace_bytes": (SZ, [I64]),
    "pccnn_grid_build": (I32, [P, P, P, P, P, I64, I32, I32, I64, I64, P, P, P, P, P, P, P, SZ, P]),
    "pccnn_compute_pdf": (I32, [I32, P, P, I64, I32, P, I64, P, P, P]),
    "pccnn_compute_pdf_sorted": (I32, [I32, P, P, P, I64, I32, P, I64, P, P, P]),
    "pccnn_compute_pdf_grads": (I32, [I32, P, P, I64, I32, P, I64, P, P, P, P]),
    "pccnn_compute_pdf_grid": (I32, [I32, P, P, P, I64, P, P, I64, P, I64, P, P, I32, I32, P, P, P]),
    "pccnn_poisson_disk_workspace_bytes": (SZ, [I64]),
    "pccnn_poisson_disk_select": (I32, [P, I64, P, I64, P, P, I32, P, P, P, SZ, P]),
    "pccnn_compact_selected": (I32, [P, P, I64, P, P]),
    "pccnn_poisson_disk_grid": (I32, [P, P, I64, P, I64, P, I64, P, P, I32, P, P, P, SZ, P]),
    "pccnn_bounding_box_host": (I32, [P, P, I64, I32, I32, P, P, P, P, P]),
    "pccnn_pool_poisson_workspace_bytes": (SZ, [I64, I64, I64]),
    "pccnn_pool_poisson_select": (I32, [P, P, I64, I32, P, P, P, I32, I32, P, P, P, P, P, P, P, P, P, SZ, P]),
    "pccnn_bounding_box_queued": (I32, [P, P, I64, I32, I32, P, P, P, P, P]),
    "pccnn_pool_poisson_select_queued": (I32, [P, P, I64, I32, P, P, P, I32, I32, P, P, P, P, P, P, P, P, SZ, P]),
    "pccnn_compact_selected_remap": (I32, [P, P, P, I64, P, P]),
    "pccnn_compact_pooled": (I32, [P, P, P, P, P, I64, I32, P, P, P, P]),
    "pccnn_grid_build_sized": (I32, [P, P, P, P, P, I64, I32, I32, I32, I32, P, P, P, P, P, P, P, P, SZ, P]),
    "pccnn_pdf_cloud_workspace_bytes": (SZ, [I64, I64, I64]),
    "pccnn_pdf_cloud": (I32, [I32, P, P, P, I64, I32, P, P, P, I32, I32, I32, P, P, P, SZ, P]),
    "pccnn_neighborhood_count": (I32, [P, P, I64, I32, P, P, P, I32, I32, P, P, P, P, P, P, P, P, P, I64, P, P, P, P,
                                       I32, P, P, P, SZ, P, SZ, P]),
    "pccnn_conv_workspace_bytes": (SZ, [I64, I64, I32, I32, I32, I32]),
    "pccnn_conv_workspace_bytes_deterministic": (SZ, [I64, I64, I64, I32, I32, I32]),
    "pccnn_kpconv_forward": (I32, [P, P, P, P, P, P, P, F32, P, I64, I64, I64, I32, I32, I32, I32, P, P, P, SZ, P]),
    "pccnn_set_fused_forward": (I32, [I32]),
    "pccnn_mirror_pairs": (I32, [P, P, I64, I64, P, P, P]),
    "pccnn_kpconv_backward": (I32, [P, P, P, P, P, P, P, F32, P, P, P, P, I32, I64, I64, I64, I32, I32, I32, I32,
                                    P, P, P, P, P, P, SZ, P]),
    "pccnn_mcconv_forward": (I32, [P, P, P, P, P, P, P, P, P, P, I64, I64, I64, I32, I32, I32, I32, I32,
                                   P, P, P, SZ, P]),
    "pccnn_mcconv_backward": (I32, [P, P, P, P, P, P, P, P, P, P, P, P, P, I32, I64, I64, I64, I32, I32, I32, I32, I32,
                                    P, P, P, P, P, P, P, P, SZ, P]),
    "pccnn_conv_weight_var_workspace_bytes": (SZ, [I64, I64, I32, I32]),
    "pccnn_kpconv_weight_var": (I32, [P, P, P, P, P, P, P, F32, I64, I64, I64, I32, I32, I32, P, P, SZ, P]),
    "pccnn_mcconv_weight_var": (I32, [P, P, P, P, P, P, P, P, P, I64, I64, I64, I32, I32, I32, P, P, SZ, P]),
    "pccnn_conv_forward": (I32, [BP, P, P, P, P, P, P, P, I64, I64, I64, I32, I32, I32, I32, I32, P, P, P, SZ, P]),
    "pccnn_conv_backward": (I32, [BP, P, P, P, P, P, P, P, P, P, P, I32, I64, I64, I64, I32, I32, I32, I32, I32,
                                  P, P, P, P, P, P, P, P, SZ, P]),
    "pccnn_conv_forward_bf16": (I32, [BP, P, P, P, P, P, P, P, I64, I64, I64, I32, I32, I32, I32, I32, P, P, P, SZ,
                                      P]),
    "pccnn_conv_backward_bf16": (I32, [BP, P, P, P, P, P, P, P, P, P, P, I32, I64, I64, I64, I32, I32, I32, I32, I32,
                                       P, P, P, P, P, P, P, P, SZ, P]),
    "pccnn_f32_to_bf16": (I32, [P, P, I64, P]),
    "pccnn_gemm_bf16": (I32, [P, P, P, I64, I64, I64, I32, I32, I64, I64, I64, I32, I64, I64, I64, I32, P, SZ, P]),
    "pccnn_conv_weight_var": (I32, [BP, P, P, P, P, P, P, I64, I64, I64, I32, I32, I32, P, P, SZ, P]),
    "pccnn_linear_basis_forward": (I32, [P, P, P, P, P, P, I64, I64, I64, I32, I32, P, P]),
    "pccnn_linear_basis_workspace_bytes": (SZ, [I64]),
    "pccnn_linear_basis_backward": (I32, [P, P, P, P, P, P, P, I64, I64, I64, I32, I32, P, P, P, P, P, SZ, P]),
    "pccnn_timing_enable": (I32, [I32]),
    "pccnn_timing_reset": (I32, []),
    "pccnn_timing_count": (I32, []),
    "pccnn_timing_name": (ctypes.c_char_p, [I32]),
    "pccnn_timing_read": (I32, [I32, P, P]),
    "pccnn_calibration_copy": (I32, [P, P, I64, P]),
    "pccnn_gather_rows_f32": (I32, [P, P, P, I64, I32, I64, P]),
    "pccnn_invert_permutation_i32": (I32, [P, P, I64, P]),
    "pccnn_gemm_f32": (I32, [P, P, P, I64, I64, I64, I32, I32, I64, I64, I64, I32, I64, I64, I64, I32, P, SZ, P]),
}

_lib = None


def load():
    """Load the shared library once and attach the C signatures."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "pccnn_lib_amd: %s is missing; build it with `python -m pccnn_lib_amd.build` "
            "(needs hipcc; there is no fallback implementation)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name, None)
        if fn is None:
            raise RuntimeError("pccnn_lib_amd: %s does not export %s: it was built from older sources; rebuild it "
                               "with `python -m pccnn_lib_amd.build`" % (LIB_PATH, name))
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().pccnn_last_error()
        raise RuntimeError("%s failed (%d): %s" % (what, rc, msg.decode() if msg else "?"))


def call(name, *args):
    """Call an int-returning entry point and raise on a non-zero status."""
    check(getattr(load(), name)(*args), name)


def timing(enable=None, reset=False):
    """Switch the per-kernel timers on/off, optionally reset them, and return
    {name: (launches, total_ms)} for the timers that fired."""
    lib = load()
    if reset:
        lib.pccnn_timing_reset()
    if enable is not None:
        lib.pccnn_timing_enable(1 if enable else 0)
    out = {}
    for i in range(lib.pccnn_timing_count()):
        n, ms = ctypes.c_int64(0), ctypes.c_double(0.0)
        check(lib.pccnn_timing_read(i, ctypes.byref(n), ctypes.byref(ms)), "pccnn_timing_read")
        if n.value:
            out[lib.pccnn_timing_name(i).decode()] = (n.value, ms.value)
    return out
