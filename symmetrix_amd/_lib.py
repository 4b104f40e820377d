"""ctypes loader for libsymmetrix_amd.so (the C ABI in include/symmetrix_amd.h).

There is no fallback: if the shared library is missing, importing the engine
classes raises.  `build()` compiles it in-tree with hipcc for gfx950.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsymmetrix_amd.so")
_lib = None

SMX_FP64 = 0
SMX_FP32_FEATURES = 1

ERROR_NAMES = {-1: "SMX_EINVAL", -2: "SMX_EFILE", -3: "SMX_EUNSUPPORTED", -4: "SMX_ENODEVICE",
               -5: "SMX_EHIP", -6: "SMX_ERANGE", -7: "SMX_ENOMEM"}

EXPORTS = [
    "smx_last_error", "smx_model_load", "smx_model_free", "smx_model_get_int", "smx_model_get_double",
    "smx_model_get_atomic_numbers", "smx_model_get_atomic_energies", "smx_compute_node_energies_forces",
    "smx_compute_device", "smx_compute_ghosted", "smx_compute_ghosted_device", "smx_set_num_H1_rows", "smx_compute_Y", "smx_compute_R0", "smx_compute_R1",
    "smx_compute_A0", "smx_reverse_A0", "smx_compute_A0_scaled", "smx_reverse_A0_scaled", "smx_compute_A1_scaled",
    "smx_reverse_A1_scaled", "smx_compute_M0", "smx_reverse_M0", "smx_compute_H1", "smx_reverse_H1",
    "smx_compute_Phi1", "smx_reverse_Phi1", "smx_compute_A1", "smx_reverse_A1", "smx_compute_M1",
    "smx_reverse_M1", "smx_compute_H2", "smx_reverse_H2", "smx_compute_readouts", "smx_get_array",
    "smx_set_array", "smx_set_profiling", "smx_stage_names", "smx_get_stage_times", "smx_synchronize",
    "smx_reduce_forces", "smx_set_staging_limit", "smx_nlist_create", "smx_nlist_free", "smx_nlist_build", "smx_nlist_update", "smx_nlist_build_host", "smx_nlist_update_host", "smx_nlist_inputs", "smx_reduce_forces_device", "smx_nlist_arrays",
    "smx_nlist_copy_to_host", "smx_compute_ZBL", "smx_fill_array", "smx_reduce_forces_device_noalloc",
]


def build(jobs=8):
    """Compile the HIP extension in-tree (hipcc cross-compiles without a GPU)."""
    subprocess.check_call(["make", "-C", os.path.join(_HERE, "csrc"), f"-j{jobs}"])
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C symmetrix_amd/csrc`.  The engine has no CPU fallback.")
        L = C.CDLL(LIB_PATH)
        L.smx_last_error.restype = C.c_char_p
        L.smx_stage_names.restype = C.c_char_p
        L.smx_model_free.restype = None
        L.smx_nlist_create.restype = C.c_void_p
        L.smx_nlist_free.restype = None
        L.smx_nlist_free.argtypes = [C.c_void_p]
        _lib = L
    return _lib


class SymmetrixError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"{ERROR_NAMES.get(code, code)}: {message}")
        self.code = code


def check(code):
    """Map C-ABI error codes to the exceptions the reference raises through
    pybind: std::invalid_argument -> ValueError (spline range,
    libsymmetrix/source/cubic_spline.cpp:19-20), everything else ->
    RuntimeError (what symmetrix_calc.py:54-56 catches for bad files)."""
    if code == 0:
        return
    msg = lib().smx_last_error().decode()
    if code in (-1, -6):
        raise ValueError(f"{ERROR_NAMES.get(code)}: {msg}")
    raise SymmetrixError(code, msg)
