"""ctypes binding of ``libhpcdnn.so`` (the C ABI declared in ``include/hpcdnn.h``).

There is no CPU fallback: if the library has not been built, or a call returns
a non-zero status, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libhpcdnn.so")
CSRC = os.path.join(_PKG, "csrc")

OP_SGEMM = 0
OP_SDOT = 1
OP_FT_SGEMM = 2
OP_FT_SGEMM_CM_NT = 5
OP_SGEMV = 3
OP_OFFLINE_FT_SGEMM = 4
OFFLINE_FT_PANEL_K = 256
FT_TILE_M = 256
FT_TILE_N = 128
FT_NUM_CLASSES = 5

# every symbol include/hpcdnn.h declares
EXPORTS = (
    "hpcdnn_version",
    "hpcdnn_error_string",
    "hpcdnn_sgemm",
    "hpcdnn_sgemm_ex",
    "hpcdnn_sgemm_tn",
    "hpcdnn_sgemm_tn_ex",
    "hpcdnn_sgemm_cm_nt",
    "hpcdnn_sgemm_num_tiles",
    "hpcdnn_sgemm_tile_info",
    "hpcdnn_sgemm_plan",
    "hpcdnn_sgemm_row_split",
    "hpcdnn_ft_sgemm",
    "hpcdnn_ft_num_tiles",
    "hpcdnn_ft_sgemm_ex",
    "hpcdnn_ft_sgemm_static",
    "hpcdnn_ft_sgemm_opt",
    "hpcdnn_ft_sgemm_cm_nt",
    "hpcdnn_ft_check_tile_info",
    "hpcdnn_ft_num_check_tiles",
    "hpcdnn_ft_tile_info",
    "hpcdnn_ft_num_tiles_ex",
    "hpcdnn_ft_pick_class",
    "hpcdnn_ft_pick_class_ws",
    "hpcdnn_ft_default_tau",
    "hpcdnn_sgemv",
    "hpcdnn_offline_ft_sgemm",
    "hpcdnn_offline_ft_sgemm_scalar",
    "hpcdnn_saxpy",
    "hpcdnn_sdot",
    "hpcdnn_workspace_bytes",
    "hpcdnn_workspace_init",
    "hpcdnn_fill_uniform",
    "hpcdnn_fill_uniform_matrix",
    "hpcdnn_cpu_gemm",
)


class Fault(C.Structure):
    _fields_ = [("tile", C.c_int32), ("row", C.c_int32), ("col", C.c_int32), ("delta", C.c_float)]


FT_GRAN_TILE = 0
FT_LOCATE_ROW_COL = 0
FT_LOCATE_WEIGHTED = 1
FT_GRAN_WAVE = 1
FT_MAX_FAULTS = 4


class FaultAt(C.Structure):
    _fields_ = [("tile", C.c_int32), ("row", C.c_int32), ("col", C.c_int32), ("delta", C.c_float), ("check", C.c_int32)]


class FtOptions(C.Structure):
    _fields_ = [("tile_class", C.c_int32), ("granularity", C.c_int32), ("check_interval", C.c_int32),
                ("n_faults", C.c_int32), ("faults", FaultAt * FT_MAX_FAULTS), ("locator", C.c_int32)]


class HpcdnnError(RuntimeError):
    pass


def build(jobs: int = 8) -> str:
    """Compile the HIP sources for gfx950 (cross-compiles without a GPU) into ``lib/libhpcdnn.so``."""
    subprocess.run(["make", "-C", CSRC, f"-j{jobs}"], check=True)
    return LIB_PATH


_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HpcdnnError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            f"or `make -C {CSRC}`; there is no CPU fallback"
        )
    L = C.CDLL(LIB_PATH)
    vp, fp, i, f, sz, i64, u64 = C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_int64, C.c_uint64
    L.hpcdnn_version.restype = C.c_char_p
    L.hpcdnn_version.argtypes = []
    L.hpcdnn_error_string.restype = C.c_char_p
    L.hpcdnn_error_string.argtypes = [i]
    L.hpcdnn_sgemm.restype = i
    L.hpcdnn_sgemm.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, vp, sz, vp]
    L.hpcdnn_sgemm_ex.restype = i
    L.hpcdnn_sgemm_ex.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, vp, sz, i, i, vp]
    L.hpcdnn_sgemm_tn.restype = i
    L.hpcdnn_sgemm_tn.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, vp, sz, vp]
    L.hpcdnn_sgemm_tn_ex.restype = i
    L.hpcdnn_sgemm_tn_ex.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, vp, sz, i, i, vp]
    L.hpcdnn_sgemm_cm_nt.restype = i
    L.hpcdnn_sgemm_cm_nt.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, vp, sz, vp]
    L.hpcdnn_sgemm_num_tiles.restype = i
    L.hpcdnn_sgemm_num_tiles.argtypes = []
    L.hpcdnn_sgemm_tile_info.restype = i
    L.hpcdnn_sgemm_tile_info.argtypes = [i, C.POINTER(i), C.POINTER(i), C.POINTER(i)]
    L.hpcdnn_sgemm_plan.restype = i
    L.hpcdnn_sgemm_plan.argtypes = [i, i, i, sz, C.POINTER(i), C.POINTER(i)]
    L.hpcdnn_sgemm_row_split.restype = i
    L.hpcdnn_sgemm_row_split.argtypes = [i, i, i, sz, C.POINTER(i), C.POINTER(i), C.POINTER(i)]
    L.hpcdnn_ft_sgemm.restype = i
    L.hpcdnn_ft_sgemm.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, f, C.POINTER(Fault), vp, vp, sz, vp]
    L.hpcdnn_ft_sgemm_static.restype = i
    L.hpcdnn_ft_sgemm_static.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, f, C.POINTER(Fault), vp, vp]
    L.hpcdnn_ft_sgemm_cm_nt.restype = i
    L.hpcdnn_ft_sgemm_cm_nt.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, f, C.POINTER(FtOptions), vp, vp, sz, vp]
    L.hpcdnn_ft_sgemm_opt.restype = i
    L.hpcdnn_ft_sgemm_opt.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, f, C.POINTER(FtOptions), vp, vp, sz, vp]
    L.hpcdnn_ft_check_tile_info.restype = i
    L.hpcdnn_ft_check_tile_info.argtypes = [i, i, C.POINTER(i), C.POINTER(i)]
    L.hpcdnn_ft_num_check_tiles.restype = i
    L.hpcdnn_ft_num_check_tiles.argtypes = [i, i, i, i]
    L.hpcdnn_ft_sgemm_ex.restype = i
    L.hpcdnn_ft_sgemm_ex.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, f, C.POINTER(Fault), vp, vp, sz, i, vp]
    L.hpcdnn_ft_tile_info.restype = i
    L.hpcdnn_ft_tile_info.argtypes = [i, C.POINTER(i), C.POINTER(i)]
    L.hpcdnn_ft_num_tiles_ex.restype = i
    L.hpcdnn_ft_num_tiles_ex.argtypes = [i, i, i]
    L.hpcdnn_ft_pick_class.restype = i
    L.hpcdnn_ft_pick_class.argtypes = [i, i, i]
    L.hpcdnn_ft_pick_class_ws.restype = i
    L.hpcdnn_ft_pick_class_ws.argtypes = [i, i, i, C.c_size_t]
    L.hpcdnn_ft_num_tiles.restype = i
    L.hpcdnn_ft_num_tiles.argtypes = [i, i]
    L.hpcdnn_ft_default_tau.restype = f
    L.hpcdnn_ft_default_tau.argtypes = [i]
    L.hpcdnn_sgemv.restype = i
    L.hpcdnn_sgemv.argtypes = [i, i, i, f, fp, i, fp, f, fp, vp, sz, vp]
    L.hpcdnn_offline_ft_sgemm.restype = i
    L.hpcdnn_offline_ft_sgemm.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, C.POINTER(Fault), fp, vp, sz, vp]
    L.hpcdnn_offline_ft_sgemm_scalar.restype = i
    L.hpcdnn_offline_ft_sgemm_scalar.argtypes = [i, i, i, fp, i, fp, i, fp, i, f, f, C.POINTER(Fault), fp, vp, sz, vp]
    L.hpcdnn_saxpy.restype = i
    L.hpcdnn_saxpy.argtypes = [i64, f, fp, fp, vp]
    L.hpcdnn_sdot.restype = i
    L.hpcdnn_sdot.argtypes = [i64, fp, fp, fp, vp, sz, vp]
    L.hpcdnn_workspace_bytes.restype = sz
    L.hpcdnn_workspace_bytes.argtypes = [i, i, i, i]
    L.hpcdnn_workspace_init.restype = i
    L.hpcdnn_workspace_init.argtypes = [vp, sz, vp]
    L.hpcdnn_fill_uniform.restype = i
    L.hpcdnn_fill_uniform.argtypes = [fp, i64, u64, vp]
    L.hpcdnn_fill_uniform_matrix.restype = i
    L.hpcdnn_fill_uniform_matrix.argtypes = [fp, i, i, i, u64, vp]
    L.hpcdnn_cpu_gemm.restype = None
    L.hpcdnn_cpu_gemm.argtypes = [f, f, vp, vp, i, vp]
    _lib = L
    return L


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().hpcdnn_error_string(code).decode()
        raise HpcdnnError(f"{what} failed: {msg} (code {code})")
