"""ctypes loader for the CPU oracle (``oracle/oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; the shipped package never
imports it.  All arrays are C-contiguous numpy arrays (float32 unless noted).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force: bool = False) -> str:
    """Compile ``oracle.c`` with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


class FtStatus(C.Structure):
    _fields_ = [
        ("flag", C.c_int32),
        ("row", C.c_int32),
        ("col", C.c_int32),
        ("n_bad_rows", C.c_int32),
        ("n_bad_cols", C.c_int32),
        ("row_residual", C.c_float),
        ("col_residual", C.c_float),
        ("max_clean_residual", C.c_float),
    ]


FT_STATUS_DTYPE = np.dtype(
    [
        ("flag", "<i4"),
        ("row", "<i4"),
        ("col", "<i4"),
        ("n_bad_rows", "<i4"),
        ("n_bad_cols", "<i4"),
        ("row_residual", "<f4"),
        ("col_residual", "<f4"),
        ("max_clean_residual", "<f4"),
    ]
)

_lib = None


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    fp = C.POINTER(C.c_float)
    dp = C.POINTER(C.c_double)
    ip = C.POINTER(C.c_int)
    lib.oracle_uniform.restype = C.c_float
    lib.oracle_uniform.argtypes = [C.c_uint64, C.c_uint64]
    lib.oracle_fill_uniform.restype = None
    lib.oracle_fill_uniform.argtypes = [fp, C.c_int64, C.c_uint64]
    lib.oracle_fill_uniform_matrix.restype = None
    lib.oracle_fill_uniform_matrix.argtypes = [fp, C.c_int, C.c_int, C.c_int, C.c_uint64]
    lib.oracle_num_threads.restype = C.c_int
    lib.oracle_cpu_gemm.restype = None
    lib.oracle_cpu_gemm.argtypes = [C.c_float, C.c_float, fp, fp, C.c_int, fp]
    lib.oracle_gemm_f64_rows.restype = None
    lib.oracle_gemm_f64_rows.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int,
                                         C.c_float, C.c_float, ip, C.c_int, dp, dp]
    lib.oracle_gemm_cm_nt_f64.restype = None
    lib.oracle_gemm_cm_nt_f64.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int,
                                          C.c_float, C.c_float, dp, dp]
    lib.oracle_gemm_max_err.restype = C.c_double
    lib.oracle_gemm_max_err.argtypes = [C.c_int, fp, C.c_int, ip, C.c_int, dp, dp]
    lib.oracle_saxpy.restype = None
    lib.oracle_saxpy.argtypes = [C.c_int64, C.c_float, fp, fp]
    lib.oracle_saxpy_omp.restype = None
    lib.oracle_saxpy_omp.argtypes = [C.c_int64, C.c_float, fp, fp]
    lib.oracle_sdot_f64_serial.restype = C.c_double
    lib.oracle_sdot_f64_serial.argtypes = [C.c_int64, fp, fp]
    lib.oracle_sdot_f64.restype = C.c_double
    lib.oracle_sdot_f64.argtypes = [C.c_int64, fp, fp]
    lib.oracle_sdot_f32.restype = C.c_float
    lib.oracle_sdot_f32.argtypes = [C.c_int64, fp, fp]
    lib.oracle_recompute_element.restype = C.c_float
    lib.oracle_recompute_element.argtypes = [C.c_int, C.c_int, fp, fp, C.c_int]
    lib.oracle_sgemm_device_order.restype = None
    lib.oracle_sgemm_device_order.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int,
                                              C.c_float, C.c_float]
    lib.oracle_tile_acc.restype = None
    lib.oracle_tile_acc.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp]
    lib.oracle_abft_reference_checksums.restype = None
    lib.oracle_abft_reference_checksums.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, dp, dp]
    lib.oracle_abft_observe.restype = None
    lib.oracle_abft_observe.argtypes = [C.c_int, C.c_int, fp, C.c_int, dp, dp, dp, dp]
    lib.oracle_abft_residuals.restype = None
    lib.oracle_abft_residuals.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int, dp, dp]
    lib.oracle_abft_decide.restype = C.c_float
    lib.oracle_abft_decide.argtypes = [C.c_int, C.c_int, dp, dp, C.c_float, C.POINTER(FtStatus)]
    lib.oracle_abft_set_rows_screen.restype = None
    lib.oracle_abft_set_rows_screen.argtypes = [C.c_int]
    lib.oracle_abft_decide_lines.restype = C.c_float
    lib.oracle_abft_decide_lines.argtypes = [C.c_int, C.c_int, dp, dp, dp, dp, C.POINTER(FtStatus)]
    lib.oracle_ft_sgemm.restype = None
    lib.oracle_ft_sgemm.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int, C.c_float,
                                    C.c_float, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int, C.c_int, C.c_float,
                                    C.c_void_p]
    lib.oracle_ft_sgemm_checked.restype = None
    lib.oracle_ft_sgemm_checked.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int, C.c_float,
                                            C.c_float, C.c_int, C.c_int, C.c_float, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.oracle_ft_sgemm_weighted.restype = None
    lib.oracle_ft_sgemm_weighted.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int, C.c_float,
                                             C.c_float, C.c_int, C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_void_p]
    lib.oracle_abft_relative_thresholds.restype = None
    lib.oracle_abft_relative_thresholds.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, C.c_float, dp, dp]
    lib.oracle_sgemv_f64.restype = None
    lib.oracle_sgemv_f64.argtypes = [C.c_int, C.c_int, C.c_int, C.c_float, fp, C.c_int, fp, C.c_float, fp, dp, dp]
    lib.oracle_offline_ft_sgemm.restype = None
    lib.oracle_offline_ft_sgemm.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int, C.c_float,
                                            C.c_float, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, dp]
    lib.oracle_offline_ft_sgemm_scalar.restype = None
    lib.oracle_offline_ft_sgemm_scalar.argtypes = [C.c_int, C.c_int, C.c_int, fp, C.c_int, fp, C.c_int, fp, C.c_int, C.c_float,
                                            C.c_float, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, dp]
    _lib = lib
    return lib


def _f(a):
    assert a.dtype == np.float32
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _d(a):
    assert a.dtype == np.float64 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_double))


def num_threads() -> int:
    return int(_load().oracle_num_threads())


def uniform(seed: int, idx: int) -> float:
    return float(_load().oracle_uniform(seed, idx))


def fill_uniform(n: int, seed: int) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _load().oracle_fill_uniform(_f(out), n, seed)
    return out


def fill_uniform_matrix(rows: int, cols: int, seed: int, ld: int | None = None, pad=np.nan) -> np.ndarray:
    """rows x ld array whose first ``cols`` columns hold the seeded values; padding holds ``pad``."""
    ld = cols if ld is None else ld
    out = np.full((rows, ld), pad, dtype=np.float32)
    _load().oracle_fill_uniform_matrix(_f(out), rows, cols, ld, seed)
    return out


def cpu_gemm(alpha: float, beta: float, a: np.ndarray, b: np.ndarray, n: int, c: np.ndarray) -> None:
    """In-place C = alpha*A*B + beta*C, argument order of utils/utils.cu:93."""
    assert a.flags.c_contiguous and b.flags.c_contiguous and c.flags.c_contiguous
    _load().oracle_cpu_gemm(alpha, beta, _f(a), _f(b), n, _f(c))


def gemm_f64_rows(M, N, K, a, lda, b, ldb, c0, ldc, alpha, beta, rows=None):
    """FP64 reference and |alpha|(|A||B|)+|beta||C0| denominators for the given rows (all if None)."""
    if rows is None:
        rows_arr, nrows, rp = None, M, None
    else:
        rows_arr = np.ascontiguousarray(rows, dtype=np.int32)
        nrows = len(rows_arr)
        rp = rows_arr.ctypes.data_as(C.POINTER(C.c_int))
    ref = np.empty((nrows, N), dtype=np.float64)
    den = np.empty((nrows, N), dtype=np.float64)
    c0p = _f(c0) if c0 is not None else None
    _load().oracle_gemm_f64_rows(M, N, K, _f(a), lda, _f(b), ldb, c0p, ldc, alpha, beta, rp, nrows, _d(ref), _d(den))
    return ref, den


def gemm_cm_nt_f64(M, N, K, a, lda, b, ldb, c0, ldc, alpha, beta):
    """FP64 reference and denominators of column-major C = alpha*A*B^T + beta*C (kernel/ft_sgemm/sgemm.cu:111).
    ``a``, ``b``, ``c0`` are the flat column-major buffers (any array whose memory is that buffer); the results are
    returned as N x M row-major arrays, i.e. the column-major M x N matrix as it lies in memory with ld = M."""
    ref = np.empty((N, M), dtype=np.float64)
    den = np.empty((N, M), dtype=np.float64)
    c0p = _f(c0) if c0 is not None else None
    _load().oracle_gemm_cm_nt_f64(M, N, K, _f(a), lda, _f(b), ldb, c0p, ldc, alpha, beta, _d(ref), _d(den))
    return ref, den


def gemm_max_err(N, c, ldc, ref, den, rows=None) -> float:
    if rows is None:
        rp, nrows = None, ref.shape[0]
    else:
        rows_arr = np.ascontiguousarray(rows, dtype=np.int32)
        rp, nrows = rows_arr.ctypes.data_as(C.POINTER(C.c_int)), len(rows_arr)
    return float(_load().oracle_gemm_max_err(N, _f(c), ldc, rp, nrows, _d(ref), _d(den)))


def saxpy(alpha: float, x: np.ndarray, y: np.ndarray) -> None:
    """In-place y = fmaf(alpha, x, y)."""
    assert x.size == y.size
    _load().oracle_saxpy(x.size, alpha, _f(x), _f(y))


def saxpy_omp(alpha: float, x: np.ndarray, y: np.ndarray) -> None:
    """In-place y = fmaf(alpha, x, y) on the OpenMP pool (same bits as ``saxpy``)."""
    assert x.size == y.size
    _load().oracle_saxpy_omp(x.size, alpha, _f(x), _f(y))


def sdot_f64_serial(x: np.ndarray, y: np.ndarray) -> float:
    """Double-accumulated dot product on one thread (``sdot_f64`` is the OpenMP form)."""
    return float(_load().oracle_sdot_f64_serial(x.size, _f(x), _f(y)))


def sdot_f64(x: np.ndarray, y: np.ndarray) -> float:
    return float(_load().oracle_sdot_f64(x.size, _f(x), _f(y)))


def sdot_f32(x: np.ndarray, y: np.ndarray) -> float:
    return float(_load().oracle_sdot_f32(x.size, _f(x), _f(y)))


def recompute_element(a_row: np.ndarray, b_col: np.ndarray, ldb: int, k0: int, k1: int) -> float:
    """The accumulator of one element formed again over k0 <= k < k1: a_row points at the element's row of A, b_col at
    its column's first element of B (rows ldb apart)."""
    return float(_load().oracle_recompute_element(k0, k1, _f(a_row), _f(b_col), ldb))


def sgemm_device_order(M, N, K, a, lda, b, ldb, c, ldc, alpha, beta) -> None:
    """C = alpha*A*B + beta*C in place, in the summation order of the device's tile kernels (float accumulator,
    one fused multiply-add per k, k permuted inside each group of 16): the bits an unsplit device product has."""
    _load().oracle_sgemm_device_order(M, N, K, _f(a), lda, _f(b), ldb, _f(c), ldc, alpha, beta)


def tile_acc(a_tile, lda, b_tile, ldb, tm, tn, K) -> np.ndarray:
    """Float-accumulated (k ascending, fused) product block of one tile, tm x tn packed."""
    acc = np.empty((tm, tn), dtype=np.float32)
    _load().oracle_tile_acc(tm, tn, K, _f(a_tile), lda, _f(b_tile), ldb, _f(acc))
    return acc


def abft_reference_checksums(a_tile, lda, b_tile, ldb, tm, tn, K):
    cr = np.empty(tm, dtype=np.float64)
    cc = np.empty(tn, dtype=np.float64)
    _load().oracle_abft_reference_checksums(tm, tn, K, _f(a_tile), lda, _f(b_tile), ldb, _d(cr), _d(cc))
    return cr, cc


def abft_observe(acc, ldacc, cr_ref, cc_ref):
    tm, tn = len(cr_ref), len(cc_ref)
    dr = np.empty(tm, dtype=np.float64)
    dc = np.empty(tn, dtype=np.float64)
    _load().oracle_abft_observe(tm, tn, _f(acc), ldacc, _d(cr_ref), _d(cc_ref), _d(dr), _d(dc))
    return dr, dc


def abft_residuals(a_tile, lda, b_tile, ldb, acc, ldacc, tm, tn, K):
    dr = np.empty(tm, dtype=np.float64)
    dc = np.empty(tn, dtype=np.float64)
    _load().oracle_abft_residuals(tm, tn, K, _f(a_tile), lda, _f(b_tile), ldb, _f(acc), ldacc, _d(dr), _d(dc))
    return dr, dc


def abft_decide(dr: np.ndarray, dc: np.ndarray, tau: float):
    """Returns (status dict, correction to add to acc[row, col])."""
    st = FtStatus()
    dr = np.ascontiguousarray(dr, dtype=np.float64)
    dc = np.ascontiguousarray(dc, dtype=np.float64)
    fix = _load().oracle_abft_decide(len(dr), len(dc), _d(dr), _d(dc), tau, C.byref(st))
    return {k: getattr(st, k) for k, _ in FtStatus._fields_}, float(fix)


def abft_decide_lines(dr: np.ndarray, dc: np.ndarray, tau_r: np.ndarray, tau_c: np.ndarray):
    """Like abft_decide with one threshold per row (tau_r) and per column (tau_c)."""
    st = FtStatus()
    dr, dc, tau_r, tau_c = (np.ascontiguousarray(v, dtype=np.float64) for v in (dr, dc, tau_r, tau_c))
    assert len(tau_r) == len(dr) and len(tau_c) == len(dc)
    fix = _load().oracle_abft_decide_lines(len(dr), len(dc), _d(dr), _d(dc), _d(tau_r), _d(tau_c), C.byref(st))
    return {k: getattr(st, k) for k, _ in FtStatus._fields_}, float(fix)


class rows_screen:
    """Context manager: inside it the ABFT decision model takes the rows as the screen (columns looked at only when a
    row is flagged), the library's rule for row x column location on products one tile wide with a workspace."""

    def __enter__(self):
        _load().oracle_abft_set_rows_screen(1)
        return self

    def __exit__(self, *exc):
        _load().oracle_abft_set_rows_screen(0)
        return False


def ft_sgemm(M, N, K, a, lda, b, ldb, c, ldc, alpha, beta, tile_m, tile_n, tau, fault=None):
    """In-place ABFT GEMM model; ``fault`` = (tile, i, j, delta) or None.  Returns the per-tile status array."""
    ntiles = ((M + tile_m - 1) // tile_m) * ((N + tile_n - 1) // tile_n)
    status = np.zeros(ntiles, dtype=FT_STATUS_DTYPE)
    ft, fi, fj, fd = (-1, 0, 0, 0.0) if fault is None else fault
    _load().oracle_ft_sgemm(M, N, K, _f(a), lda, _f(b), ldb, _f(c), ldc, alpha, beta, tile_m, tile_n, tau,
                            int(ft), int(fi), int(fj), float(fd), status.ctypes.data_as(C.c_void_p))
    return status


FAULT_AT_DTYPE = np.dtype([("tile", "<i4"), ("row", "<i4"), ("col", "<i4"), ("delta", "<f4"), ("check", "<i4")])


def ft_sgemm_checked(M, N, K, a, lda, b, ldb, c, ldc, alpha, beta, tile_m, tile_n, tau, check_interval=0, faults=()):
    """In-place ABFT GEMM model with a verification every ``check_interval`` values of k (0: once, at the end) and
    re-synchronised references; ``faults`` = iterable of (tile, i, j, delta, check).  Returns the per-tile status array."""
    ntiles = ((M + tile_m - 1) // tile_m) * ((N + tile_n - 1) // tile_n)
    status = np.zeros(ntiles, dtype=FT_STATUS_DTYPE)
    fa = np.zeros(max(len(faults), 1), dtype=FAULT_AT_DTYPE)
    for i, f in enumerate(faults):
        fa[i] = (int(f[0]), int(f[1]), int(f[2]), float(f[3]), int(f[4]) if len(f) > 4 else 0)
    _load().oracle_ft_sgemm_checked(M, N, K, _f(a), lda, _f(b), ldb, _f(c), ldc, alpha, beta, tile_m, tile_n, tau,
                                    int(check_interval), len(faults), fa.ctypes.data_as(C.c_void_p),
                                    status.ctypes.data_as(C.c_void_p))
    return status


def ft_sgemm_weighted(M, N, K, a, lda, b, ldb, c, ldc, alpha, beta, tile_m, tile_n, tau, faults=()):
    """In-place ABFT GEMM model with the weighted-checksum locator (two row sums of B, weights [1, 1, ...] and
    [1, 2, ...] over each tile's columns); ``faults`` = iterable of (tile, i, j, delta).  Returns the per-tile status."""
    ntiles = ((M + tile_m - 1) // tile_m) * ((N + tile_n - 1) // tile_n)
    status = np.zeros(ntiles, dtype=FT_STATUS_DTYPE)
    fa = np.zeros(max(len(faults), 1), dtype=FAULT_AT_DTYPE)
    for i, f in enumerate(faults):
        fa[i] = (int(f[0]), int(f[1]), int(f[2]), float(f[3]), 0)
    _load().oracle_ft_sgemm_weighted(M, N, K, _f(a), lda, _f(b), ldb, _f(c), ldc, alpha, beta, tile_m, tile_n, tau,
                                     len(faults), fa.ctypes.data_as(C.c_void_p), status.ctypes.data_as(C.c_void_p))
    return status


def sgemv_f64(trans: bool, M: int, N: int, alpha: float, a: np.ndarray, lda: int, x: np.ndarray, beta: float,
              y: np.ndarray | None):
    """FP64 row-major SGEMV and its absolute-value scale: (out, den), both float64 of length N if trans else M."""
    ylen = N if trans else M
    out, den = np.empty(ylen, np.float64), np.empty(ylen, np.float64)
    yp = _f(y) if (y is not None and beta != 0.0) else None
    _load().oracle_sgemv_f64(int(bool(trans)), M, N, alpha, _f(a), lda, _f(x), beta, yp, _d(out), _d(den))
    return out, den


def offline_ft_sgemm(M, N, K, a, lda, b, ldb, c, ldc, alpha, beta, panel, fault=None) -> np.ndarray:
    """FP64 model of the panel-wise ABFT GEMM; updates ``c`` in place and returns the 2*ceil(K/panel) residual sums."""
    panels = -(-K // panel)
    res = np.zeros(2 * max(panels, 1), np.float64)
    fp_, fr, fc, fd = (-1, 0, 0, 0.0) if fault is None else fault
    _load().oracle_offline_ft_sgemm(M, N, K, _f(a), lda, _f(b), ldb, _f(c), ldc, alpha, beta, panel, int(fp_), int(fr),
                                    int(fc), float(fd), _d(res))
    return res[:2 * panels]


def offline_ft_sgemm_scalar(M, N, K, a, lda, b, ldb, c, ldc, alpha, beta, panel, fault=None) -> np.ndarray:
    """FP64 model of the panel-wise ABFT GEMM with one scalar checksum per panel; updates ``c`` in place and returns
    the ceil(K/panel) residuals."""
    panels = -(-K // panel)
    res = np.zeros(max(panels, 1), np.float64)
    fp_, fr, fc, fd = (-1, 0, 0, 0.0) if fault is None else fault
    _load().oracle_offline_ft_sgemm_scalar(M, N, K, _f(a), lda, _f(b), ldb, _f(c), ldc, alpha, beta, panel, int(fp_), int(fr),
                                           int(fc), float(fd), _d(res))
    return res[:panels]


def abft_relative_thresholds(acc: np.ndarray, K: int, factor: float = 1.0):
    """Per-row and per-column thresholds of the data-scaled mode for one tile of accumulators."""
    tm, tn = acc.shape
    acc = np.ascontiguousarray(acc, dtype=np.float32)
    tr, tc = np.empty(tm, np.float64), np.empty(tn, np.float64)
    _load().oracle_abft_relative_thresholds(tm, tn, K, _f(acc), tn, factor, _d(tr), _d(tc))
    return tr, tc
