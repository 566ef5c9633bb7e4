"""Host-side mirror of the reference's entry points, on torch device tensors.

The reference's "API" is a set of ``__global__`` kernels launched from its
drivers with arguments ``(dims, A, B, C, alpha, beta)`` / ``(n, alpha, x, y)`` /
``(n, x, y, out)``.  The functions here keep those names and that argument
order, take FP32 CUDA(HIP) tensors in place of raw device pointers, and call
the C ABI of ``libhpcdnn.so`` on torch's current stream.  torch only provides
device memory and streams; all arithmetic is in the HIP library.
"""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib
from ._lib import FT_TILE_M, FT_TILE_N, Fault, HpcdnnError, check

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

_sdot_ws: dict = {}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, name: str) -> int:
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32):
        raise HpcdnnError(f"{name} must be a float32 tensor on the GPU")
    return t.data_ptr()


def _matrix(t: torch.Tensor, rows: int, cols: int, name: str):
    """Pointer and leading dimension of a row-major (possibly row-strided) 2-D view."""
    ptr = _dev(t, name)
    if t.dim() != 2 or t.shape[0] < rows or t.shape[1] < cols:
        raise HpcdnnError(f"{name} must be 2-D with at least {rows}x{cols} elements, got {tuple(t.shape)}")
    if t.shape[1] > 1 and t.stride(1) != 1:
        raise HpcdnnError(f"{name} must be row-major (unit stride along columns)")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)
    return ptr, max(int(ld), 1)


def workspace(nbytes: int, device=None) -> torch.Tensor:
    """A zero-initialised scratch buffer (zeroed by the library's own fill kernel)."""
    ws = torch.empty(max((nbytes + 3) // 4, 1), dtype=torch.int32, device=device or "cuda")
    check(_lib.lib().hpcdnn_workspace_init(ws.data_ptr(), ws.numel() * 4, _stream()), "hpcdnn_workspace_init")
    return ws


def sgemm_workspace_bytes(M: int, N: int, K: int) -> int:
    return int(_lib.lib().hpcdnn_workspace_bytes(_lib.OP_SGEMM, M, N, K))


def sgemm_plan(M: int, N: int, K: int, ws_bytes: int = 0):
    """(tile, split_k) the library picks for this shape."""
    t, sp = C.c_int(), C.c_int()
    check(_lib.lib().hpcdnn_sgemm_plan(M, N, K, ws_bytes, C.byref(t), C.byref(sp)), "hpcdnn_sgemm_plan")
    return t.value, sp.value


def sgemm_row_split(M: int, N: int, K: int, ws_bytes: int = 0):
    """(rows_first, tile_first, tile_rest) when the library covers C with two launches, rows_first = 0 otherwise."""
    r, t1, t2 = C.c_int(), C.c_int(), C.c_int()
    check(_lib.lib().hpcdnn_sgemm_row_split(M, N, K, ws_bytes, C.byref(r), C.byref(t1), C.byref(t2)), "hpcdnn_sgemm_row_split")
    return r.value, t1.value, t2.value


def tile_table():
    L = _lib.lib()
    out = []
    for t in range(L.hpcdnn_sgemm_num_tiles()):
        bm, bn, bk = C.c_int(), C.c_int(), C.c_int()
        check(L.hpcdnn_sgemm_tile_info(t, C.byref(bm), C.byref(bn), C.byref(bk)), "hpcdnn_sgemm_tile_info")
        out.append((bm.value, bn.value, bk.value))
    return out


def sgemm(M: int, N: int, K: int, A: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, alpha: float, beta: float,
          ws: torch.Tensor | None = None, tile: int = -1, split_k: int = 0) -> None:
    """In place ``C = alpha*A@B + beta*C`` (row-major; leading dimensions are the tensors' row strides).

    Counterpart of ``sgemm_k<<<...>>>(N, A, B, C, alpha, beta)`` (kernel/sgemm/sgemm.cu:120-141) and
    ``sgemm_<shape><<<...>>>(M, N, K, A, B, C, alpha, beta)`` (kernel/ft_sgemm/sgemm.cu:114-157).
    """
    pa, lda = _matrix(A, M, K, "A")
    pb, ldb = _matrix(B, K, N, "B")
    pc, ldc = _matrix(Cm, M, N, "C")
    wsp, wsb = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
    L = _lib.lib()
    if tile < 0 and split_k == 0:
        rc = L.hpcdnn_sgemm(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, wsp, wsb, _stream())
    else:
        rc = L.hpcdnn_sgemm_ex(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, wsp, wsb, tile, split_k, _stream())
    check(rc, "hpcdnn_sgemm")


def sgemm_tn(M: int, N: int, K: int, At: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, alpha: float, beta: float,
             ws: torch.Tensor | None = None, tile: int = -1, split_k: int = 0) -> None:
    """In place ``C = alpha*At.T@B + beta*C`` with ``At`` the K x M row-major transpose of the left operand."""
    pa, lda = _matrix(At, K, M, "At")
    pb, ldb = _matrix(B, K, N, "B")
    pc, ldc = _matrix(Cm, M, N, "C")
    wsp, wsb = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
    L = _lib.lib()
    if tile < 0 and split_k == 0:
        rc = L.hpcdnn_sgemm_tn(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, wsp, wsb, _stream())
    else:
        rc = L.hpcdnn_sgemm_tn_ex(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, wsp, wsb, tile, split_k, _stream())
    check(rc, "hpcdnn_sgemm_tn")


def sgemm_cm_nt(M: int, N: int, K: int, A: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, alpha: float, beta: float,
                ws: torch.Tensor | None = None) -> None:
    """Column-major ``C (M x N) = alpha*A (M x K) @ B (N x K).T + beta*C``, the layout of the reference's
    ``sgemm_<shape><<<...>>>(M, N, K, A, B, C, alpha, beta)`` (kernel/ft_sgemm/include/sgemm_huge.cuh:14) and of the cuBLAS
    call beside it (kernel/ft_sgemm/sgemm.cu:111).  The tensors hold the column-major matrices as their row-major
    transposes: ``A`` is K x M, ``B`` is K x N, ``C`` is N x M; their row strides are the leading dimensions."""
    pa, lda = _matrix(A, K, M, "A")
    pb, ldb = _matrix(B, K, N, "B")
    pc, ldc = _matrix(Cm, N, M, "C")
    wsp, wsb = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
    check(_lib.lib().hpcdnn_sgemm_cm_nt(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, wsp, wsb, _stream()), "hpcdnn_sgemm_cm_nt")


def ft_sgemm(M: int, N: int, K: int, A: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, alpha: float, beta: float,
             tau: float = 0.0, fault=None, status: torch.Tensor | None = None, ws: torch.Tensor | None = None,
             tile_class: int = 0, granularity: int = 0, check_interval: int = 0, faults=None, locator: int = 0) -> None:
    """ABFT GEMM; ``fault`` = (tile, row, col, delta) or None; ``status`` = int32 tensor of 8*ft_num_check_tiles words;
    ``ws`` = optional scratch tensor of ``ft_workspace_bytes(M, N, K)`` bytes (checksum vectors are then formed
    by a pre-pass instead of inside the main loop); ``tile_class`` selects the ABFT tile (0 = 256x128, 1 = 128x128, 3 = 128x64, 4 = 64x64,
    2 = 64x128).  ``granularity`` FT_GRAN_TILE keeps one checksum pair, verification and status record per tile of the
    class, FT_GRAN_WAVE one per wave tile (``ft_check_tile``); ``check_interval`` > 0 also verifies every that many
    values of k inside the K loop, with re-synchronised references; ``faults`` = up to four
    (tile, row, col, delta[, check]) in check-tile units, ``check`` = the verification each precedes; ``locator``
    FT_LOCATE_ROW_COL finds a fault where a faulty row meets a faulty column, FT_LOCATE_WEIGHTED from two row checksums
    with weights [1, 1, ...] and [1, 2, ...] (the reference's "kernel 2", kernel/ft_sgemm/README.md:16-26; needs ``ws``).

    Counterpart of ``ft_sgemm_huge<<<...>>>(M, N, K, A, B, C, alpha, beta)`` (kernel/ft_sgemm/sgemm.cu:159-165), of its
    warp- and thread-level variants and of its verification every 256 k (ft_sgemm_huge.cuh:143).
    """
    pa, lda = _matrix(A, M, K, "A")
    pb, ldb = _matrix(B, K, N, "B")
    pc, ldc = _matrix(Cm, M, N, "C")
    L = _lib.lib()
    sp = None
    if status is not None:
        need = 8 * L.hpcdnn_ft_num_check_tiles(tile_class, granularity, M, N)
        if not (status.is_cuda and status.dtype == torch.int32 and status.numel() >= need and status.is_contiguous()):
            raise HpcdnnError(f"status must be a contiguous int32 GPU tensor with >= {need} elements")
        sp = status.data_ptr()
    wp, wb = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
    if granularity == 0 and check_interval == 0 and not faults and locator == 0:
        f = None
        if fault is not None:
            f = C.byref(Fault(int(fault[0]), int(fault[1]), int(fault[2]), float(fault[3])))
        check(L.hpcdnn_ft_sgemm_ex(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, tau, f, sp, wp, wb, tile_class, _stream()),
              "hpcdnn_ft_sgemm")
        return
    every = list(faults or []) + ([fault] if fault is not None else [])
    if len(every) > _lib.FT_MAX_FAULTS:
        raise HpcdnnError(f"at most {_lib.FT_MAX_FAULTS} faults per call")
    opt = _lib.FtOptions()
    opt.tile_class, opt.granularity, opt.check_interval, opt.n_faults = tile_class, granularity, check_interval, len(every)
    opt.locator = locator
    for i, fl in enumerate(every):
        opt.faults[i] = _lib.FaultAt(int(fl[0]), int(fl[1]), int(fl[2]), float(fl[3]), int(fl[4]) if len(fl) > 4 else 0)
    check(L.hpcdnn_ft_sgemm_opt(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, tau, C.byref(opt), sp, wp, wb, _stream()),
          "hpcdnn_ft_sgemm_opt")


FT_GRAN_TILE, FT_GRAN_WAVE = _lib.FT_GRAN_TILE, _lib.FT_GRAN_WAVE
FT_LOCATE_ROW_COL, FT_LOCATE_WEIGHTED = _lib.FT_LOCATE_ROW_COL, _lib.FT_LOCATE_WEIGHTED
FT_STATIC_SCRATCH_BYTES = 4 << 20


def ft_cm_nt_workspace_bytes(M: int, N: int, K: int) -> int:
    return int(_lib.lib().hpcdnn_workspace_bytes(_lib.OP_FT_SGEMM_CM_NT, M, N, K))


def ft_sgemm_cm_nt(M: int, N: int, K: int, A: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, alpha: float, beta: float,
                   ws: torch.Tensor | None, tau: float = 0.0, status: torch.Tensor | None = None, tile_class: int = 0,
                   granularity: int = 0, check_interval: int = 0, faults=None, locator: int = 0) -> None:
    """ABFT GEMM on the column-major buffers of ``ft_sgemm_huge<<<...>>>(M, N, K, A, B, C, alpha, beta)``
    (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:21): ``C (M x N) = alpha*A (M x K) @ B (N x K).T + beta*C``.  The tensors hold
    the column-major matrices as their row-major transposes (``A`` K x M, ``B`` K x N, ``C`` N x M).  Tiles, status
    records and fault coordinates are those of ``ft_sgemm(N, M, K, ...)`` on the row-major ``C^T``.  ``ws``: optional
    scratch of ``ft_cm_nt_workspace_bytes(M, N, K)`` bytes, as for ``ft_sgemm``."""
    pa, lda = _matrix(A, K, M, "A")
    pb, ldb = _matrix(B, K, N, "B")
    pc, ldc = _matrix(Cm, N, M, "C")
    L = _lib.lib()
    sp = None
    if status is not None:
        need = 8 * L.hpcdnn_ft_num_check_tiles(tile_class, granularity, N, M)
        if not (status.is_cuda and status.dtype == torch.int32 and status.numel() >= need and status.is_contiguous()):
            raise HpcdnnError(f"status must be a contiguous int32 GPU tensor with >= {need} elements")
        sp = status.data_ptr()
    every = list(faults or [])
    if len(every) > _lib.FT_MAX_FAULTS:
        raise HpcdnnError(f"at most {_lib.FT_MAX_FAULTS} faults per call")
    opt = _lib.FtOptions()
    opt.tile_class, opt.granularity, opt.check_interval, opt.n_faults = tile_class, granularity, check_interval, len(every)
    opt.locator = locator
    for i, fl in enumerate(every):
        opt.faults[i] = _lib.FaultAt(int(fl[0]), int(fl[1]), int(fl[2]), float(fl[3]), int(fl[4]) if len(fl) > 4 else 0)
    wp, wb = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
    check(L.hpcdnn_ft_sgemm_cm_nt(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, tau, C.byref(opt), sp, wp, wb, _stream()),
          "hpcdnn_ft_sgemm_cm_nt")


def ft_sgemm_static(M: int, N: int, K: int, A: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, alpha: float, beta: float,
                    tau: float = 0.0, fault=None, status: torch.Tensor | None = None) -> None:
    """``ft_sgemm`` with the library's own fixed scratch array instead of a workspace: allocates nothing; refuses
    problems whose checksum vectors exceed ``FT_STATIC_SCRATCH_BYTES``; calls on one device must not overlap."""
    pa, lda = _matrix(A, M, K, "A")
    pb, ldb = _matrix(B, K, N, "B")
    pc, ldc = _matrix(Cm, M, N, "C")
    L = _lib.lib()
    sp = None
    if status is not None:
        need = 8 * L.hpcdnn_ft_num_tiles(M, N)
        if not (status.is_cuda and status.dtype == torch.int32 and status.numel() >= need and status.is_contiguous()):
            raise HpcdnnError(f"status must be a contiguous int32 GPU tensor with >= {need} elements")
        sp = status.data_ptr()
    f = None
    if fault is not None:
        f = C.byref(Fault(int(fault[0]), int(fault[1]), int(fault[2]), float(fault[3])))
    check(L.hpcdnn_ft_sgemm_static(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, tau, f, sp, _stream()),
          "hpcdnn_ft_sgemm_static")


def ft_workspace_bytes(M: int, N: int, K: int) -> int:
    return int(_lib.lib().hpcdnn_workspace_bytes(_lib.OP_FT_SGEMM, M, N, K))


def sgemv(trans: bool, M: int, N: int, alpha: float, A: torch.Tensor, x: torch.Tensor, beta: float, y: torch.Tensor,
          ws: torch.Tensor | None = None) -> None:
    """Row-major SGEMV on an ``M x N`` matrix: ``y = alpha*A*x + beta*y`` or, with ``trans``, ``alpha*A^T*x + beta*y``.

    Counterpart of the cublasSgemv calls in kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:8-23.
    """
    pa, lda = _matrix(A, M, N, "A")
    px, py = _dev(x, "x"), _dev(y, "y")
    if x.numel() < (M if trans else N) or y.numel() < (N if trans else M):
        raise HpcdnnError("x or y shorter than the matrix dimension it pairs with")
    wp, wb = (ws.data_ptr(), ws.numel() * ws.element_size()) if ws is not None else (None, 0)
    check(_lib.lib().hpcdnn_sgemv(1 if trans else 0, M, N, alpha, pa, lda, px, beta, py, wp, wb, _stream()), "hpcdnn_sgemv")


def sgemv_workspace_bytes(M: int, N: int) -> int:
    return int(_lib.lib().hpcdnn_workspace_bytes(_lib.OP_SGEMV, M, N, 0))


def offline_ft_sgemm(M: int, N: int, K: int, A: torch.Tensor, B: torch.Tensor, Cm: torch.Tensor, alpha: float,
                     beta: float, residuals: torch.Tensor, ws: torch.Tensor, fault=None, scalar: bool = False) -> None:
    """Panel-wise (offline) ABFT GEMM; ``residuals`` = float32 tensor of ``2*ceil(K/256)`` elements (column-side and
    row-side residual sums per panel), or of ``ceil(K/256)`` with ``scalar=True`` (one scalar checksum per panel:
    total of C against the reference carried through the operands); ``fault`` = (panel, row, col, delta) with global
    row/col, or None.

    Counterpart of ``baseline_ft_sgemm(...)`` (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:1-34) and, with
    ``scalar=True``, of ``offline_ft_sgemm(...)`` (:36-91).
    """
    pa, lda = _matrix(A, M, K, "A")
    pb, ldb = _matrix(B, K, N, "B")
    pc, ldc = _matrix(Cm, M, N, "C")
    panels = -(-K // _lib.OFFLINE_FT_PANEL_K)
    need = panels if scalar else 2 * panels
    pr = _dev(residuals, "residuals")
    if residuals.numel() < need or not residuals.is_contiguous():
        raise HpcdnnError(f"residuals must be a contiguous float32 GPU tensor with >= {need} elements")
    f = None
    if fault is not None:
        f = C.byref(Fault(int(fault[0]), int(fault[1]), int(fault[2]), float(fault[3])))
    fn = _lib.lib().hpcdnn_offline_ft_sgemm_scalar if scalar else _lib.lib().hpcdnn_offline_ft_sgemm
    check(fn(M, N, K, pa, lda, pb, ldb, pc, ldc, alpha, beta, f, pr, ws.data_ptr(), ws.numel() * ws.element_size(), _stream()),
          "hpcdnn_offline_ft_sgemm_scalar" if scalar else "hpcdnn_offline_ft_sgemm")


def offline_ft_workspace_bytes(M: int, N: int, K: int) -> int:
    return int(_lib.lib().hpcdnn_workspace_bytes(_lib.OP_OFFLINE_FT_SGEMM, M, N, K))


def ft_num_tiles(M: int, N: int, tile_class: int = 0) -> int:
    return int(_lib.lib().hpcdnn_ft_num_tiles_ex(tile_class, M, N))


def ft_tile(tile_class: int = 0):
    bm, bn = C.c_int(), C.c_int()
    check(_lib.lib().hpcdnn_ft_tile_info(tile_class, C.byref(bm), C.byref(bn)), "hpcdnn_ft_tile_info")
    return bm.value, bn.value


def ft_pick_class(M: int, N: int, K: int, ws_bytes: int | None = None) -> int:
    """The tile class with the shortest predicted run: for a call with the full workspace, or with one of ``ws_bytes``
    (0: none)."""
    if ws_bytes is None:
        return int(_lib.lib().hpcdnn_ft_pick_class(M, N, K))
    return int(_lib.lib().hpcdnn_ft_pick_class_ws(M, N, K, ws_bytes))


def ft_default_tau(K: int) -> float:
    return float(_lib.lib().hpcdnn_ft_default_tau(K))


def ft_check_tile(tile_class: int = 0, granularity: int = 0):
    """(rows, columns) of the unit that has its own checksum pair, verification and status record."""
    cm, cn = C.c_int(), C.c_int()
    check(_lib.lib().hpcdnn_ft_check_tile_info(tile_class, granularity, C.byref(cm), C.byref(cn)), "hpcdnn_ft_check_tile_info")
    return cm.value, cn.value


def ft_num_check_tiles(M: int, N: int, tile_class: int = 0, granularity: int = 0) -> int:
    return int(_lib.lib().hpcdnn_ft_num_check_tiles(tile_class, granularity, M, N))


def ft_status_alloc(M: int, N: int, device=None, tile_class: int = 0, granularity: int = 0) -> torch.Tensor:
    return torch.zeros(8 * ft_num_check_tiles(M, N, tile_class, granularity), dtype=torch.int32, device=device or "cuda")


def ft_status_numpy(status: torch.Tensor) -> np.ndarray:
    return status.cpu().numpy().view(FT_STATUS_DTYPE)


def saxpy(n: int, alpha: float, x: torch.Tensor, y: torch.Tensor) -> None:
    """In place ``y = alpha*x + y`` (one FMA per element).  Counterpart of kernel/saxpy/saxpy.cu:38-48."""
    px, py = _dev(x, "x"), _dev(y, "y")
    if x.numel() < n or y.numel() < n or not (x.is_contiguous() and y.is_contiguous()):
        raise HpcdnnError("x and y must be contiguous with at least n elements")
    check(_lib.lib().hpcdnn_saxpy(n, alpha, px, py, _stream()), "hpcdnn_saxpy")


def sdot(n: int, x: torch.Tensor, y: torch.Tensor, out: torch.Tensor, ws: torch.Tensor | None = None) -> None:
    """``out[0] = sum(x*y)`` on the device, deterministic.  Counterpart of kernel/sdot/sdot.cu:9-36."""
    px, py, po = _dev(x, "x"), _dev(y, "y"), _dev(out, "out")
    if x.numel() < n or y.numel() < n or not (x.is_contiguous() and y.is_contiguous()):
        raise HpcdnnError("x and y must be contiguous with at least n elements")
    if ws is None:
        key = (out.device.index, _stream())
        ws = _sdot_ws.get(key)
        if ws is None:
            ws = workspace(int(_lib.lib().hpcdnn_workspace_bytes(_lib.OP_SDOT, 0, 0, 0)), out.device)
            _sdot_ws[key] = ws
    check(_lib.lib().hpcdnn_sdot(n, px, py, po, ws.data_ptr(), ws.numel() * 4, _stream()), "hpcdnn_sdot")


def fill_uniform(dst: torch.Tensor, seed: int) -> None:
    """Seeded uniform[-1,1) fill of a contiguous vector (device-side generate_random_vector, utils/utils.cu:28-35)."""
    p = _dev(dst, "dst")
    if not dst.is_contiguous():
        raise HpcdnnError("dst must be contiguous")
    check(_lib.lib().hpcdnn_fill_uniform(p, dst.numel(), seed, _stream()), "hpcdnn_fill_uniform")


def fill_uniform_matrix(dst: torch.Tensor, rows: int, cols: int, seed: int) -> None:
    """Seeded fill of the leading rows x cols block of a row-major 2-D tensor (utils/utils.cu:37-44)."""
    p, ld = _matrix(dst, rows, cols, "dst")
    check(_lib.lib().hpcdnn_fill_uniform_matrix(p, rows, cols, ld, seed, _stream()), "hpcdnn_fill_uniform_matrix")


def cpu_gemm(alpha: float, beta: float, mat1: np.ndarray, mat2: np.ndarray, n: int, mat3: np.ndarray) -> None:
    """The reference's host validator (utils/utils.cu:93-103) on numpy float32 arrays, in place on ``mat3``."""
    for a in (mat1, mat2, mat3):
        if not (isinstance(a, np.ndarray) and a.dtype == np.float32 and a.flags.c_contiguous and a.size >= n * n):
            raise HpcdnnError("cpu_gemm takes C-contiguous float32 numpy arrays of n*n elements")
    _lib.lib().hpcdnn_cpu_gemm(alpha, beta, mat1.ctypes.data, mat2.ctypes.data, n, mat3.ctypes.data)


def verify_matrix(mat1: np.ndarray, mat2: np.ndarray, n: int) -> bool:
    """The reference's matrix acceptance check (utils/utils.cu:74-91): every element of the two n x n host arrays
    within 1e-2 absolute."""
    a = np.asarray(mat1, dtype=np.float64).reshape(-1)[: n * n]
    b = np.asarray(mat2, dtype=np.float64).reshape(-1)[: n * n]
    return bool(np.all(np.abs(a - b) <= 1e-2))


def verify_vector(vec1: np.ndarray, vec2: np.ndarray, n: int) -> bool:
    """The reference's vector acceptance check (utils/utils.cu:60-72): every element within 5e-3 relative to the
    first argument (its magnitude; the reference divides by the signed value)."""
    a = np.asarray(vec1, dtype=np.float64).reshape(-1)[:n]
    b = np.asarray(vec2, dtype=np.float64).reshape(-1)[:n]
    return bool(np.all(np.abs(a - b) <= 5e-3 * np.abs(a)))
