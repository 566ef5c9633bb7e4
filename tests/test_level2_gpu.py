"""GPU parity of SGEMV and of the offline (panel-wise) ABFT baseline against the CPU oracle, through the C ABI.

SGEMV criterion (stated tolerance): |y - yref| <= 1e-5 * (|alpha| sum |a||x| + |beta||y0|) per element, yref in FP64.
Offline ABFT: C as for SGEMM (1e-5 componentwise, fault excluded); residual sums against the FP64 model within a
noise allowance that is stated per test (the sums add M*N FP32-rounded entries, so they carry rounding noise).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-5


def _gemv_case(blas, oracle_mod, trans, M, N, alpha, beta, lda=None, use_ws=True, seed=700):
    lda = lda or max(N, 1)
    a = oracle_mod.fill_uniform_matrix(M, N, seed, ld=lda)
    xlen, ylen = (M, N) if trans else (N, M)
    x = oracle_mod.fill_uniform(xlen, seed + 1)
    y0 = oracle_mod.fill_uniform(ylen, seed + 2)
    if beta == 0.0:
        y0[:] = np.nan  # never read
    da, dx, dy = torch.from_numpy(a).cuda(), torch.from_numpy(x).cuda(), torch.from_numpy(y0).cuda()
    ws = None
    if use_ws:
        ws = torch.full((max(blas.sgemv_workspace_bytes(M, N) // 4, 4),), float("nan"), device="cuda")
    blas.sgemv(trans, M, N, alpha, da, dx, beta, dy, ws=ws)
    y = dy.cpu().numpy().astype(np.float64)
    ref, den = oracle_mod.sgemv_f64(trans, M, N, alpha, a, lda, x, beta, None if beta == 0.0 else y0)
    assert np.all(np.abs(y - ref) <= TOL * den + 1e-30), (trans, M, N, alpha, beta, np.max(np.abs(y - ref) / (den + 1e-30)))
    return dy


@pytest.mark.parametrize("trans", [False, True])
@pytest.mark.parametrize("M,N", [(1, 1), (3, 5), (64, 256), (257, 1023), (1000, 37), (37, 1000), (2048, 2048), (4096, 256), (256, 4096), (8195, 4100)])
def test_sgemv_shapes(blas, oracle_mod, trans, M, N):
    _gemv_case(blas, oracle_mod, trans, M, N, 1.0, 0.0)


@pytest.mark.parametrize("trans", [False, True])
@pytest.mark.parametrize("alpha,beta", [(1.5, -0.5), (0.0, 2.0), (-1.0, 1.0)])
def test_sgemv_alpha_beta_padded_ld_and_no_workspace(blas, oracle_mod, trans, alpha, beta):
    _gemv_case(blas, oracle_mod, trans, 777, 513, alpha, beta, lda=520)
    _gemv_case(blas, oracle_mod, trans, 777, 513, alpha, beta, lda=517, use_ws=False)


@pytest.mark.parametrize("trans", [False, True])
@pytest.mark.parametrize("M,N,lda", [(5, 3000, 3001), (130, 16384, 16384), (70, 16385, 16390), (300, 2048, 2052), (3, 4099, 4099),
                                     (513, 6000, 6004)])
def test_sgemv_wide_rows(blas, oracle_mod, trans, M, N, lda):
    """Rows of 2048 ... 16384 elements take the kernels that keep x in LDS (plain product) or give every wave a strip
    of 2048 columns (transposed product); sizes on either side of their limits, ragged last strips, padded rows."""
    _gemv_case(blas, oracle_mod, trans, M, N, 0.75, -1.25, lda=lda)
    _gemv_case(blas, oracle_mod, trans, M, N, 1.0, 0.0, lda=lda, use_ws=False)


def test_sgemv_exact_sums_and_reproducible(blas):
    # small integers: every partial sum is exact in FP32, so any summation order gives the same bits
    M, N = 1500, 700
    a = torch.randint(-3, 4, (M, N), device="cuda").float()
    ones_n, ones_m = torch.ones(N, device="cuda"), torch.ones(M, device="cuda")
    r, c = torch.empty(M, device="cuda"), torch.empty(N, device="cuda")
    ws = blas.workspace(max(blas.sgemv_workspace_bytes(M, N), 4))
    blas.sgemv(False, M, N, 1.0, a, ones_n, 0.0, r)
    blas.sgemv(True, M, N, 1.0, a, ones_m, 0.0, c, ws=ws)
    assert torch.equal(r, a.sum(dim=1)) and torch.equal(c, a.sum(dim=0))
    # random data: two runs give identical bits (fixed summation order)
    b = torch.rand(M, N, device="cuda")
    x = torch.rand(M, device="cuda")
    c1, c2 = torch.empty(N, device="cuda"), torch.empty(N, device="cuda")
    blas.sgemv(True, M, N, 1.0, b, x, 0.0, c1, ws=ws)
    blas.sgemv(True, M, N, 1.0, b, x, 0.0, c2, ws=ws)
    assert torch.equal(c1, c2)


def test_sgemv_empty_and_bad_arguments(blas):
    a = torch.zeros(4, 4, device="cuda")
    x = torch.ones(4, device="cuda")
    y = torch.full((4,), 3.0, device="cuda")
    blas.sgemv(False, 4, 0, 1.0, a[:, :0], x[:0], 2.0, y)  # no columns: y = beta * y
    assert torch.equal(y, torch.full((4,), 6.0, device="cuda"))
    blas.sgemv(False, 0, 4, 1.0, a[:0], x, 0.0, y[:0])     # no rows: nothing to do
    from hpcdeepneuralnetworks_amd import _lib
    L = _lib.lib()
    assert L.hpcdnn_sgemv(2, 4, 4, 1.0, a.data_ptr(), 4, x.data_ptr(), 0.0, y.data_ptr(), None, 0, None) == 1
    assert L.hpcdnn_sgemv(0, 4, 4, 1.0, a.data_ptr(), 3, x.data_ptr(), 0.0, y.data_ptr(), None, 0, None) == 1


def _offline_case(blas, oracle_mod, M, N, K, alpha, beta, fault, seed=800, lda=None, ldb=None, ldc=None):
    lda, ldb, ldc = lda or K, ldb or N, ldc or N
    a = oracle_mod.fill_uniform_matrix(M, K, seed, ld=lda)
    b = oracle_mod.fill_uniform_matrix(K, N, seed + 1, ld=ldb)
    c0 = oracle_mod.fill_uniform_matrix(M, N, seed + 2, ld=ldc)
    da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
    panels = -(-K // 256)
    res = torch.full((2 * panels,), float("nan"), device="cuda")
    ws = torch.full((blas.offline_ft_workspace_bytes(M, N, K) // 4,), float("nan"), device="cuda")  # poisoned
    blas.offline_ft_sgemm(M, N, K, da, db, dc, alpha, beta, res, ws, fault=fault)
    c = dc.cpu().numpy()
    c_model = np.where(np.isnan(c0), 0, c0).astype(np.float32)
    c_model[:, :N] = c0[:, :N]
    res_model = oracle_mod.offline_ft_sgemm(M, N, K, a, lda, b, ldb, c_model, ldc, alpha, beta, 256, fault)
    # values: FP64 GEMM criterion, with the (uncorrected) fault added to the reference
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, lda, b, ldb, c0, ldc, alpha, beta)
    if fault is not None:
        ref[fault[1], fault[2]] += fault[3]
        den[fault[1], fault[2]] += abs(fault[3])
    assert oracle_mod.gemm_max_err(N, c, ldc, ref, den) <= TOL
    assert np.all(np.isnan(c[:, N:]))
    return res.cpu().numpy().astype(np.float64), res_model


@pytest.mark.parametrize("M,N,K,alpha,beta", [(512, 384, 1024, 1.0, 0.0), (300, 200, 700, 1.5, -0.5), (1024, 1024, 256, 1.0, 1.0)])
def test_offline_ft_fault_free_residuals_are_noise(blas, oracle_mod, M, N, K, alpha, beta):
    res, res_model = _offline_case(blas, oracle_mod, M, N, K, alpha, beta, None)
    assert np.abs(res_model).max() < 1e-8
    # noise allowance: the sums add M*N entries of magnitude ~sqrt(K/3) rounded to FP32 (relative 6e-8 each,
    # random signs) plus FP32 accumulation in the matrix-vector products: well under 0.05 at these sizes
    assert np.abs(res).max() < 0.05, res


def test_offline_ft_detects_fault_from_its_panel_on(blas, oracle_mod):
    M, N, K = 600, 500, 1100  # 5 panels, the last one ragged; padded leading dimensions
    for fault in [(0, 10, 20, 4.0), (2, 599, 499, -7.5), (4, 0, 0, 3.0)]:
        res, res_model = _offline_case(blas, oracle_mod, M, N, K, 1.0, 1.0, fault, lda=K + 4, ldb=N + 8, ldc=N + 4)
        expect = np.repeat(np.where(np.arange(5) >= fault[0], fault[3], 0.0), 2)
        assert np.abs(res_model - expect).max() < 1e-8
        assert np.abs(res - res_model).max() < 0.05, (fault, res)


def test_offline_ft_bad_arguments(blas):
    from hpcdeepneuralnetworks_amd import _lib
    import ctypes as C
    L = _lib.lib()
    t = torch.zeros(64 * 64, device="cuda")
    p = t.data_ptr()
    # missing workspace, fault outside the matrix / the panels
    assert L.hpcdnn_offline_ft_sgemm(64, 64, 64, p, 64, p, 64, p, 64, 1.0, 0.0, None, p, None, 0, None) == 2
    ws = torch.zeros(blas.offline_ft_workspace_bytes(64, 64, 64) // 4, device="cuda")
    bad = _lib.Fault(1, 0, 0, 1.0)
    assert L.hpcdnn_offline_ft_sgemm(64, 64, 64, p, 64, p, 64, p, 64, 1.0, 0.0, C.byref(bad), p, ws.data_ptr(), ws.numel() * 4, None) == 1
    bad = _lib.Fault(0, 64, 0, 1.0)
    assert L.hpcdnn_offline_ft_sgemm(64, 64, 64, p, 64, p, 64, p, 64, 1.0, 0.0, C.byref(bad), p, ws.data_ptr(), ws.numel() * 4, None) == 1


@pytest.mark.parametrize("M,N,K,alpha,beta,fault", [(512, 384, 1024, 1.0, 0.0, None), (300, 200, 700, 1.5, -0.5, (1, 299, 0, 6.0)),
                                                    (1024, 1024, 256, 1.0, 1.0, (0, 17, 1000, -4.0))])
def test_offline_ft_scalar_checksum(blas, oracle_mod, M, N, K, alpha, beta, fault):
    """One scalar checksum per panel (baseline_ft_sgemm.cuh:36-91): residuals against the FP64 model within the noise
    of adding M*N FP32-rounded entries, C as for SGEMM, and equal to residual [2p] of the row/column variant up to
    the same noise."""
    a = oracle_mod.fill_uniform_matrix(M, K, 850, ld=K + 4)
    b = oracle_mod.fill_uniform_matrix(K, N, 851, ld=N + 4)
    c0 = oracle_mod.fill_uniform_matrix(M, N, 852, ld=N + 8)
    da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
    panels = -(-K // 256)
    res = torch.full((panels,), float("nan"), device="cuda")
    ws = torch.full((blas.offline_ft_workspace_bytes(M, N, K) // 4,), float("nan"), device="cuda")  # poisoned
    blas.offline_ft_sgemm(M, N, K, da, db, dc, alpha, beta, res, ws, fault=fault, scalar=True)
    c_model = c0.copy()
    res_model = oracle_mod.offline_ft_sgemm_scalar(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, alpha, beta, 256, fault)
    got = res.cpu().numpy().astype(np.float64)
    assert np.abs(got - res_model).max() < 0.05, (got, res_model)
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, K + 4, b, N + 4, c0, N + 8, alpha, beta)
    if fault is not None:
        ref[fault[1], fault[2]] += fault[3]
        den[fault[1], fault[2]] += abs(fault[3])
    assert oracle_mod.gemm_max_err(N, dc.cpu().numpy(), N + 8, ref, den) <= TOL
    # the row/column variant's column-side residual is the same quantity
    dc2 = torch.from_numpy(c0).cuda()
    res2 = torch.full((2 * panels,), float("nan"), device="cuda")
    blas.offline_ft_sgemm(M, N, K, da, db, dc2, alpha, beta, res2, ws, fault=fault)
    assert np.abs(got - res2.cpu().numpy()[0::2]).max() < 0.05

