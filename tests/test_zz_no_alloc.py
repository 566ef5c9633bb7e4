"""The entry point that allocates nothing: hpcdnn_ft_sgemm_static keeps its scratch in a fixed device array of the
library.  Its results must equal those of hpcdnn_ft_sgemm called with a workspace (same kernels, same order of
operations: bit-identical C, identical status records), on two calls in a row, the second on a smaller problem, so
that anything the first call left in the array would show."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

FIELDS = ("flag", "row", "col", "n_bad_rows", "n_bad_cols", "row_residual", "col_residual", "max_clean_residual")


def _both(blas, oracle_mod, M, N, K, alpha, beta, fault, seed):
    a = oracle_mod.fill_uniform_matrix(M, K, seed, ld=K + 4)
    b = oracle_mod.fill_uniform_matrix(K, N, seed + 1, ld=N + 4)
    c0 = oracle_mod.fill_uniform_matrix(M, N, seed + 2, ld=N + 8)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    tau = blas.ft_default_tau(K)
    # reference: the existing entry point with a caller-provided (poisoned) workspace of the array's size, so that
    # both take the same decisions about splitting a partial last round along K
    ws = torch.full((blas.FT_STATIC_SCRATCH_BYTES // 4,), float("nan"), dtype=torch.float32, device="cuda")
    c_ws = torch.from_numpy(c0).cuda()
    st_ws = blas.ft_status_alloc(M, N)
    blas.ft_sgemm(M, N, K, da, db, c_ws, alpha, beta, tau=tau, fault=fault, status=st_ws, ws=ws)
    c_st = torch.from_numpy(c0).cuda()
    st_st = blas.ft_status_alloc(M, N)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    blas.ft_sgemm_static(M, N, K, da, db, c_st, alpha, beta, tau=tau, fault=fault, status=st_st)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return a, b, c0, c_ws.cpu().numpy(), blas.ft_status_numpy(st_ws), c_st.cpu().numpy(), blas.ft_status_numpy(st_st)


def _same(r, N):
    a, b, c0, c_ws, st_ws, c_st, st_st = r
    assert np.array_equal(c_ws[:, :N], c_st[:, :N])
    assert np.all(np.isnan(c_st[:, N:]))
    for f in FIELDS:
        assert np.array_equal(st_ws[f], st_st[f]), f


def test_static_scratch_entry_point_equals_the_workspace_one_twice_in_a_row(blas, oracle_mod):
    # first call: 250 x 380 x 2048 -> three 256 x 128 tiles, all split 8 ways along K (checksum vectors and K slices
    # both live in the array: 3.1 MiB), one fault; second call: a smaller, ragged problem with a different fault
    assert blas.ft_workspace_bytes(250, 380, 2048) > 3 << 20
    big = _both(blas, oracle_mod, 250, 380, 2048, 1.5, -1.0, (1, 17, 90, 12.5), 3100)
    _same(big, 380)
    assert big[6]["flag"][1] == 1 and (big[6]["row"][1], big[6]["col"][1]) == (17, 90)
    small = _both(blas, oracle_mod, 300, 200, 100, 1.0, 0.0, (3, 40, 70, -0.75), 3200)
    _same(small, 200)
    assert small[6]["flag"][3] == 1 and (small[6]["row"][3], small[6]["col"][3]) == (40, 70)
    # and against the oracle, like every other ABFT path
    a, b, c0, _, _, c_st, st_st = small
    c_model = c0.copy()
    st_model = oracle_mod.ft_sgemm(300, 200, 100, a, 104, b, 204, c_model, 208, 1.0, 0.0, 256, 128, blas.ft_default_tau(100), (3, 40, 70, -0.75))
    for f in ("flag", "row", "col", "n_bad_rows", "n_bad_cols"):
        assert np.array_equal(st_st[f], st_model[f]), f
    ref, den = oracle_mod.gemm_f64_rows(300, 200, 100, a, 104, b, 204, c0, 208, 1.0, 0.0)
    assert oracle_mod.gemm_max_err(200, c_st, 208, ref, den) <= 1e-5
    # fault-free repeat of the first shape: nothing of the two earlier calls is left behind
    clean = _both(blas, oracle_mod, 250, 380, 2048, 1.5, -1.0, None, 3100)
    _same(clean, 380)
    assert np.all(clean[6]["flag"] == 0)


def test_static_scratch_entry_point_refuses_what_does_not_fit(blas):
    n = 12288   # (48 + 96) tile rows and columns x (768 + 2) K steps x 64 bytes = 6.8 MiB of checksum vectors
    t = torch.zeros(1, device="cuda")
    from hpcdeepneuralnetworks_amd import _lib
    L = _lib.lib()
    rc = L.hpcdnn_ft_sgemm_static(n, n, n, t.data_ptr(), n, t.data_ptr(), n, t.data_ptr(), n, 1.0, 0.0, 0.0, None, None, None)
    assert rc == 2 and b"workspace" in L.hpcdnn_error_string(rc)   # refused before anything is launched
