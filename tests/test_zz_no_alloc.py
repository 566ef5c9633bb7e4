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


_CAPTURE_SCRIPT = r"""
import sys
import numpy as np
import torch
sys.path.insert(0, sys.argv[1])
import oracle
from hpcdeepneuralnetworks_amd import blas, _lib

M, N, K = 300, 200, 420
tau = blas.ft_default_tau(K)
a = torch.from_numpy(oracle.fill_uniform_matrix(M, K, 1)).cuda()
b = torch.from_numpy(oracle.fill_uniform_matrix(K, N, 2)).cuda()
c0 = torch.from_numpy(oracle.fill_uniform_matrix(M, N, 3)).cuda()
c = c0.clone()
status = blas.ft_status_alloc(M, N)
fault = (3, 40, 70, -0.75)
side = torch.cuda.Stream()
side.wait_stream(torch.cuda.current_stream())

# 1. the very first call of the process under capture: refused with the set-up error, nothing enqueued
graph = torch.cuda.CUDAGraph()
refused = False
with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
        try:
            blas.ft_sgemm_static(M, N, K, a, b, c, 1.5, -1.0, tau=tau, fault=fault, status=status)
        except blas.HpcdnnError as e:
            refused = "set-up" in str(e)
assert refused, "a first call under capture must be refused"
torch.cuda.synchronize()

# 2. the documented remedy: one eager call that launches nothing
rc = _lib.lib().hpcdnn_ft_sgemm_static(0, 0, 0, None, 1, None, 1, None, 1, 1.0, 0.0, 0.0, None, None, None)
assert rc == 0, rc

# 3. now the call can be captured, without any eager call on these operands before
graph = torch.cuda.CUDAGraph()
with torch.cuda.stream(side):
    with torch.cuda.graph(graph, stream=side):
        blas.ft_sgemm_static(M, N, K, a, b, c, 1.5, -1.0, tau=tau, fault=fault, status=status)
torch.cuda.synchronize()

def reference():
    ws = torch.full((blas.FT_STATIC_SCRATCH_BYTES // 4,), float("nan"), dtype=torch.float32, device="cuda")
    c_ws, st_ws = c0.clone(), blas.ft_status_alloc(M, N)
    blas.ft_sgemm(M, N, K, a, b, c_ws, 1.5, -1.0, tau=tau, fault=fault, status=st_ws, ws=ws)
    torch.cuda.synchronize()
    return c_ws, blas.ft_status_numpy(st_ws)

for replay in range(3):
    if replay:   # changed operands between the replays, and eager work on the device
        a.mul_(-0.5)
        b.add_(0.25)
    c.copy_(c0)
    status.zero_()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    c_ws, st_ws = reference()
    assert torch.equal(c, c_ws), replay
    st = blas.ft_status_numpy(status)
    assert np.array_equal(st, st_ws), replay
    assert st["flag"][3] == 1 and (st["row"][3], st["col"][3]) == (40, 70), replay
print("CAPTURE-OK")
"""


def test_static_scratch_entry_point_under_stream_capture():
    """The entry point is meant for code under HIP graph capture.  Its one-time set-up per device (address of the array,
    LDS limit of its kernels) cannot be captured: a first call under capture is refused with HPCDNN_ERR_NOT_READY, and
    after one eager call that launches nothing the call is captured and replayed - with changed operands between the
    replays - bit for bit like the workspace entry point.  A process of its own, so that the call under capture really is
    the first."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-c", _CAPTURE_SCRIPT, root], capture_output=True, text=True, timeout=280)
    assert p.returncode == 0 and "CAPTURE-OK" in p.stdout, (p.stdout[-2000:], p.stderr[-4000:])
