"""Every entry point only enqueues kernels on the caller's stream (no allocation, no memset, no synchronisation), so a
sequence of calls can be captured into a HIP graph and replayed.  Each replay is checked against the eager result,
with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_captured_sequence_replays_like_eager(blas):
    dev = "cuda"
    M, N, K, nv = 768, 640, 1100, (1 << 18) + 5
    a = torch.empty(M, K, device=dev)
    b = torch.empty(K, N, device=dev)
    blas.fill_uniform_matrix(a, M, K, 11)
    blas.fill_uniform_matrix(b, K, N, 12)
    c_plain = torch.zeros(M, N, device=dev)
    c_split = torch.zeros(M, N, device=dev)
    c_ft = torch.zeros(M, N, device=dev)
    x = torch.empty(nv, device=dev)
    y0 = torch.empty(nv, device=dev)
    blas.fill_uniform(x, 13)
    blas.fill_uniform(y0, 14)
    y = y0.clone()
    dot = torch.zeros(1, device=dev)
    gv = torch.zeros(N, device=dev)
    status = blas.ft_status_alloc(M, N)
    ws_split = blas.workspace(M * N * 4 * 4)
    ws_ft = blas.workspace(blas.ft_workspace_bytes(M, N, K))
    ws_dot = blas.workspace(64 + 8 * 4096)
    ws_gv = blas.workspace(max(blas.sgemv_workspace_bytes(M, N), 4))
    fault = (3, 17, 33, 2.5)
    # the same product on column-major operands: A as its K x M row-major transpose, B (N x K) = the memory of b, C as N x M
    a_t = a.t().contiguous()
    c_cm = torch.zeros(N, M, device=dev)
    c_ftcm = torch.zeros(N, M, device=dev)
    status_cm = blas.ft_status_alloc(N, M)
    ws_ftcm = blas.workspace(blas.ft_cm_nt_workspace_bytes(M, N, K))
    fault_cm = (2, 5, 9, 1.5)

    def sequence():
        blas.sgemm(M, N, K, a, b, c_plain, 1.0, 0.0)
        blas.sgemm(M, N, K, a, b, c_split, 1.0, 0.0, ws=ws_split, tile=1, split_k=4)
        blas.ft_sgemm(M, N, K, a, b, c_ft, 1.0, 0.0, fault=fault, status=status, ws=ws_ft)
        blas.saxpy(nv, 0.5, x, y)
        blas.sdot(nv, x, y, dot, ws=ws_dot)
        blas.sgemv(True, M, N, 1.0, c_plain, x[:M], 0.0, gv, ws=ws_gv)
        blas.sgemm_cm_nt(M, N, K, a_t, b, c_cm, 1.0, 0.0)
        blas.ft_sgemm_cm_nt(M, N, K, a_t, b, c_ftcm, 1.0, 0.0, ws_ftcm, status=status_cm, faults=[fault_cm])

    # eager reference (y accumulates: replay r leaves y = y0 + 0.5 * (r + 1) * x applied step by step)
    sequence()
    torch.cuda.synchronize()
    ref_plain, ref_split, ref_ft = c_plain.clone(), c_split.clone(), c_ft.clone()
    ref_status = blas.ft_status_numpy(status).copy()
    ref_gv = gv.clone()
    ref_cm, ref_ftcm = c_cm.clone(), c_ftcm.clone()
    ref_status_cm = blas.ft_status_numpy(status_cm).copy()
    assert ref_status_cm["flag"][2] == 1 and (ref_status_cm["row"][2], ref_status_cm["col"][2]) == (5, 9)
    assert torch.allclose(ref_cm.t(), ref_plain, rtol=0, atol=1e-3)
    assert ref_status["flag"][3] == 1 and (ref_status["row"][3], ref_status["col"][3]) == (17, 33)

    y.copy_(y0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        sequence()  # warm-up on the capture stream
        torch.cuda.synchronize()
        y.copy_(y0)
        with torch.cuda.graph(graph, stream=side):
            sequence()
    torch.cuda.synchronize()

    y_eager = y0.clone()
    for replay in range(4):
        for t in (c_plain, c_split, c_ft, gv, c_cm, c_ftcm):
            t.fill_(float("nan"))          # eager work between replays: results must come from the replay itself
        status.zero_()
        status_cm.zero_()
        dot.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        blas.saxpy(nv, 0.5, x, y_eager)    # the eager twin of the captured SAXPY
        dot_eager = torch.zeros(1, device=dev)
        blas.sdot(nv, x, y_eager, dot_eager)
        torch.cuda.synchronize()
        assert torch.equal(c_plain, ref_plain) and torch.equal(c_split, ref_split) and torch.equal(c_ft, ref_ft), replay
        assert torch.equal(gv, ref_gv), replay
        assert torch.equal(c_cm, ref_cm) and torch.equal(c_ftcm, ref_ftcm), replay
        assert np.array_equal(blas.ft_status_numpy(status_cm)["flag"], ref_status_cm["flag"]), replay
        assert torch.equal(y, y_eager), replay
        assert torch.equal(dot, dot_eager), replay
        st = blas.ft_status_numpy(status)
        for f in ("flag", "row", "col", "n_bad_rows", "n_bad_cols"):
            assert np.array_equal(st[f], ref_status[f]), (replay, f)
