"""GPU parity of the transposed-left-operand SGEMM and of the column-major ``C = alpha*A*B^T + beta*C`` entry point (the
operand layout of the reference's ft_sgemm family, kernel/ft_sgemm/sgemm.cu:111) against the CPU oracle, through the C ABI.

Same acceptance criterion as the row-major tests: max |C - Cref| / (|alpha| (|A||B|)_ij + |beta| |C0_ij|) <= 1e-5 with
Cref accumulated in FP64; and the same bits as ``hpcdnn_sgemm`` on the explicitly transposed operand, since every
element sums its products in the same order.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-5


def _transposed_with_padding(a, M, K, ldat):
    """K x ldat buffer holding a[:, :K]^T with NaN in the padding columns."""
    at = np.full((K, ldat), np.nan, np.float32)
    at[:, :M] = a[:, :K].T
    return at


def _check_tn(oracle_mod, blas, M, N, K, alpha, beta, pad=(0, 0, 0), tile=-1, split_k=0, ws=None, seed=100, same_bits=True):
    ldat, ldb, ldc = max(M, 1) + pad[0], max(N, 1) + pad[1], max(N, 1) + pad[2]
    a = oracle_mod.fill_uniform_matrix(M, K, seed, ld=max(K, 1))
    b = oracle_mod.fill_uniform_matrix(K, N, seed + 1, ld=ldb)
    c0 = oracle_mod.fill_uniform_matrix(M, N, seed + 2, ld=ldc)
    at = _transposed_with_padding(a, M, K, ldat)
    dat, da, db = torch.from_numpy(at).cuda(), torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    dc, dc_nn = torch.from_numpy(c0).cuda(), torch.from_numpy(c0).cuda()
    blas.sgemm_tn(M, N, K, dat, db, dc, alpha, beta, ws=ws, tile=tile, split_k=split_k)
    c = dc.cpu().numpy()
    if M and N:
        ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, a.shape[1], b, ldb, c0, ldc, alpha, beta)
        err = oracle_mod.gemm_max_err(N, c, ldc, ref, den)
        assert err <= TOL, (M, N, K, alpha, beta, tile, split_k, err)
    assert np.all(np.isnan(c[:, N:]))  # padding of C untouched; NaN padding of A^T and B never used
    if same_bits and M and N:
        blas.sgemm(M, N, K, da, db, dc_nn, alpha, beta, ws=ws, tile=tile, split_k=split_k)
        assert torch.equal(dc[:, :N], dc_nn[:, :N]), (M, N, K, tile, split_k)
    return c


def _tiles(blas):
    return list(range(len(blas.tile_table())))


def test_every_tile_small_and_ragged_shapes(blas, oracle_mod):
    shapes = [(1, 1, 1), (5, 7, 3), (33, 31, 17), (64, 64, 64), (130, 70, 40), (257, 129, 33), (40, 300, 8), (300, 40, 100),
              (256, 256, 48), (512, 384, 160)]
    for tile in _tiles(blas):
        for i, (M, N, K) in enumerate(shapes):
            _check_tn(oracle_mod, blas, M, N, K, 1.0, 0.0, pad=((0, 0, 0), (3, 5, 8))[i % 2], tile=tile, split_k=1, seed=400 + tile)


@pytest.mark.parametrize("alpha,beta", [(1.5, -0.5), (0.0, 2.0), (-1.0, 1.0)])
def test_alpha_beta_and_padded_leading_dimensions(blas, oracle_mod, alpha, beta):
    for tile in (0, 1, 7, 12):
        _check_tn(oracle_mod, blas, 300, 200, 150, alpha, beta, pad=(5, 3, 9), tile=tile, split_k=1, seed=430)


def test_split_k_and_tail_split_give_the_bits_of_the_untransposed_call(blas, oracle_mod):
    for (M, N, K, tile, split) in [(128, 128, 4096, 1, 8), (256, 128, 2048, 0, 4), (200, 100, 1000, 4, 3), (64, 64, 8192, 12, 16)]:
        ws = blas.workspace(M * N * split * 4)
        _check_tn(oracle_mod, blas, M, N, K, 1.0, 1.0, pad=(0, 4, 4), tile=tile, split_k=split, ws=ws, seed=450)
    # tail split: 17 x 16 = 272 tiles of 128 x 128 on 256 CUs leave 16 tiles for a second round
    M, N, K = 17 * 128, 16 * 128, 512
    ws = blas.workspace(64 << 20)
    _check_tn(oracle_mod, blas, M, N, K, 1.0, 0.0, tile=1, split_k=-4, ws=ws, seed=460)


@pytest.mark.parametrize("M,N,K,use_ws", [(1000, 1000, 1000, True), (128, 128, 16384, True), (2304, 2304, 1040, True), (4608, 4608, 512, False),
                                         (1, 700, 300, False), (700, 1, 300, True), (31, 33, 1, False), (1023, 513, 2049, True)])
def test_library_chosen_plans(blas, oracle_mod, M, N, K, use_ws):
    """Whatever the selector picks (split-K, tail split, two launches over row ranges): FP64 criterion on every element."""
    ws = blas.workspace(max(blas.sgemm_workspace_bytes(M, N, K), 1 << 20)) if use_ws else None
    _check_tn(oracle_mod, blas, M, N, K, 1.0, -1.5, pad=(1, 2, 3), ws=ws, seed=470, same_bits=False)


def test_hand_cases_that_a_wrong_transposition_fails(blas):
    dev = "cuda"
    # At[k][m] = 1 iff k == perm[m], i.e. A[m][k] picks row perm[m] of B: C = B[perm] exactly; At read untransposed
    # would give the inverse permutation
    M, N, K = 96, 80, 96
    perm = torch.randperm(K, device=dev)[:M]
    at = torch.zeros(K, M, device=dev)
    at[perm, torch.arange(M, device=dev)] = 1.0
    b = torch.rand(K, N, device=dev)
    c = torch.empty(M, N, device=dev)
    blas.sgemm_tn(M, N, K, at, b, c, 1.0, 0.0)
    assert torch.equal(c, b[perm])
    # index-valued operands on a rectangular problem: C[m][n] = m * n * K, exact in FP32 for these sizes
    M, N, K = 70, 50, 16
    at = torch.arange(M, device=dev, dtype=torch.float32)[None, :].expand(K, M).contiguous()
    bj = torch.arange(N, device=dev, dtype=torch.float32)[None, :].expand(K, N).contiguous()
    c = torch.empty(M, N, device=dev)
    blas.sgemm_tn(M, N, K, at, bj, c, 1.0, 0.0)
    assert torch.equal(c, (torch.arange(M, device=dev)[:, None] * torch.arange(N, device=dev)[None, :] * K).float())
    # column-major entry point on the same idea: A[m][k] = m, B[n][k] = 10 n, C[m + n*M] = 10 m n K
    a_cm = torch.arange(M, device=dev, dtype=torch.float32)[None, :].expand(K, M).contiguous()       # memory of column-major A
    b_cm = (10 * torch.arange(N, device=dev, dtype=torch.float32))[None, :].expand(K, N).contiguous()
    c_cm = torch.empty(N, M, device=dev)                                                              # memory of column-major C
    blas.sgemm_cm_nt(M, N, K, a_cm, b_cm, c_cm, 1.0, 0.0)
    assert torch.equal(c_cm, (10 * torch.arange(N, device=dev)[:, None] * torch.arange(M, device=dev)[None, :] * K).float())


def test_empty_and_k_zero(blas):
    dummy = torch.zeros(8, 8, device="cuda")
    c = torch.full((4, 6), 2.0, device="cuda")
    blas.sgemm_tn(0, 6, 5, dummy, dummy, c, 1.0, 0.0)   # nothing to do
    blas.sgemm_tn(4, 0, 5, dummy, dummy, c, 1.0, 0.0)
    assert torch.equal(c, torch.full((4, 6), 2.0, device="cuda"))
    blas.sgemm_tn(4, 6, 0, dummy, dummy, c, 1.0, 0.5)   # K = 0: C = beta * C without reading A or B
    assert torch.equal(c, torch.full((4, 6), 1.0, device="cuda"))


def test_large_whole_tile_shape_matches_untransposed_bits(blas, oracle_mod):
    M, N, K = 4096, 2048, 1024
    da, db = torch.empty(M, K, device="cuda"), torch.empty(K, N, device="cuda")
    blas.fill_uniform_matrix(da, M, K, 41)
    blas.fill_uniform_matrix(db, K, N, 42)
    dat = da.t().contiguous()
    c1 = torch.full((M, N), float("nan"), device="cuda")
    c2 = torch.full((M, N), float("nan"), device="cuda")
    blas.sgemm_tn(M, N, K, dat, db, c1, 1.0, 0.0)
    blas.sgemm(M, N, K, da, db, c2, 1.0, 0.0)
    assert torch.equal(c1, c2)
    rows = np.array([0, 1, 777, 4095], np.int32)
    a = oracle_mod.fill_uniform_matrix(M, K, 41)
    b = oracle_mod.fill_uniform_matrix(K, N, 42)
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, K, b, N, None, N, 1.0, 0.0, rows=rows)
    got = np.ascontiguousarray(c1[torch.from_numpy(rows).long().cuda()].cpu().numpy())
    assert oracle_mod.gemm_max_err(N, got, N, ref, den) <= TOL


@pytest.mark.parametrize("M,N,K,tile", [(2176, 4608, 320, 7), (4352, 2304, 192, 0), (3264, 4608, 320, 5), (2176, 4608, 320, 1)])
@pytest.mark.parametrize("alpha,beta", [(1.5, 0.0), (1.0, -1.5)])
def test_persistent_kernels_on_several_rounds_of_whole_tiles(blas, oracle_mod, M, N, K, tile, alpha, beta):
    """More whole tiles than CUs and an even number (>= 10) of K steps: the persistent kernels of the 256x128, 128x256,
    192x256 (beta == 0 only) and 128x128 tiles run, here with the transposed staging.  Same bits as the 128x64
    tile-per-workgroup kernel on the untransposed operand; padded ldat / ldc with NaN padding, NaN in C when beta == 0."""
    dev = "cuda"
    ldat, ldc = M + 8, N + 24
    da, db = torch.empty(M, K, device=dev), torch.empty(K, N, device=dev)
    blas.fill_uniform_matrix(da, M, K, 51)
    blas.fill_uniform_matrix(db, K, N, 52)
    dat = torch.full((K, ldat), float("nan"), device=dev)
    dat[:, :M] = da.t()
    c0 = torch.full((M, ldc), float("nan"), device=dev)
    if beta != 0.0:
        c0[:, :N] = torch.rand(M, N, device=dev) * 2 - 1
    c1, c2 = c0.clone(), c0.clone()
    blas.sgemm_tn(M, N, K, dat, db, c1, alpha, beta, tile=tile, split_k=1)
    blas.sgemm(M, N, K, da, db, c2, alpha, beta, tile=2, split_k=1)
    assert torch.equal(c1[:, :N], c2[:, :N])
    assert not torch.isnan(c1[:, :N]).any()
    assert torch.isnan(c1[:, N:]).all()
    rows = np.array([0, 1, M // 2 + 3, M - 1], np.int32)
    a, b = oracle_mod.fill_uniform_matrix(M, K, 51), oracle_mod.fill_uniform_matrix(K, N, 52)
    c0h = np.ascontiguousarray(c0[:, :N].cpu().numpy()) if beta != 0.0 else None
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, K, b, N, c0h, N, alpha, beta, rows=rows)
    got = np.ascontiguousarray(c1[torch.from_numpy(rows).long().cuda(), :N].cpu().numpy())
    assert oracle_mod.gemm_max_err(N, got, N, ref, den) <= TOL


@pytest.mark.parametrize("M,N,K,pad", [(128, 128, 128, (0, 0, 0)), (1024, 1024, 1024, (0, 0, 0)), (300, 170, 90, (4, 7, 2)), (17, 400, 33, (1, 0, 5)),
                                      (1, 1, 1, (0, 0, 0)), (513, 64, 2050, (3, 3, 3))])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (1.0, -1.5)])
def test_column_major_a_b_transposed(blas, oracle_mod, M, N, K, pad, alpha, beta):
    """The reference's column-major family: C (M x N, ldc) = alpha * A (M x K, lda) * B (N x K, ldb)^T + beta * C, checked
    against the oracle's restatement of that indexing (kernel/ft_sgemm/include/sgemm_huge.cuh:14, kernel/ft_sgemm/sgemm.cu:111).
    1024^3 with alpha = 1, beta = -1.5 is the driver's own case (kernel/ft_sgemm/sgemm.cu:25-26)."""
    lda, ldb, ldc = M + pad[0], N + pad[1], M + pad[2]
    abuf = oracle_mod.fill_uniform_matrix(K, M, 500, ld=lda)   # column k of A = row k of the buffer
    bbuf = oracle_mod.fill_uniform_matrix(K, N, 501, ld=ldb)
    cbuf = oracle_mod.fill_uniform_matrix(N, M, 502, ld=ldc)
    da, db, dc = torch.from_numpy(abuf).cuda(), torch.from_numpy(bbuf).cuda(), torch.from_numpy(cbuf).cuda()
    ws = blas.workspace(max(blas.sgemm_workspace_bytes(N, M, K), 1 << 16))
    blas.sgemm_cm_nt(M, N, K, da, db, dc, alpha, beta, ws=ws)
    c = dc.cpu().numpy()
    ref, den = oracle_mod.gemm_cm_nt_f64(M, N, K, abuf, lda, bbuf, ldb, cbuf, ldc, alpha, beta)
    assert oracle_mod.gemm_max_err(M, c, ldc, ref, den) <= TOL
    assert np.all(np.isnan(c[:, M:]))


def test_operands_that_start_four_bytes_off_a_16_byte_boundary(blas, oracle_mod):
    """A^T, B and C as views that begin one float into their allocations, with odd leading dimensions: no row of any
    operand starts on a 16-byte boundary, for plain SGEMM (two tile families) and for ABFT in both modes."""
    M, N, K = 203, 149, 77
    ldat, ldb, ldc = M + 2, N + 2, M + 4                      # column-major C: N rows of M in memory
    a = oracle_mod.fill_uniform_matrix(K, M, 520, ld=ldat)
    b = oracle_mod.fill_uniform_matrix(K, N, 521, ld=ldb)
    c0 = oracle_mod.fill_uniform_matrix(N, M, 522, ld=ldc)
    ref, den = oracle_mod.gemm_cm_nt_f64(M, N, K, a, ldat, b, ldb, c0, ldc, 1.0, -0.5)

    def off_by_one(x):
        buf = torch.full((x.size + 1,), float("nan"), device="cuda")
        buf[1:] = torch.from_numpy(x.ravel()).cuda()
        return buf[1:].view(x.shape)

    da, db = off_by_one(a), off_by_one(b)
    assert da.data_ptr() % 16 == 4
    for run in ("sgemm", "ft_fused", "ft_workspace"):
        dc = off_by_one(c0)
        if run == "sgemm":
            blas.sgemm_cm_nt(M, N, K, da, db, dc, 1.0, -0.5)
        else:
            ws = blas.workspace(blas.ft_cm_nt_workspace_bytes(M, N, K)) if run == "ft_workspace" else None
            blas.ft_sgemm_cm_nt(M, N, K, da, db, dc, 1.0, -0.5, ws)
        c = dc.cpu().numpy()
        assert oracle_mod.gemm_max_err(M, c, ldc, ref, den) <= TOL, run
        assert np.all(np.isnan(c[:, M:])), run
    # the transposed-operand entry point with a pinned big tile on the same buffers: C^T (N x M) = B^T^T A^T
    dc = off_by_one(c0)
    blas.sgemm_tn(N, M, K, db, da, dc, 1.0, -0.5, tile=0, split_k=1)
    assert oracle_mod.gemm_max_err(M, dc.cpu().numpy(), ldc, ref, den) <= TOL


def test_alternating_layouts_on_one_thread(blas):
    """The library remembers its last plan per thread; calls that alternate between the two layouts (and between shapes
    that take two launches over row ranges, a K split and a plain launch) must not pick up each other's decision."""
    shapes = [(3584, 3584, 256, False), (128, 128, 8192, True), (700, 300, 200, False)]
    ops = []
    for i, (M, N, K, use_ws) in enumerate(shapes):
        a = torch.empty(M, K, device="cuda")
        b = torch.empty(K, N, device="cuda")
        blas.fill_uniform_matrix(a, M, K, 60 + i)
        blas.fill_uniform_matrix(b, K, N, 70 + i)
        ws = blas.workspace(max(blas.sgemm_workspace_bytes(M, N, K), 1 << 16)) if use_ws else None
        ref = torch.empty(M, N, device="cuda")
        blas.sgemm(M, N, K, a, b, ref, 1.0, 0.0, ws=ws)
        ops.append((M, N, K, a, a.t().contiguous(), b, ws, ref))
    for rep in range(3):
        for (M, N, K, a, at, b, ws, ref) in ops:
            c1 = torch.full((M, N), float("nan"), device="cuda")
            c2 = torch.full((M, N), float("nan"), device="cuda")
            blas.sgemm_tn(M, N, K, at, b, c1, 1.0, 0.0, ws=ws)
            blas.sgemm(M, N, K, a, b, c2, 1.0, 0.0, ws=ws)
            assert torch.equal(c1, ref) and torch.equal(c2, ref), (rep, M, N, K)


def test_maximum_leading_dimensions(blas):
    """ldat and ldb at the documented limit of the K-major operands (a K step is 16 of their rows; byte offsets inside one
    tile are 32-bit) and ldc at its own, for several kernel families and for the ABFT entry point; one more is refused."""
    ldat, ldb, ldc = (1 << 25) - 1024, (1 << 25) - 1024, (1 << 21) - 64
    M, N, K = 300, 100, 40
    atbuf = torch.empty(K * ldat + 8, device="cuda")
    bbuf = torch.empty(K * ldb + 8, device="cuda")
    at, b = atbuf[:K * ldat].view(K, ldat)[:, :M], bbuf[:K * ldb].view(K, ldb)[:, :N]
    gen = torch.Generator(device="cuda").manual_seed(5)
    at.copy_(torch.rand(K, M, device="cuda", generator=gen) * 2 - 1)
    b.copy_(torch.rand(K, N, device="cuda", generator=gen) * 2 - 1)
    ref = at.double().t() @ b.double()
    den = at.abs().double().t() @ b.abs().double()
    cbuf = torch.empty(M * ldc, device="cuda")
    c = cbuf.view(M, ldc)[:, :N]
    c0 = torch.rand(M, N, device="cuda", generator=gen) * 2 - 1
    for tile in (-1, 0, 4, 8, len(blas.tile_table()) - 1):
        for beta in (0.0, -1.5):
            c.copy_(c0)
            blas.sgemm_tn(M, N, K, at, b, c, 1.0, beta, tile=tile, split_k=0 if tile < 0 else 1)
            assert float(((c.double() - ref - beta * c0.double()).abs() / (den + abs(beta) * c0.abs().double())).max()) <= TOL, (tile, beta)
    # the column-major ABFT entry point on the same buffers: A (M x K, lda = ldat), B (N x K, ldb), C (M x N) held as N x M
    ccm = torch.zeros(N, M, device="cuda")
    blas.ft_sgemm_cm_nt(M, N, K, at, b, ccm, 1.0, 0.0, None)
    assert float(((ccm.double() - ref.t()).abs() / den.t()).max()) <= TOL
    with pytest.raises(blas.HpcdnnError):
        blas.sgemm_tn(M, N, 8, atbuf[:7 * (ldat + 1) + M].as_strided((8, M), (ldat + 1, 1)), b, torch.zeros(M, N, device="cuda"), 1.0, 0.0)


def test_bad_arguments(blas):
    from hpcdeepneuralnetworks_amd.blas import HpcdnnError
    x = torch.zeros(64, 64, device="cuda")
    small = [t for t, (bm, bn, _) in enumerate(blas.tile_table()) if (bm, bn) == (32, 32)]
    with pytest.raises(HpcdnnError):
        blas.sgemm_tn(64, 64, 64, x, x, x, 1.0, 0.0, ws=blas.workspace(1 << 20), tile=small[0], split_k=-2)   # the 32 x 32 tile has no tail split
    with pytest.raises(HpcdnnError):
        blas.sgemm_tn(65, 64, 64, x, x, torch.zeros(65, 64, device="cuda"), 1.0, 0.0)   # At narrower than M
