"""GPU parity of SGEMM against the CPU oracle, through the C ABI.

Acceptance criterion (stated tolerance): max |C - Cref| / (|alpha| (|A||B|)_ij + |beta| |C0_ij|) <= 1e-5 with Cref
accumulated in FP64.  Small shapes are checked on every element, large ones on sampled rows plus a Freivalds
check (C v against A (B v) in FP64) that covers every element.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-5


def _problem(oracle_mod, M, N, K, lda=None, ldb=None, ldc=None, seed=100):
    lda, ldb, ldc = lda or max(K, 1), ldb or max(N, 1), ldc or max(N, 1)
    a = oracle_mod.fill_uniform_matrix(M, K, seed, ld=lda)
    b = oracle_mod.fill_uniform_matrix(K, N, seed + 1, ld=ldb)
    c = oracle_mod.fill_uniform_matrix(M, N, seed + 2, ld=ldc)
    return a, b, c


def _check(oracle_mod, blas, M, N, K, alpha, beta, lda=None, ldb=None, ldc=None, tile=-1, split_k=0, ws=None, seed=100):
    a, b, c0 = _problem(oracle_mod, M, N, K, lda, ldb, ldc, seed)
    da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
    blas.sgemm(M, N, K, da, db, dc, alpha, beta, ws=ws, tile=tile, split_k=split_k)
    c = dc.cpu().numpy()
    if M and N:
        ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, a.shape[1], b, b.shape[1], c0, c0.shape[1], alpha, beta)
        err = oracle_mod.gemm_max_err(N, c, c.shape[1], ref, den)
        assert err <= TOL, (M, N, K, alpha, beta, tile, split_k, err)
    # padding columns of C (NaN) are never written; padding of A and B (NaN) is never used
    assert np.all(np.isnan(c[:, N:]))
    return c


def test_config1_1024_cube_against_reference_cpu_gemm(blas, oracle_mod):
    """The reference's own CPU-checkable case: M=N=K=1024, alpha=1, beta=0, C zero-initialised, validated against the reference's
    CPU triple loop (utils/utils.cu:93-103) and against the FP64 criterion."""
    n = 1024
    a = oracle_mod.fill_uniform_matrix(n, n, 1)
    b = oracle_mod.fill_uniform_matrix(n, n, 2)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    dc = torch.zeros(n, n, dtype=torch.float32, device="cuda")
    blas.sgemm(n, n, n, da, db, dc, 1.0, 0.0)
    c = dc.cpu().numpy()
    c_ref = np.zeros((n, n), dtype=np.float32)
    oracle_mod.cpu_gemm(1.0, 0.0, a, b, n, c_ref)
    assert np.max(np.abs(c - c_ref)) < 1e-2            # the reference's own acceptance test (utils.cu:84)
    ref, den = oracle_mod.gemm_f64_rows(n, n, n, a, n, b, n, None, n, 1.0, 0.0)
    assert oracle_mod.gemm_max_err(n, c, n, ref, den) <= TOL
    # the reference's calling convention: sgemm(N, A, B, C, alpha, beta) with square packed operands
    dc2 = torch.zeros(n, n, dtype=torch.float32, device="cuda")
    blas.sgemm(n, n, n, da, db, dc2, 1.0, 0.0, tile=1)
    assert oracle_mod.gemm_max_err(n, dc2.cpu().numpy(), n, ref, den) <= TOL


def _num_tiles(blas):
    return len(blas.tile_table())


def test_every_tile_config_small_and_ragged_shapes(blas, oracle_mod):
    shapes = [(1, 1, 1), (5, 7, 3), (33, 31, 17), (64, 64, 64), (130, 70, 40), (257, 129, 33), (40, 300, 8), (300, 40, 100)]
    for tile in range(_num_tiles(blas)):
        for (M, N, K) in shapes:
            _check(oracle_mod, blas, M, N, K, 1.0, 0.0, tile=tile, seed=200 + tile)


def test_unsplit_products_have_the_bits_of_the_summation_order_model(blas, oracle_mod):
    """Every tile of the LDS-staged kernel (and the persistent kernels the library picks for large products) sums each
    element of C in one float accumulator, one fused multiply-add per k, k permuted 0,4,1,5,... inside each group of
    16: the CPU model of that order predicts the result bit for bit - ragged shapes, padded leading dimensions,
    alpha/beta included.  (The 32x32 small-problem tile splits K over its waves and sums in another order.)"""
    small_tile = [i for i, t in enumerate(blas.tile_table()) if t[0] == 32 and t[1] == 32]
    shapes = [(1, 1, 1), (33, 31, 17), (130, 70, 40), (257, 129, 100), (300, 200, 333)]
    for tile in range(_num_tiles(blas)):
        if tile in small_tile:
            continue
        for (M, N, K) in shapes:
            for alpha, beta in ((1.0, 0.0), (1.5, -0.75)):
                a, b, c0 = _problem(oracle_mod, M, N, K, K + 3, N + 1, N + 2, seed=900 + tile)
                da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
                blas.sgemm(M, N, K, da, db, dc, alpha, beta, tile=tile, split_k=1)
                want = c0.copy()
                oracle_mod.sgemm_device_order(M, N, K, a, K + 3, b, N + 1, want, N + 2, alpha, beta)
                got = dc.cpu().numpy()
                assert np.array_equal(got[:, :N], want[:, :N]), (tile, M, N, K, alpha, beta)
    # the library's own choice on a product large enough for the persistent kernel, K not a multiple of 16
    M, N, K = 2048, 1536, 200
    a, b, c0 = _problem(oracle_mod, M, N, K, seed=950)
    da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
    blas.sgemm(M, N, K, da, db, dc, 1.0, 1.0)
    want = c0.copy()
    oracle_mod.sgemm_device_order(M, N, K, a, K, b, N, want, N, 1.0, 1.0)
    assert np.array_equal(dc.cpu().numpy(), want)


@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (1.0, 1.0), (1.5, -1.0), (1.0, -1.5), (0.0, 2.0), (-0.5, 0.0)])
def test_alpha_beta_pairs_with_padded_leading_dimensions(blas, oracle_mod, alpha, beta):
    # 1.5/-1.0 and 1.0/-1.5 are the reference drivers' values (kernel/sgemm/sgemm.cu:33-34, ft_sgemm/sgemm.cu:32-34)
    _check(oracle_mod, blas, 200, 150, 90, alpha, beta, lda=96, ldb=152, ldc=160)
    _check(oracle_mod, blas, 200, 150, 90, alpha, beta, lda=91, ldb=151, ldc=153)  # odd ld: unaligned rows


def test_beta_zero_ignores_nan_in_c(blas, oracle_mod):
    M, N, K = 100, 60, 50
    a, b, _ = _problem(oracle_mod, M, N, K)
    dc = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    blas.sgemm(M, N, K, torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), dc, 1.0, 0.0)
    assert torch.isfinite(dc).all()


def test_every_edge_residue_brute_force(blas, oracle_mod):
    # every (M, N, K) residue class of the vector width and a few around the MFMA block size
    vals = [1, 2, 3, 4, 5, 7, 8, 9, 31, 32, 33, 40]
    rng = np.random.default_rng(0)
    for _ in range(40):
        M, N, K = (int(rng.choice(vals)) for _ in range(3))
        _check(oracle_mod, blas, M, N, K, 1.0, 1.0, seed=int(rng.integers(1, 1000)))
        _check(oracle_mod, blas, M, N, K, 1.0, 0.0, tile=4, seed=int(rng.integers(1, 1000)))


def test_exact_special_cases(blas):
    n = 192
    dev = "cuda"
    # identity: A @ I == A bit for bit, I @ B == B
    a = torch.rand(n, n, device=dev) * 2 - 1
    eye = torch.eye(n, device=dev)
    c = torch.empty(n, n, device=dev)
    blas.sgemm(n, n, n, a, eye, c, 1.0, 0.0)
    assert torch.equal(c, a)
    blas.sgemm(n, n, n, eye, a, c, 1.0, 0.0)
    assert torch.equal(c, a)
    # a permutation picks rows: transposed operands or a swapped k index would be caught
    perm = torch.randperm(n, device=dev)
    p = torch.zeros(n, n, device=dev)
    p[torch.arange(n, device=dev), perm] = 1.0
    blas.sgemm(n, n, n, p, a, c, 1.0, 0.0)
    assert torch.equal(c, a[perm])
    # all ones: C == K exactly (K <= 2^24), any accumulation order
    M, N, K = 96, 160, 4096
    c = torch.empty(M, N, device=dev)
    blas.sgemm(M, N, K, torch.ones(M, K, device=dev), torch.ones(K, N, device=dev), c, 1.0, 0.0)
    assert torch.all(c == float(K))
    # index-valued operands: C[i][j] = i * j * K, exact in FP32 for these sizes
    M, N, K = 70, 50, 16
    ai = torch.arange(M, device=dev, dtype=torch.float32)[:, None].expand(M, K).contiguous()
    bj = torch.arange(N, device=dev, dtype=torch.float32)[None, :].expand(K, N).contiguous()
    c = torch.empty(M, N, device=dev)
    blas.sgemm(M, N, K, ai, bj, c, 1.0, 0.0)
    assert torch.equal(c, (torch.arange(M, device=dev)[:, None] * torch.arange(N, device=dev)[None, :] * K).float())
    # alpha = 0, beta = 1 leaves C unchanged; K = 0 scales C by beta
    c0 = torch.rand(M, N, device=dev)
    c = c0.clone()
    blas.sgemm(M, N, K, ai, bj, c, 0.0, 1.0)
    assert torch.equal(c, c0)
    blas.sgemm(M, N, 0, ai[:, :0], bj[:0, :], c, 1.0, 0.5)
    assert torch.equal(c, c0 * 0.5)


def _sampled_check(oracle_mod, blas, M, N, K, alpha, beta, nrows=48, seed=300, tile=-1, split_k=0, ws=None):
    """Device-generated operands (same counters as the oracle), sampled-row FP64 check + Freivalds over all of C."""
    dev = "cuda"
    da = torch.empty(M, K, device=dev)
    db = torch.empty(K, N, device=dev)
    dc = torch.empty(M, N, device=dev)
    blas.fill_uniform_matrix(da, M, K, seed)
    blas.fill_uniform_matrix(db, K, N, seed + 1)
    blas.fill_uniform_matrix(dc, M, N, seed + 2)
    dc0 = dc.clone() if beta != 0.0 else None
    blas.sgemm(M, N, K, da, db, dc, alpha, beta, ws=ws, tile=tile, split_k=split_k)
    rng = np.random.default_rng(seed)
    rows = np.unique(np.concatenate([[0, M - 1], rng.integers(0, M, nrows)])).astype(np.int32)
    a = oracle_mod.fill_uniform_matrix(M, K, seed)
    b = oracle_mod.fill_uniform_matrix(K, N, seed + 1)
    c0 = oracle_mod.fill_uniform_matrix(M, N, seed + 2) if beta != 0.0 else None
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, K, b, N, c0, N, alpha, beta, rows=rows)
    c_rows = np.ascontiguousarray(dc[torch.from_numpy(rows).long().cuda()].cpu().numpy())
    err = oracle_mod.gemm_max_err(N, c_rows, N, ref, den)
    assert err <= TOL, (M, N, K, alpha, beta, err)
    # Freivalds in FP64 over the whole matrix: C v == alpha A (B v) + beta C0 v
    v = (torch.randint(0, 2, (N,), device=dev, dtype=torch.float64) * 2 - 1)
    lhs = dc.double() @ v
    rhs = alpha * (da.double() @ (db.double() @ v))
    bound = abs(alpha) * (da.double().abs() @ (db.double().abs() @ torch.ones(N, device=dev, dtype=torch.float64)))
    if beta != 0.0:
        rhs = rhs + beta * (dc0.double() @ v)
        bound = bound + abs(beta) * dc0.double().abs().sum(dim=1)
    assert torch.all((lhs - rhs).abs() <= TOL * bound), (M, N, K)
    return dc


@pytest.mark.parametrize("n,beta", [(1000, 0.0), (3001, 1.0), (2048, 1.0), (4096, 0.0)])
def test_square_sizes_from_the_sweep(blas, oracle_mod, n, beta):
    _sampled_check(oracle_mod, blas, n, n, n, 1.0, beta)


@pytest.mark.parametrize("n,beta", [(6000, 0.0), (6144, 0.0), (6144, 1.0)])
def test_largest_square_sizes(blas, oracle_mod, n, beta):
    _sampled_check(oracle_mod, blas, n, n, n, 1.0, beta, nrows=24)


@pytest.mark.parametrize("M,N,K", [(8192, 8192, 256), (16384, 64, 4096), (128, 128, 65536), (64, 64, 131072), (40, 52, 200000),
                                   (192, 192, 65536)])
def test_skinny_and_deep_shapes(blas, oracle_mod, M, N, K):
    ws = blas.workspace(max(blas.sgemm_workspace_bytes(M, N, K), 4))
    c1 = _sampled_check(oracle_mod, blas, M, N, K, 1.0, 0.0, nrows=16, ws=ws)
    c2 = _sampled_check(oracle_mod, blas, M, N, K, 1.0, 0.0, nrows=16, ws=ws)
    assert torch.equal(c1, c2)  # fixed-order split-K reduction: same bits on every run


def test_split_k_forced_matches_and_is_deterministic(blas, oracle_mod):
    M, N, K = 200, 136, 2000
    ws = blas.workspace(M * N * 8 * 4)
    outs = []
    for split in (1, 2, 5, 8):
        outs.append(_check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=1, split_k=split, ws=ws, ldc=144))
    again = _check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=1, split_k=8, ws=ws, ldc=144)
    assert np.array_equal(outs[-1][:, :N], again[:, :N])


@pytest.mark.parametrize("tile", [1, 4])
def test_split_k_slices_are_the_products_of_their_k_ranges(blas, tile):
    """Eight slices (a multiple of the XCD count: the launch hands whole K slices to each XCD): the result has the bits of
    the eight products over the K ranges, each computed by an unsplit call, added in slice order."""
    M, N, K, split = 200, 136, 2048, 8
    g = torch.Generator(device="cpu").manual_seed(77 + tile)
    a = (torch.rand(M, K, generator=g) * 2 - 1).cuda()
    b = (torch.rand(K, N, generator=g) * 2 - 1).cuda()
    ws = blas.workspace(M * N * split * 4)
    c = torch.full((M, N), 3.0, device="cuda")
    blas.sgemm(M, N, K, a, b, c, 1.0, 0.0, ws=ws, tile=tile, split_k=split)
    kc = K // split
    total = None
    for i in range(split):
        part = torch.empty(M, N, device="cuda")
        blas.sgemm(M, N, kc, a[:, i * kc:(i + 1) * kc], b[i * kc:(i + 1) * kc, :], part, 1.0, 0.0, tile=tile, split_k=1)
        total = part if total is None else total + part
    torch.cuda.synchronize()
    assert torch.equal(c, total)


@pytest.mark.parametrize("M,N,K,split", [(200, 136, 4200, 13), (200, 136, 4200, 32), (77, 132, 9000, 64), (200, 138, 4200, 16)])
def test_split_k_many_slices(blas, oracle_mod, M, N, K, split):
    """More than eight slices are added by the reduction whose lanes share the slices of a group of elements (N a
    multiple of 4; 138 columns take the other one): ragged element counts, beta != 0, padded ldc, same bits twice."""
    ws = blas.workspace(M * N * split * 4)
    first = _check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=4, split_k=split, ws=ws, ldc=N + 8)
    again = _check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=4, split_k=split, ws=ws, ldc=N + 8)
    assert np.array_equal(first[:, :N], again[:, :N])


def test_tail_split_forced_matches_and_is_deterministic(blas, oracle_mod):
    """Only the tiles left over after the last full round of CUs are split along K (split_k < -1)."""
    M, N, K = 1088, 1024, 520  # 64x64 tiles: 17 x 16 = 272 = 256 + 16 leftover tiles; ragged K
    ws = blas.workspace(16 * 8 * 64 * 64 * 4)
    outs = []
    for ways in (2, 3, 8):
        outs.append(_check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=4, split_k=-ways, ws=ws, ldc=N + 8))
    again = _check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=4, split_k=-8, ws=ws, ldc=N + 8)
    assert np.array_equal(outs[-1][:, :N], again[:, :N])
    # the full tiles do not depend on how the leftover ones are split
    plain = _check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=4, split_k=1, ldc=N + 8)
    same = (plain[:, :N] == outs[0][:, :N])
    assert same.mean() > 0.9
    # ragged M and N with a leftover round, and no leftover at all (falls back to a plain launch)
    _check(oracle_mod, blas, 1085, 1001, 300, 1.0, 0.0, tile=4, split_k=-2, ws=ws)
    _check(oracle_mod, blas, 1024, 1024, 256, 1.0, 0.0, tile=4, split_k=-4, ws=ws)
    with pytest.raises(blas.HpcdnnError):
        _check(oracle_mod, blas, M, N, K, 1.0, 0.0, tile=4, split_k=-8, ws=None)
    # tail split forced, tile left to the library: a shape whose unforced plan is the 32 x 32 tile (which has no tail
    # split) must get a tile that has one
    big = blas.workspace(64 << 20)
    assert blas.tile_table()[blas.sgemm_plan(256, 1056, 256, ws_bytes=64 << 20)[0]][:2] == (32, 32)
    _check(oracle_mod, blas, 256, 1056, 256, 1.0, 1.0, split_k=-2, ws=big)


def test_small_problem_tile_splits_k_between_its_waves(blas, oracle_mod):
    """The 32 x 32 tile: four waves share K block-wise and meet in LDS; picked where 64 x 64 tiles cannot fill the CUs."""
    small = [t for t, (bm, bn, _) in enumerate(blas.tile_table()) if (bm, bn) == (32, 32)]
    assert len(small) == 1
    tile = small[0]
    # fewer K blocks than waves, every kind of K tail inside a lane's 16-value run, ragged M and N, NaN padding
    for (M, N, K) in [(32, 32, 1), (32, 32, 31), (40, 50, 33), (64, 96, 64), (70, 45, 95), (33, 65, 129), (96, 32, 160),
                      (1, 1, 17), (128, 128, 1000), (31, 200, 48)]:
        _check(oracle_mod, blas, M, N, K, 1.0, 0.0, tile=tile, lda=K + 3, ldb=N + 5, ldc=N + 1, seed=300 + K)
    for alpha, beta in [(1.5, -1.0), (0.0, 2.0), (-0.5, 0.0), (1.0, 1.0)]:
        _check(oracle_mod, blas, 200, 150, 90, alpha, beta, tile=tile, lda=96, ldb=152, ldc=160)
    # K slices through the workspace on top of the split between the waves; fixed order, same bits every run
    M, N, K = 100, 90, 1000
    ws = blas.workspace(M * N * 4 * 4)
    for split in (2, 3, 4):
        c1 = _check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=tile, split_k=split, ws=ws, ldc=N + 6)
        c2 = _check(oracle_mod, blas, M, N, K, 1.5, -1.0, tile=tile, split_k=split, ws=ws, ldc=N + 6)
        assert np.array_equal(c1[:, :N], c2[:, :N])
    with pytest.raises(blas.HpcdnnError):  # no tail split for this tile
        _check(oracle_mod, blas, M, N, K, 1.0, 0.0, tile=tile, split_k=-2, ws=ws)
    # K = 0 scales C; exact cases: ones (any summation order), identity
    n = 96
    c0 = torch.rand(n, n, device="cuda")
    c = c0.clone()
    blas.sgemm(n, n, 0, c0[:, :0], c0[:0, :], c, 1.0, 0.5, tile=tile)
    assert torch.equal(c, c0 * 0.5)
    a = torch.rand(n, n, device="cuda") * 2 - 1
    c = torch.empty(n, n, device="cuda")
    blas.sgemm(n, n, n, a, torch.eye(n, device="cuda"), c, 1.0, 0.0, tile=tile)
    assert torch.equal(c, a)
    blas.sgemm(n, n, 4096, torch.ones(n, 4096, device="cuda"), torch.ones(4096, n, device="cuda"), c, 1.0, 0.0, tile=tile)
    assert torch.all(c == 4096.0)
    # the selector: small squares and thin deep shapes without a workspace, never the large squares
    for shape in [(256, 256, 256), (512, 512, 512), (512, 512, 4096)]:
        assert blas.sgemm_plan(*shape, 0)[0] == tile
        c1 = _check(oracle_mod, blas, *shape, 1.0, 0.0)
        c2 = _check(oracle_mod, blas, *shape, 1.0, 0.0)
        assert np.array_equal(c1, c2)
    for shape in [(1024, 1024, 1024), (2048, 2048, 2048), (6144, 6144, 6144)]:
        assert blas.sgemm_plan(*shape, 0)[0] != tile


def test_deep_prefetch_tile_every_k_remainder(blas, oracle_mod):
    """The 64 x 64 tile that keeps four K steps in flight: its loop runs in groups of four steps plus a remainder."""
    table = blas.tile_table()
    tiles = [t for t, shape in enumerate(table) if shape[:2] == (64, 64)]
    assert len(tiles) == 2
    deep = tiles[1]
    for steps in range(1, 12):
        for extra in (0, 5):
            K = 16 * steps + extra
            _check(oracle_mod, blas, 128, 64, K, 1.0, 0.0, tile=deep, seed=400 + K)                       # full tiles
            _check(oracle_mod, blas, 100, 70, K, 1.5, -1.0, tile=deep, lda=K + 3, ldb=75, ldc=72, seed=500 + K)  # ragged
    # same summation order as the other large tiles: same bits as the two-slot 64 x 64 tile
    a = _check(oracle_mod, blas, 192, 128, 1000, 1.0, 0.0, tile=tiles[0])
    b = _check(oracle_mod, blas, 192, 128, 1000, 1.0, 0.0, tile=deep)
    assert np.array_equal(a, b)
    ws = blas.workspace(192 * 128 * 4 * 4)
    _check(oracle_mod, blas, 192, 128, 1000, 1.0, 1.0, tile=deep, split_k=3, ws=ws)
    # picked for a long operand that is read once with one workgroup per CU
    assert blas.sgemm_plan(16384, 64, 4096, 0)[0] == deep
    _sampled_check(oracle_mod, blas, 16384, 64, 4096, 1.0, 0.0, nrows=16)


def test_plan_is_a_function_of_the_shape_and_runs(blas, oracle_mod):
    for shape in [(3072, 3072, 3072), (5120, 5120, 1024), (4352, 4352, 4352)]:
        need = blas.sgemm_workspace_bytes(*shape)
        plan = blas.sgemm_plan(*shape, need)
        assert plan == blas.sgemm_plan(*shape, need)
        assert blas.sgemm_plan(*shape, 0)[1] == 1  # no workspace, no split of any kind
        ws = blas.workspace(max(need, 4))
        _sampled_check(oracle_mod, blas, *shape, 1.0, 1.0, nrows=12, ws=ws)


SWEEP = list(range(256, 6145, 256)) + [1000, 3001, 6000]


@pytest.mark.parametrize("n", SWEEP)
def test_config3_square_sweep_every_size(blas, oracle_mod, n):
    """Every size of the square sweep (256..6144 step 256, plus 1000, 3001, 6000): beta = 0 with the optional
    workspace (whatever split the library picks), beta = 1 without."""
    ws = blas.workspace(max(blas.sgemm_workspace_bytes(n, n, n), 4))
    _sampled_check(oracle_mod, blas, n, n, n, 1.0, 0.0, nrows=6, seed=900 + n, ws=ws)
    _sampled_check(oracle_mod, blas, n, n, n, 1.0, 1.0, nrows=6, seed=901 + n)


def test_operands_larger_than_4_gib(blas):
    """A of 5.3 GB and C of 5.3 GB in two shapes: row offsets past 2^32 bytes in A, in C and in the split-K
    workspace.  Checked with FP64 products of sampled rows and a Freivalds identity formed on the device."""
    dev = "cuda"
    for (M, N, K) in [(33000, 200, 40000), (40000, 33000, 96)]:
        a = torch.empty(M, K, device=dev)
        b = torch.empty(K, N, device=dev)
        c = torch.empty(M, N, device=dev)
        blas.fill_uniform_matrix(a, M, K, 71)
        blas.fill_uniform_matrix(b, K, N, 72)
        ws = blas.workspace(max(blas.sgemm_workspace_bytes(M, N, K), 4))
        blas.sgemm(M, N, K, a, b, c, 1.0, 0.0, ws=ws)
        rows = torch.tensor([0, 1, M // 2, M - 300, M - 2, M - 1], device=dev)
        ref = a[rows].double() @ b.double()
        den = a[rows].double().abs() @ b.double().abs()
        assert torch.all((c[rows].double() - ref).abs() <= TOL * den), (M, N, K)
        v = torch.randint(0, 2, (N,), device=dev, dtype=torch.float64) * 2 - 1
        bv = b.double() @ v
        babs = b.double().abs().sum(dim=1)
        for s in range(0, M, 8192):
            e = min(M, s + 8192)
            lhs = c[s:e].double() @ v
            rhs = a[s:e].double() @ bv
            bound = a[s:e].double().abs() @ babs
            assert torch.all((lhs - rhs).abs() <= TOL * bound), (M, N, K, s)
        del a, b, c, ws


def test_row_split_gives_the_same_bits_as_one_launch(blas, oracle_mod):
    """Sizes where the library covers C with two launches (no workspace): same bits as one launch of the first
    launch's tile, because every element still sums K in one workgroup and in the same order."""
    found = 0
    for n in (3584, 4608, 5120):
        rows, t1, t2 = blas.sgemm_row_split(n, n, n, 0)
        if rows == 0:
            continue
        found += 1
        assert 0 < rows < n and t1 >= 0 and t2 >= 0
        c_auto = _sampled_check(oracle_mod, blas, n, n, n, 1.0, 1.0, nrows=6, seed=950 + n)
        c_one = _sampled_check(oracle_mod, blas, n, n, n, 1.0, 1.0, nrows=6, seed=950 + n, tile=t1, split_k=1)
        assert torch.equal(c_auto, c_one), n
    assert found >= 1


@pytest.mark.parametrize("M,N,K,tile", [(2176, 4608, 320, 7), (4352, 2304, 192, 0), (4096, 4096, 160, 7), (4096, 2048, 256, 0),
                                        (3264, 4608, 320, 5), (3072, 4096, 512, 5), (2176, 4608, 320, 1), (4096, 4096, 160, 1)])
@pytest.mark.parametrize("alpha,beta", [(1.5, 0.0), (1.0, -1.5)])
def test_persistent_kernel_on_several_rounds_of_whole_tiles(blas, oracle_mod, M, N, K, tile, alpha, beta):
    """More tiles than CUs, every tile whole, an even number (>= 10) of K steps: the 256x128 and 128x256 tiles run as
    one persistent workgroup per CU that stores a finished tile while it multiplies the next.  Checked against the
    FP64 criterion (sampled rows + Freivalds over all of C), for the same bits as the 128x64 tile-per-workgroup
    kernel, with a padded ldc whose padding stays untouched, and with NaN in C when beta == 0.  306 tiles leave a
    partial last round, 512 tiles give every workgroup two, 256 tiles (one round) take the ordinary kernel.  The 192x256
    tile stores a third of a finished tile at the tile boundary and has no beta != 0 variant (the ordinary kernel runs).
    The 128x128 tile runs two persistent workgroups per CU, so it takes more than 512 tiles."""
    _sampled_check(oracle_mod, blas, M, N, K, alpha, beta, nrows=12, seed=700 + tile, tile=tile, split_k=1)
    dev = "cuda"
    ldc = N + 24
    da, db = torch.empty(M, K, device=dev), torch.empty(K, N, device=dev)
    blas.fill_uniform_matrix(da, M, K, 31)
    blas.fill_uniform_matrix(db, K, N, 32)
    c0 = torch.full((M, ldc), float("nan"), device=dev)
    if beta != 0.0:
        c0[:, :N] = torch.rand(M, N, device=dev) * 2 - 1
    c1, c2 = c0.clone(), c0.clone()
    blas.sgemm(M, N, K, da, db, c1, alpha, beta, tile=tile, split_k=1)  # ldc = the row stride of c1
    blas.sgemm(M, N, K, da, db, c2, alpha, beta, tile=2, split_k=1)
    assert torch.equal(c1[:, :N], c2[:, :N])
    assert not torch.isnan(c1[:, :N]).any()
    assert torch.isnan(c1[:, N:]).all()


def test_seeded_random_shapes_every_path(blas, oracle_mod):
    """Seeded random (M, N, K, leading dimensions, alpha, beta) with and without workspace, so that whatever the
    selector picks for them (tile, split-K, tail split, row split, ragged kernels) is checked on every element."""
    rng = np.random.default_rng(2025)
    seen = set()
    for case in range(48):
        M, N = int(rng.integers(1, 1400)), int(rng.integers(1, 1400))
        K = int(rng.choice([1, 7, 16, 100, 257, 1024, 3000, 9000]))
        if case % 6 == 0:   # shapes with many tiles, where the splits come into play
            M, N, K = int(rng.integers(2000, 2600)), int(rng.integers(2000, 2600)), int(rng.choice([512, 1040]))
        lda, ldb, ldc = K + int(rng.integers(0, 9)), N + int(rng.integers(0, 9)), N + int(rng.integers(0, 9))
        alpha = float(rng.choice([1.0, -0.5, 2.0]))
        beta = float(rng.choice([0.0, 1.0, -1.5]))
        use_ws = bool(case % 2)
        need = blas.sgemm_workspace_bytes(M, N, K)
        ws = blas.workspace(max(need, 4)) if use_ws else None
        plan = blas.sgemm_plan(M, N, K, need if use_ws else 0)
        rows = blas.sgemm_row_split(M, N, K, need if use_ws else 0)[0]
        seen.add(("rows" if rows else "split" if plan[1] > 1 else "tail" if plan[1] < -1 else "plain"))
        _check(oracle_mod, blas, M, N, K, alpha, beta, lda=lda, ldb=ldb, ldc=ldc, ws=ws, seed=3000 + case)
    assert {"plain", "split"} <= seen, seen


def test_host_threads_on_their_own_streams(blas, oracle_mod):
    """Four host threads, each on its own stream with its own shapes and workspace: the library keeps no state that
    they could trample (the plan memo is per thread), so every result has the bits of the serial run."""
    import threading
    shapes = [(512, 512, 512), (1024, 1024, 1024), (700, 900, 300), (128, 128, 8192), (2048, 2048, 512), (1536, 1536, 1536)]
    ops = {}
    for i, (M, N, K) in enumerate(shapes):
        a = torch.empty(M, K, device="cuda"); b = torch.empty(K, N, device="cuda")
        blas.fill_uniform_matrix(a, M, K, 900 + i); blas.fill_uniform_matrix(b, K, N, 950 + i)
        ws = blas.workspace(max(blas.sgemm_workspace_bytes(M, N, K), 16))
        ref = torch.empty(M, N, device="cuda")
        blas.sgemm(M, N, K, a, b, ref, 1.0, 0.0, ws=ws)
        ops[(M, N, K)] = (a, b, ref)
    torch.cuda.synchronize()
    errors = []

    def work(tid):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for rep in range(6):
                    M, N, K = shapes[(tid + rep) % len(shapes)]
                    a, b, ref = ops[(M, N, K)]
                    ws = blas.workspace(max(blas.sgemm_workspace_bytes(M, N, K), 16))   # own scratch: slices would race
                    c = torch.empty(M, N, device="cuda")
                    blas.sgemm(M, N, K, a, b, c, 1.0, 0.0, ws=ws)
                    stream.synchronize()
                    if not torch.equal(c, ref):
                        errors.append((tid, rep, M, N, K))
        except Exception as e:  # surfaced below: an assert in a thread would be lost
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_maximum_leading_dimensions(blas):
    """lda, ldb and ldc at the documented limits (32-bit byte offsets inside one tile), for every kernel family; one
    more is refused."""
    lda, ldb, ldc = (1 << 21) - 64, (1 << 25) - 1024, (1 << 21) - 64
    M, N, K = 300, 100, 40
    abuf = torch.empty(M * lda, device="cuda")
    bbuf = torch.empty(K * ldb + 8, device="cuda")
    a, b = abuf.view(M, lda)[:, :K], bbuf[:K * ldb].view(K, ldb)[:, :N]
    gen = torch.Generator(device="cuda").manual_seed(3)
    a.copy_(torch.rand(M, K, device="cuda", generator=gen) * 2 - 1)
    b.copy_(torch.rand(K, N, device="cuda", generator=gen) * 2 - 1)
    ref = a.double() @ b.double()
    den = a.abs().double() @ b.abs().double()
    small = [t for t, shape in enumerate(blas.tile_table()) if shape[:2] == (32, 32)][0]
    cbuf = torch.empty(M * ldc, device="cuda")
    c = cbuf.view(M, ldc)[:, :N]
    c0 = torch.rand(M, N, device="cuda", generator=gen) * 2 - 1
    for tile in (-1, 0, 4, 8, small, len(blas.tile_table()) - 1):
        for beta in (0.0, -1.5):
            c.copy_(c0)
            blas.sgemm(M, N, K, a, b, c, 1.0, beta, tile=tile, split_k=0 if tile < 0 else 1)
            assert float(((c.double() - ref - beta * c0.double()).abs() / (den + abs(beta) * c0.abs().double())).max()) <= TOL, (tile, beta)
    with pytest.raises(blas.HpcdnnError):
        blas.sgemm(8, N, K, a, b, cbuf[:7 * (ldc + 1) + N].as_strided((8, N), (ldc + 1, 1)), 1.0, 0.0)
    with pytest.raises(blas.HpcdnnError):
        blas.sgemm(M, N, K, a, bbuf[:(K - 1) * (ldb + 1) + N].as_strided((K, N), (ldb + 1, 1)), torch.zeros(M, N, device="cuda"), 1.0, 0.0)
    with pytest.raises(blas.HpcdnnError):
        blas.sgemm(8, N, K, abuf[:7 * (lda + 1) + K].as_strided((8, K), (lda + 1, 1)), b, torch.zeros(8, N, device="cuda"), 1.0, 0.0)
