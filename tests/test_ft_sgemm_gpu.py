"""GPU parity of the ABFT SGEMM against the CPU model of the reference's checksum logic, in both of its modes:
checksum vectors formed inside the main loop (no workspace) and by the pre-pass kernels (with workspace).

Values: same 1e-5 componentwise criterion as plain SGEMM (after correction).  Decisions (flag, located row and
column, number of flagged lines) must equal the CPU model's exactly on the same seeded faults.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-5
DECISION_FIELDS = ("flag", "row", "col", "n_bad_rows", "n_bad_cols")


@pytest.fixture(params=["fused", "workspace"])
def ft_mode(request):
    return request.param


def _ws(blas, mode, M, N, K):
    if mode == "fused":
        return None
    nbytes = blas.ft_workspace_bytes(M, N, K)
    # the checksum vectors of the class with the most tile rows, plus room for the K slices of a partial last round
    assert nbytes >= 4 * (-(-M // 64) + -(-N // 128)) * ((-(-K // 16) + 2) * 16)
    # poisoned: the library must not rely on the workspace's previous contents
    return torch.full((max(nbytes // 4, 4),), float("nan"), dtype=torch.float32, device="cuda")


def _run(blas, oracle_mod, mode, M, N, K, alpha, beta, tau, fault, seed=400, lda=None, ldb=None, ldc=None):
    lda, ldb, ldc = lda or K, ldb or N, ldc or N
    a = oracle_mod.fill_uniform_matrix(M, K, seed, ld=lda)
    b = oracle_mod.fill_uniform_matrix(K, N, seed + 1, ld=ldb)
    c0 = oracle_mod.fill_uniform_matrix(M, N, seed + 2, ld=ldc)
    da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
    status = blas.ft_status_alloc(M, N)
    blas.ft_sgemm(M, N, K, da, db, dc, alpha, beta, tau=tau, fault=fault, status=status, ws=_ws(blas, mode, M, N, K))
    st = blas.ft_status_numpy(status)
    c = dc.cpu().numpy()
    # model: a, b with zeroed padding so that the model never multiplies NaN padding (it indexes with ld too)
    c_model = c0.copy()
    st_model = oracle_mod.ft_sgemm(M, N, K, a, lda, b, ldb, c_model, ldc, alpha, beta, blas.FT_TILE_M, blas.FT_TILE_N,
                                   tau, fault)
    return a, b, c0, c, st, c_model, st_model


def _assert_values(oracle_mod, M, N, K, a, b, c0, c, alpha, beta):
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, a.shape[1], b, b.shape[1], c0, c0.shape[1], alpha, beta)
    err = oracle_mod.gemm_max_err(N, c, c.shape[1], ref, den)
    assert err <= TOL, err
    assert np.all(np.isnan(c[:, N:]))


@pytest.mark.parametrize("M,N,K", [(256, 128, 64), (512, 384, 320), (300, 200, 100), (1, 1, 1), (257, 129, 17), (1024, 1024, 1024), (256, 256, 16384)])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (1.0, -1.5)])
def test_fault_free_matches_model_and_oracle(blas, oracle_mod, ft_mode, M, N, K, alpha, beta):
    tau = blas.ft_default_tau(K)
    a, b, c0, c, st, c_model, st_model = _run(blas, oracle_mod, ft_mode, M, N, K, alpha, beta, tau, None)
    _assert_values(oracle_mod, M, N, K, a, b, c0, c, alpha, beta)
    for f in DECISION_FIELDS:
        assert np.array_equal(st[f], st_model[f]), f
    assert np.all(st["flag"] == 0) and np.all(st["row"] == -1) and np.all(st["col"] == -1)
    # fault-free residuals are rounding noise, far below the threshold
    assert st["max_clean_residual"].max() < 0.6 * tau


def test_reference_known_answer_plus_one_at_0_1(blas, oracle_mod, ft_mode):
    """The reference's only fault experiment: +1.0 into local element (m=0, n=1) of a tile, threshold 0.1
    (ft_sgemm_huge.cuh:30,40,145) -> row 0 / column 1 located, 1.0 removed."""
    M, N, K = 512, 256, 256
    for tile in range(4):
        a, b, c0, c, st, c_model, st_model = _run(blas, oracle_mod, ft_mode, M, N, K, 1.0, 0.0, 0.1, (tile, 0, 1, 1.0))
        exp = [0, 0, 0, 0]
        exp[tile] = 1
        assert st["flag"].tolist() == exp
        assert (st["row"][tile], st["col"][tile]) == (0, 1)
        assert round(-float(st["row_residual"][tile])) == 1 and abs(st["row_residual"][tile] + 1.0) < 1e-3
        assert abs(st["col_residual"][tile] + 1.0) < 1e-3
        _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 0.0)


def test_seeded_faults_decisions_equal_cpu_model(blas, oracle_mod, ft_mode):
    # ragged problem: 3 x 3 tiles, last row/column of tiles clipped; padded leading dimensions
    M, N, K = 600, 300, 512
    tau = blas.ft_default_tau(K)
    rng = np.random.default_rng(7)
    ntiles = blas.ft_num_tiles(M, N)
    assert ntiles == 9
    for trial in range(24):
        tile = int(rng.integers(ntiles))
        tm = min(blas.FT_TILE_M, M - (tile // 3) * blas.FT_TILE_M)
        tn = min(blas.FT_TILE_N, N - (tile % 3) * blas.FT_TILE_N)
        i, j = int(rng.integers(tm)), int(rng.integers(tn))
        delta = float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-2, 2)))
        fault = (tile, i, j, delta)
        a, b, c0, c, st, c_model, st_model = _run(blas, oracle_mod, ft_mode, M, N, K, 1.0, 1.0, tau, fault,
                                                  seed=500 + trial, lda=K + 4, ldb=N + 4, ldc=N + 8)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (fault, f, st[f], st_model[f])
        assert st["flag"][tile] == 1 and (st["row"][tile], st["col"][tile]) == (i, j), fault
        assert abs(st["row_residual"][tile] + delta) < 2e-3 and abs(st["col_residual"][tile] + delta) < 2e-3
        assert np.allclose(st["row_residual"], st_model["row_residual"], atol=2e-3)
        _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 1.0)


def test_fault_below_threshold_or_outside_matrix_is_not_flagged(blas, oracle_mod, ft_mode):
    M, N, K = 300, 200, 256
    tau = blas.ft_default_tau(K)
    # far below the threshold: stays in C (documented behaviour), nothing flagged
    a, b, c0, c, st, c_model, st_model = _run(blas, oracle_mod, ft_mode, M, N, K, 1.0, 0.0, tau, (0, 3, 5, tau * 0.1))
    assert np.all(st["flag"] == 0) and np.array_equal(st["flag"], st_model["flag"])
    # a fault aimed at a clipped-away element of an edge tile lands in zero padding that is never stored:
    # it is detected and removed by both the device and the model, or ignored by both
    a, b, c0, c, st, c_model, st_model = _run(blas, oracle_mod, ft_mode, M, N, K, 1.0, 0.0, tau, (3, 200, 100, 5.0))
    _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 0.0)
    for f in DECISION_FIELDS:
        assert np.array_equal(st[f], st_model[f]), f
    assert np.all(st["flag"] == 0)   # a fault aimed outside the matrix is ignored by the device and by the model


def test_many_flagged_lines_are_reported_uncorrectable(blas, oracle_mod, ft_mode):
    """More than one faulty row or column cannot be located by row x column intersection: a threshold below the
    rounding noise flags many lines, and the kernel must report flag 2 and leave the accumulators alone."""
    M, N, K = 256, 128, 512
    a, b, c0, c, st, c_model, st_model = _run(blas, oracle_mod, ft_mode, M, N, K, 1.0, 0.0, 1e-9, None)
    assert st["flag"][0] == 2 and st["n_bad_rows"][0] > 1 and st["n_bad_cols"][0] > 1
    assert (st["row"][0], st["col"][0]) == (-1, -1)
    _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 0.0)


class _TileModel:
    """CPU model of one 256x128 tile at full K, cached so that each further fault on the tile costs O(tile)."""

    def __init__(self, oracle_mod, a, b, K, N, tile, tm, tn, ntn):
        m0, n0 = (tile // ntn) * tm, (tile % ntn) * tn
        at, bt = a[m0:m0 + tm], b[:, n0:n0 + tn]
        self.acc = oracle_mod.tile_acc(at, K, bt, N, tm, tn, K)
        self.cr, self.cc = oracle_mod.abft_reference_checksums(at, K, bt, N, tm, tn, K)
        self.oracle = oracle_mod

    def decide(self, i, j, delta, tau):
        acc = self.acc.copy()
        acc[i, j] += np.float32(delta)
        dr, dc = self.oracle.abft_observe(acc, acc.shape[1], self.cr, self.cc)
        return self.oracle.abft_decide(dr, dc, tau)


def test_config4_4096_cube_seeded_fault_campaign(blas, oracle_mod, ft_mode):
    """The 4096-cube fault campaign: M=N=K=4096, alpha=1, beta=0, one seeded fault (tile, i, j, magnitude in [1e-2, 1e2],
    random sign) per launch.  Every launch: detected, located at the injected element, corrected, no other tile
    flagged; decisions equal the CPU model's for every launch (the model is evaluated on the faulted tile)."""
    M = N = K = 4096
    launches = 1000
    dev = "cuda"
    da, db = torch.empty(M, K, device=dev), torch.empty(K, N, device=dev)
    dc = torch.zeros(M, N, device=dev)
    blas.fill_uniform_matrix(da, M, K, 20)
    blas.fill_uniform_matrix(db, K, N, 21)
    a = oracle_mod.fill_uniform_matrix(M, K, 20)
    b = oracle_mod.fill_uniform_matrix(K, N, 21)
    tau = blas.ft_default_tau(K)
    status = blas.ft_status_alloc(M, N)
    ws = _ws(blas, ft_mode, M, N, K)
    ntiles, ntn = blas.ft_num_tiles(M, N), N // blas.FT_TILE_N
    assert ntiles == 512

    blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=tau, status=status, ws=ws)
    clean = blas.ft_status_numpy(status)
    assert np.count_nonzero(clean["flag"]) == 0          # no false positives on the fault-free run
    assert clean["max_clean_residual"].max() < 0.6 * tau
    c_clean = dc.clone()
    plain = torch.zeros(M, N, device=dev)
    blas.sgemm(M, N, K, da, db, plain, 1.0, 0.0, tile=0, split_k=1)
    assert torch.equal(plain, c_clean)                   # fault-free ABFT output is bit-identical to plain SGEMM

    rng = np.random.default_rng(2024)
    models = {}
    for launch in range(launches):
        tile = int(rng.integers(ntiles))
        i, j = int(rng.integers(blas.FT_TILE_M)), int(rng.integers(blas.FT_TILE_N))
        delta = float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-2, 2)))
        blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=tau, fault=(tile, i, j, delta), status=status, ws=ws)
        st = blas.ft_status_numpy(status)
        assert st["flag"][tile] == 1, (launch, tile, i, j, delta, st[tile])
        assert (st["row"][tile], st["col"][tile]) == (i, j), (launch, tile, i, j, delta, st[tile])
        assert np.count_nonzero(st["flag"]) == 1, (launch, "false positive elsewhere")
        # the located accumulator is computed again in the matrix cores' own order: bit-identical to the fault-free run
        assert torch.equal(dc, c_clean), (launch, tile, i, j, delta, float((dc - c_clean).abs().max()))
        if tile not in models:
            models[tile] = _TileModel(oracle_mod, a, b, K, N, tile, blas.FT_TILE_M, blas.FT_TILE_N, ntn)
        st_model, fix_model = models[tile].decide(i, j, delta, tau)
        for f in DECISION_FIELDS:
            assert st[f][tile] == st_model[f], (launch, f, st[tile], st_model)
        assert abs(float(st["row_residual"][tile]) - fix_model) < 3e-3
    print(f"campaign ({ft_mode}): {launches} launches, every corrected C bit-identical to the fault-free one, "
          f"fault-free max residual {clean['max_clean_residual'].max():.3e}, tau {tau:.1e}")


@pytest.mark.parametrize("tile_class", [1, 2, 3, 4])
def test_smaller_tile_classes_match_the_model(blas, oracle_mod, ft_mode, tile_class):
    """The 128x128 and 64x128 ABFT tiles: tiles, status records and fault coordinates are per tile of the class."""
    bm, bn = blas.ft_tile(tile_class)
    assert (bm, bn) == {1: (128, 128), 2: (64, 128), 3: (128, 64), 4: (64, 64)}[tile_class]
    M, N, K = 333, 300, 520  # ragged in every dimension
    tau = blas.ft_default_tau(K)
    ntm, ntn = -(-M // bm), -(-N // bn)
    assert blas.ft_num_tiles(M, N, tile_class) == ntm * ntn
    rng = np.random.default_rng(40 + tile_class)
    for trial in range(8):
        a = oracle_mod.fill_uniform_matrix(M, K, 600 + trial, ld=K + 4)
        b = oracle_mod.fill_uniform_matrix(K, N, 700 + trial, ld=N + 4)
        c0 = oracle_mod.fill_uniform_matrix(M, N, 800 + trial, ld=N + 8)
        fault = None
        if trial:
            tile = int(rng.integers(ntm * ntn))
            tm = min(bm, M - (tile // ntn) * bm)
            tn = min(bn, N - (tile % ntn) * bn)
            fault = (tile, int(rng.integers(tm)), int(rng.integers(tn)),
                     float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-2, 2))))
        da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
        status = blas.ft_status_alloc(M, N, tile_class=tile_class)
        blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 1.0, tau=tau, fault=fault, status=status, ws=_ws(blas, ft_mode, M, N, K),
                      tile_class=tile_class)
        st = blas.ft_status_numpy(status)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 1.0, bm, bn, tau, fault)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (tile_class, fault, f, st[f], st_model[f])
        if fault is not None:
            assert st["flag"][fault[0]] == 1 and (st["row"][fault[0]], st["col"][fault[0]]) == fault[1:3]
        _assert_values(oracle_mod, M, N, K, a, b, c0, dc.cpu().numpy(), 1.0, 1.0)


def test_pick_class_and_bad_class(blas):
    assert blas.ft_pick_class(4096, 4096, 4096) == 0      # 512 tiles of 256x128: every CU has one
    assert blas.ft_pick_class(2048, 2048, 1024) == 1      # 128 tiles of 256x128, 256 of 128x128
    assert blas.ft_pick_class(512, 512, 512) == 4         # 64 tiles of 64x64 against 32 of 64x128
    assert blas.ft_pick_class(3072, 3072, 3072) in (0, 1)  # either class ends its partial round with a K split
    assert blas.ft_pick_class(3072, 3072, 128) in (2, 4)  # too short a K to split: small tiles fill the rounds best
    assert blas.ft_pick_class(16384, 64, 4096) == 3       # 64 columns: the 128-column classes would multiply empty ones
    # without a workspace no round can end in a K split, and the vectors formed in the loop cost the small tiles more
    assert blas.ft_pick_class(4096, 4096, 4096, ws_bytes=0) == 0
    assert blas.ft_pick_class(3072, 3072, 3072, ws_bytes=0) == 2   # 4.5 rounds of 64x128 against 2.25 of 128x128
    assert blas.ft_pick_class(2560, 2560, 2560, ws_bytes=0) == 0   # 200 tiles of 256x128: one round
    assert blas.ft_pick_class(1536, 1536, 1536, ws_bytes=0) == 4
    assert blas.ft_pick_class(2048, 2048, 1024, ws_bytes=0) == 1
    assert blas.ft_pick_class(16384, 64, 4096, ws_bytes=0) == 4    # 256 tiles of 64x64, none split
    for shape in [(4096, 4096, 4096), (3072, 3072, 3072), (16384, 64, 4096), (1000, 1000, 1000)]:
        assert blas.ft_pick_class(*shape, ws_bytes=blas.ft_workspace_bytes(*shape)) == blas.ft_pick_class(*shape)
    t = torch.zeros(64, 64, device="cuda")
    with pytest.raises(blas.HpcdnnError):
        blas.ft_sgemm(64, 64, 64, t, t, t.clone(), 1.0, 0.0, tile_class=5)


def test_k_zero_scales_c_and_flags_nothing(blas, ft_mode):
    M, N = 300, 200
    c0 = torch.rand(M, N, device="cuda")
    c = c0.clone()
    a = torch.zeros(M, 1, device="cuda")
    b = torch.zeros(1, N, device="cuda")
    status = blas.ft_status_alloc(M, N)
    ws = None if ft_mode == "fused" else torch.zeros(64, device="cuda")
    blas.ft_sgemm(M, N, 0, a[:, :0], b[:0, :], c, 1.0, 0.5, status=status, ws=ws)
    assert torch.equal(c, c0 * 0.5)
    st = blas.ft_status_numpy(status)
    assert np.all(st["flag"] == 0) and np.all(st["max_clean_residual"] == 0.0)
    # wave-tile granularity has more records than workgroup tiles: every one of them must come back clean, whatever
    # the buffer held before
    for cls in (0, 1, 2):
        n = blas.ft_num_check_tiles(M, N, cls, blas.FT_GRAN_WAVE)
        status = blas.ft_status_alloc(M, N, tile_class=cls, granularity=blas.FT_GRAN_WAVE)
        assert status.numel() * status.element_size() == 32 * n
        status.view(torch.int32).fill_(0x7fc00001)   # stale: flag, row, col and the residuals all garbage
        c = c0.clone()
        blas.ft_sgemm(M, N, 0, a[:, :0], b[:0, :], c, 1.0, 0.5, status=status, ws=torch.zeros(64, device="cuda"),
                      tile_class=cls, granularity=blas.FT_GRAN_WAVE, faults=[(0, 1, 1, 3.0, 0)])
        assert torch.equal(c, c0 * 0.5)
        st = blas.ft_status_numpy(status)
        assert st.shape == (n,) and np.all(st["flag"] == 0) and np.all(st["row"] == -1) and np.all(st["col"] == -1)
        assert np.all(st["n_bad_rows"] == 0) and np.all(st["n_bad_cols"] == 0) and np.all(st["max_clean_residual"] == 0.0)


def test_default_threshold_follows_the_data(blas, oracle_mod, ft_mode):
    """tau = 0, the default, is the data-scaled threshold: on operands that are neither unit-range nor zero-mean
    (x 100 + 25) a fault-free product flags nothing, a fault of 1e-3 of the typical entry is found, and the decisions
    are those of tau = -1 and of the CPU model."""
    M, N, K = 512, 384, 1024
    a = oracle_mod.fill_uniform_matrix(M, K, 920) * np.float32(100.0) + np.float32(25.0)
    b = oracle_mod.fill_uniform_matrix(K, N, 921) * np.float32(100.0) + np.float32(25.0)
    c0 = np.zeros((M, N), np.float32)
    typical = float(np.abs(a[:64].astype(np.float64) @ b.astype(np.float64)).mean())
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    for fault in (None, (3, 100, 50, 1e-3 * typical), (2, 255, 127, -1e-3 * typical)):
        results = []
        for tau in (0.0, -1.0):
            dc = torch.from_numpy(c0).cuda()
            status = blas.ft_status_alloc(M, N)
            blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=tau, fault=fault, status=status, ws=_ws(blas, ft_mode, M, N, K))
            results.append((blas.ft_status_numpy(status), dc.cpu().numpy()))
        (st, c), (st1, c1) = results
        assert np.array_equal(st, st1) and np.array_equal(c, c1)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm(M, N, K, a, K, b, N, c_model, N, 1.0, 0.0, blas.FT_TILE_M, blas.FT_TILE_N, 0.0, fault)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (fault, f, st[f], st_model[f])
        if fault is None:
            assert np.all(st["flag"] == 0)
            # the constant calibrated for unit-range operands does flag this fault-free product
            dc = torch.from_numpy(c0).cuda()
            status = blas.ft_status_alloc(M, N)
            blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=blas.ft_default_tau(K), status=status, ws=_ws(blas, ft_mode, M, N, K))
            assert np.count_nonzero(blas.ft_status_numpy(status)["flag"]) > 0
        else:
            assert st["flag"][fault[0]] == 1 and (st["row"][fault[0]], st["col"][fault[0]]) == fault[1:3]
            assert np.count_nonzero(st["flag"]) == 1
        _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 0.0)


@pytest.mark.parametrize("scale_a,scale_b,shift", [(1.0, 1.0, 0.0), (250.0, 0.004, 0.0), (1e-3, 1e-3, 0.0), (1.0, 1.0, 0.5)])
def test_data_scaled_threshold(blas, oracle_mod, ft_mode, scale_a, scale_b, shift):
    """tau < 0: thresholds follow the magnitude of the accumulators, so the same call works for operands of any scale
    and for operands with a non-zero mean (where the absolute default for unit data would flag rounding noise or miss
    small faults).  Decisions equal the CPU model's; a fault of 2e-3 of the typical |C| entry is found."""
    M, N, K = 512, 384, 1024
    a = (oracle_mod.fill_uniform_matrix(M, K, 910) + np.float32(shift)) * np.float32(scale_a)
    b = (oracle_mod.fill_uniform_matrix(K, N, 911) + np.float32(shift)) * np.float32(scale_b)
    c0 = np.zeros((M, N), np.float32)
    typical = float(np.abs(a[:64].astype(np.float64) @ b.astype(np.float64)).mean())
    for fault in (None, (3, 100, 50, 2e-3 * typical * 40), (1, 7, 9, -2e-3 * typical * 40)):
        da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
        status = blas.ft_status_alloc(M, N)
        blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=-1.0, fault=fault, status=status, ws=_ws(blas, ft_mode, M, N, K))
        st = blas.ft_status_numpy(status)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm(M, N, K, a, K, b, N, c_model, N, 1.0, 0.0, blas.FT_TILE_M, blas.FT_TILE_N, -1.0, fault)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (scale_a, shift, fault, f, st[f], st_model[f])
        if fault is None:
            assert np.all(st["flag"] == 0)
        else:
            assert st["flag"][fault[0]] == 1 and (st["row"][fault[0]], st["col"][fault[0]]) == fault[1:3]
            assert np.count_nonzero(st["flag"]) == 1
        _assert_values(oracle_mod, M, N, K, a, b, c0, dc.cpu().numpy(), 1.0, 0.0)


def test_fault_campaign_with_data_scaled_threshold(blas, oracle_mod):
    """200 seeded single faults at 2048 x 2048 x 2048 on operands that are neither unit-range nor zero-mean, with the
    data-scaled threshold (tau = -1): every fault of at least 1e-3 of the typical |C| entry is detected, located
    and corrected, nothing else is flagged."""
    M = N = K = 2048
    dev = "cuda"
    da, db = torch.empty(M, K, device=dev), torch.empty(K, N, device=dev)
    blas.fill_uniform_matrix(da, M, K, 30)
    blas.fill_uniform_matrix(db, K, N, 31)
    da.mul_(100.0).add_(25.0)
    db.mul_(0.5).add_(0.125)
    dc = torch.zeros(M, N, device=dev)
    status = blas.ft_status_alloc(M, N)
    ws = blas.workspace(blas.ft_workspace_bytes(M, N, K))
    blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=-1.0, status=status, ws=ws)
    clean = blas.ft_status_numpy(status)
    assert np.count_nonzero(clean["flag"]) == 0
    c_clean = dc.clone()
    typical = float(c_clean.abs().mean())
    ntiles = blas.ft_num_tiles(M, N)
    rng = np.random.default_rng(77)
    for launch in range(200):
        tile = int(rng.integers(ntiles))
        i, j = int(rng.integers(blas.FT_TILE_M)), int(rng.integers(blas.FT_TILE_N))
        delta = float(np.float32((1 if rng.integers(2) else -1) * typical * 10.0 ** rng.uniform(-3, 1)))
        blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=-1.0, fault=(tile, i, j, delta), status=status, ws=ws)
        st = blas.ft_status_numpy(status)
        assert st["flag"][tile] == 1 and (st["row"][tile], st["col"][tile]) == (i, j), (launch, tile, i, j, delta, st[tile])
        assert np.count_nonzero(st["flag"]) == 1, launch
        assert torch.equal(dc, c_clean), (launch, float((dc - c_clean).abs().max()))


@pytest.mark.parametrize("M,N,K,tile_class", [(512, 129, 256, 1), (600, 1, 250, 0), (512, 384, 1, 0), (200, 129, 15, 2),
                                              (129, 127, 1, 1), (64, 129, 7, 1), (257, 300, 16, 2), (1, 512, 7, 2)])
def test_data_scaled_threshold_on_thin_edge_tiles_and_short_k(blas, oracle_mod, ft_mode, M, N, K, tile_class):
    """One-column edge tiles and K below 64 (found by a randomized sweep against the CPU model): a line's own
    |accumulators| can cancel to far less than its terms, and the rounding of the sums does not shrink with K; the
    tile-wide mean and the floor on K keep fault-free lines below the threshold, and a fault is still located."""
    bm, bn = blas.ft_tile(tile_class)
    ntn = -(-N // bn)
    for trial, with_fault in enumerate([False, False, True]):
        a = oracle_mod.fill_uniform_matrix(M, K, 1600 + trial, ld=K + 1)
        b = oracle_mod.fill_uniform_matrix(K, N, 1700 + trial, ld=N + 3)
        c0 = oracle_mod.fill_uniform_matrix(M, N, 1800 + trial, ld=N)
        fault = None
        if with_fault:
            tile = blas.ft_num_tiles(M, N, tile_class) - 1          # the last tile: clipped in both directions
            tm, tn = M - (tile // ntn) * bm, N - (tile % ntn) * bn
            fault = (tile, tm - 1, tn - 1, -3.25)
        da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
        status = blas.ft_status_alloc(M, N, tile_class=tile_class)
        blas.ft_sgemm(M, N, K, da, db, dc, 1.0, -0.75, tau=-1.0, fault=fault, status=status, ws=_ws(blas, ft_mode, M, N, K),
                      tile_class=tile_class)
        st = blas.ft_status_numpy(status)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm(M, N, K, a, K + 1, b, N + 3, c_model, N, 1.0, -0.75, bm, bn, -1.0, fault)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (fault, f, st[f], st_model[f])
        if fault is None:
            assert np.all(st["flag"] == 0)
        else:
            assert st["flag"][fault[0]] == 1 and (st["row"][fault[0]], st["col"][fault[0]]) == fault[1:3]
            assert np.sum(st["flag"] != 0) == 1


def test_seeded_random_cases_equal_the_model(blas, oracle_mod):
    """Random shapes, leading dimensions, alpha/beta, tile classes, both encode modes, absolute and data-scaled
    thresholds, with and without a fault: decisions equal the CPU model's, the fault is located, C is right."""
    import random
    rnd = random.Random(11)
    dims = [1, 5, 31, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 384, 400, 512, 600]
    kd = [1, 7, 15, 16, 17, 33, 64, 100, 128, 250, 256, 400, 512, 1000]
    for case in range(80):
        M, N, K = rnd.choice(dims), rnd.choice(dims), rnd.choice(kd)
        lda, ldb, ldc = K + rnd.choice([0, 0, 1, 4]), N + rnd.choice([0, 0, 3, 4]), N + rnd.choice([0, 0, 8])
        alpha, beta = rnd.choice([1.0, 1.0, -1.5, 0.5]), rnd.choice([0.0, 1.0, -0.75])
        cls, mode = rnd.choice([0, 1, 2]), rnd.choice(["fused", "workspace"])
        tau = -1.0 if rnd.random() < 0.4 else blas.ft_default_tau(K)
        bm, bn = blas.ft_tile(cls)
        ntm, ntn = -(-M // bm), -(-N // bn)
        fault = None
        if rnd.random() < 0.7:
            tile = rnd.randrange(ntm * ntn)
            tm, tn = min(bm, M - (tile // ntn) * bm), min(bn, N - (tile % ntn) * bn)
            fault = (tile, rnd.randrange(tm), rnd.randrange(tn), float(np.float32(rnd.choice([-1, 1]) * 10.0 ** rnd.uniform(-1.3, 1.5))))
        what = (case, M, N, K, lda, ldb, ldc, alpha, beta, cls, mode, tau, fault)
        a = oracle_mod.fill_uniform_matrix(M, K, 5000 + case, ld=lda)
        b = oracle_mod.fill_uniform_matrix(K, N, 6000 + case, ld=ldb)
        c0 = oracle_mod.fill_uniform_matrix(M, N, 7000 + case, ld=ldc)
        da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
        status = blas.ft_status_alloc(M, N, tile_class=cls)
        blas.ft_sgemm(M, N, K, da, db, dc, alpha, beta, tau=tau, fault=fault, status=status, ws=_ws(blas, mode, M, N, K),
                      tile_class=cls)
        st = blas.ft_status_numpy(status)
        c = dc.cpu().numpy()
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm(M, N, K, a, lda, b, ldb, c_model, ldc, alpha, beta, bm, bn, tau, fault)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (what, f, st[f], st_model[f])
        assert np.all(np.isnan(c[:, N:])), what
        caught = fault is not None and st_model["flag"][fault[0]] == 1
        if caught:
            assert (st["row"][fault[0]], st["col"][fault[0]]) == fault[1:3], what
        if fault is None or caught:   # a sub-threshold fault stays in C
            # every element obeys the componentwise criterion, the corrected one included (it is computed again)
            ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, lda, b, ldb, c0, ldc, alpha, beta)
            err = np.abs(c[:, :N].astype(np.float64) - ref)
            assert np.all(err <= TOL * den), (what, float((err - TOL * den).max()))
            if K < 512:   # (from 512 on a workspace call may split tiles along K, which sums in another order)
                # fault-free or corrected, C has the bits of the device's summation order
                want = c0.copy()
                oracle_mod.sgemm_device_order(M, N, K, a, lda, b, ldb, want, ldc, alpha, beta)
                assert np.array_equal(c[:, :N], want[:, :N]), what


@pytest.mark.parametrize("M,N,K,tile_class", [(4200, 50, 600, 4), (8300, 64, 1030, 3), (40, 8200, 520, 2), (9000, 100, 512, 2)])
def test_products_one_tile_wide_are_split_along_k_without_a_pre_pass(blas, oracle_mod, M, N, K, tile_class):
    """A product one tile wide (or high) reads each operand panel in one workgroup only: with a workspace its tiles are
    split along K by the kernels that form the checksum vectors in their main loop (no second pass over the operands).
    Decisions equal the model's, values obey the criterion, and the result does not depend on run-to-run timing."""
    bm, bn = blas.ft_tile(tile_class)
    tau = blas.ft_default_tau(K)
    a = oracle_mod.fill_uniform_matrix(M, K, 2200, ld=K + 4)
    b = oracle_mod.fill_uniform_matrix(K, N, 2201, ld=N + 4)
    c0 = oracle_mod.fill_uniform_matrix(M, N, 2202, ld=N + 8)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    ntm, ntn = -(-M // bm), -(-N // bn)
    assert min(ntm, ntn) == 1
    last = ntm * ntn - 1
    tm, tn = M - (ntm - 1) * bm, N - (ntn - 1) * bn
    for fault in [None, (last, tm - 1, tn - 1, -0.75), (ntm * ntn // 2, 17, 9, 12.5)]:
        for t in (tau, 0.0):
            results = []
            for _ in range(2):
                ws = torch.full((blas.ft_workspace_bytes(M, N, K) // 4,), float("nan"), dtype=torch.float32, device="cuda")
                dc = torch.from_numpy(c0).cuda()
                status = blas.ft_status_alloc(M, N, tile_class=tile_class)
                blas.ft_sgemm(M, N, K, da, db, dc, 1.5, -1.0, tau=t, fault=fault, status=status, ws=ws, tile_class=tile_class)
                results.append((dc.cpu().numpy(), blas.ft_status_numpy(status)))
            (c, st), (c2, st2) = results
            assert np.array_equal(c[:, :N], c2[:, :N]) and np.array_equal(st, st2)
            c_model = c0.copy()
            if ntn == 1:   # one tile wide: the rows are the screen (B is small, A is never summed)
                with oracle_mod.rows_screen():
                    st_model = oracle_mod.ft_sgemm(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, bm, bn, t, fault)
            else:
                st_model = oracle_mod.ft_sgemm(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, bm, bn, t, fault)
            for f in DECISION_FIELDS:
                assert np.array_equal(st[f], st_model[f]), (fault, t, f, st[f], st_model[f])
            ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, K + 4, b, N + 4, c0, N + 8, 1.5, -1.0)
            assert oracle_mod.gemm_max_err(N, c, c.shape[1], ref, den) <= TOL
            assert np.all(np.isnan(c[:, N:]))
            # the split did happen: C differs in the last bits from the unsplit call (no workspace)
            dc = torch.from_numpy(c0).cuda()
            blas.ft_sgemm(M, N, K, da, db, dc, 1.5, -1.0, tau=t, fault=fault, tile_class=tile_class)
            assert not np.array_equal(dc.cpu().numpy()[:, :N], c[:, :N])


def test_one_tile_wide_takes_the_rows_as_the_screen(blas, oracle_mod):
    """Row x column location on a product one tile wide with a workspace: the row checksums (from the small B) are the
    screen and the column references are formed only when a row is flagged.  Two faults that cancel in their row are
    not seen (with the columns as the screen they would be two flagged columns: detected, not correctable); two faults
    in one column show as two rows and one column; a single fault is located and corrected to the bits of the clean
    product."""
    M, N, K, tile_class = 8300, 60, 530, 3
    bm, bn = blas.ft_tile(tile_class)
    tau = blas.ft_default_tau(K)
    a = oracle_mod.fill_uniform_matrix(M, K, 2300, ld=K + 4)
    b = oracle_mod.fill_uniform_matrix(K, N, 2301, ld=N + 4)
    c0 = oracle_mod.fill_uniform_matrix(M, N, 2302, ld=N + 8)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    ws = torch.full((blas.ft_workspace_bytes(M, N, K) // 4,), float("nan"), dtype=torch.float32, device="cuda")

    def run(faults):
        dc = torch.from_numpy(c0).cuda()
        status = blas.ft_status_alloc(M, N, tile_class=tile_class)
        blas.ft_sgemm(M, N, K, da, db, dc, 1.0, 0.0, tau=tau, faults=faults, status=status, ws=ws, tile_class=tile_class)
        return dc.cpu().numpy(), blas.ft_status_numpy(status)

    clean, st = run(None)
    assert not st["flag"].any() and not st["n_bad_rows"].any() and not st["n_bad_cols"].any()
    cases = {"cancel in a row": [(5, 7, 3, 2.0), (5, 7, 40, -2.0)], "one column": [(9, 7, 3, 2.0), (9, 90, 3, 1.0)],
             "single": [(64, 100, 59, -0.5)], "last tile": [(-(-M // bm) - 1, M - (-(-M // bm) - 1) * bm - 1, N - 1, 3.0)]}
    for name, faults in cases.items():
        c, st = run(faults)
        c_model = c0.copy()
        with oracle_mod.rows_screen():
            st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 0.0, bm, bn, tau, 0, faults)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (name, f, st[f], st_model[f])
        t = faults[0][0]
        if name == "cancel in a row":
            assert st["flag"][t] == 0 and st["n_bad_cols"][t] == 0
            assert not np.array_equal(c[:, :N], clean[:, :N])      # both faults are still in C
        elif name == "one column":
            assert st["flag"][t] == 2 and (st["n_bad_rows"][t], st["n_bad_cols"][t]) == (2, 1)
        else:
            assert st["flag"][t] == 1 and (st["row"][t], st["col"][t]) == faults[0][1:3]
            assert abs(st["col_residual"][t] + faults[0][3]) < 2e-3 and abs(st["row_residual"][t] + faults[0][3]) < 2e-3
            assert np.array_equal(c[:, :N], clean[:, :N]), name
        assert np.count_nonzero(st["flag"]) == (0 if name == "cancel in a row" else 1)


def test_partial_last_round_is_split_along_k(blas, oracle_mod):
    """With room in the workspace the tiles of a partial last round of CUs are split along K; every slice verifies its
    own partial product, a second pass adds the slices and merges their records.  Decisions and C must not depend on
    whether the split happened."""
    M, N, K = 700, 300, 2048                      # 3 x 3 tiles of 256x128 on 256 CUs: all nine are split (8 ways)
    enc_only = 4 * (-(-M // 256) + -(-N // 128)) * ((-(-K // 16) + 2) * 16)
    enc_only = (enc_only + 15) // 16 * 16
    need = blas.ft_workspace_bytes(M, N, K)
    assert need > enc_only + 9 * 2 * 256 * 128 * 4  # the query includes the slices
    tau = blas.ft_default_tau(K)
    a = oracle_mod.fill_uniform_matrix(M, K, 2100, ld=K + 4)
    b = oracle_mod.fill_uniform_matrix(K, N, 2101, ld=N + 4)
    c0 = oracle_mod.fill_uniform_matrix(M, N, 2102, ld=N + 8)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    for fault in [None, (8, 700 - 512 - 1, 300 - 256 - 1, -0.75), (4, 17, 90, 12.5)]:
        for t in (tau, -1.0):
            results = []
            for nbytes in (need, enc_only, need):   # split, not split, split again
                ws = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
                dc = torch.from_numpy(c0).cuda()
                status = blas.ft_status_alloc(M, N)
                blas.ft_sgemm(M, N, K, da, db, dc, 1.5, -1.0, tau=t, fault=fault, status=status, ws=ws)
                results.append((dc.cpu().numpy(), blas.ft_status_numpy(status)))
            c_model = c0.copy()
            st_model = oracle_mod.ft_sgemm(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, 256, 128, t, fault)
            for c, st in results:
                for f in DECISION_FIELDS:
                    assert np.array_equal(st[f], st_model[f]), (fault, t, f, st[f], st_model[f])
                _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.5, -1.0)
                if fault is not None:
                    assert abs(st["row_residual"][fault[0]] + fault[3]) < 2e-3
            assert np.array_equal(results[0][0][:, :N], results[2][0][:, :N])      # fixed order: same bits on every run
            assert not np.array_equal(results[0][0][:, :N], results[1][0][:, :N])  # the split did change the summation order
    # no status array: the slices keep no records either
    dc = torch.from_numpy(c0).cuda()
    blas.ft_sgemm(M, N, K, da, db, dc, 1.5, -1.0, tau=tau, ws=torch.empty(need // 4, dtype=torch.float32, device="cuda"))
    _assert_values(oracle_mod, M, N, K, a, b, c0, dc.cpu().numpy(), 1.5, -1.0)
    # a real partial round: 288 tiles of 256x128 at 3072^2, 32 of them split; sampled rows + every record clean
    n = 3072
    a3 = torch.empty(n, n, device="cuda"); b3 = torch.empty(n, n, device="cuda"); c3 = torch.zeros(n, n, device="cuda")
    blas.fill_uniform_matrix(a3, n, n, 2200); blas.fill_uniform_matrix(b3, n, n, 2201)
    status = blas.ft_status_alloc(n, n)
    ws = blas.workspace(blas.ft_workspace_bytes(n, n, n))
    fault = (287, 255, 127, 0.5)   # the last tile, one of the split ones
    blas.ft_sgemm(n, n, n, a3, b3, c3, 1.0, 0.0, fault=fault, status=status, ws=ws)
    st = blas.ft_status_numpy(status)
    assert st["flag"].sum() == 1 and st["flag"][287] == 1 and (st["row"][287], st["col"][287]) == (255, 127)
    rows = torch.tensor([0, 1500, 2816, 3071], device="cuda")
    ref = a3[rows].double() @ b3.double()
    den = a3[rows].abs().double() @ b3.abs().double()
    assert float(((c3[rows].double() - ref).abs() / den).max()) <= TOL


@pytest.mark.parametrize("tile_class,M,N,K", [(0, 768, 640, 1100), (1, 512, 384, 800), (4, 300, 200, 530)])
def test_workspace_reuse_and_graph_replay_see_fresh_operands(blas, tile_class, M, N, K):
    """The checksum vectors in the workspace belong to one call: a workspace of unknown contents, back-to-back calls
    that reuse it with other operands, and replays of a captured call whose operands changed in between must all
    verify against the operands of *that* call - a stale checksum vector would flag every tile."""
    dev = "cuda"
    ops = []
    for seed in (910, 920):
        a = torch.empty(M, K, device=dev)
        b = torch.empty(K, N, device=dev)
        blas.fill_uniform_matrix(a, M, K, seed)
        blas.fill_uniform_matrix(b, K, N, seed + 1)
        ops.append((a, b, (a.double() @ b.double()).float()))
    ws = torch.full((blas.ft_workspace_bytes(M, N, K) // 4,), float("nan"), device=dev)  # poisoned
    tau = blas.ft_default_tau(K)
    results = []
    for rnd in range(3):
        for a, b, _ in ops:  # no synchronisation between the calls
            c = torch.empty(M, N, device=dev)
            status = blas.ft_status_alloc(M, N, tile_class=tile_class)
            blas.ft_sgemm(M, N, K, a, b, c, 1.0, 0.0, tau=tau, status=status, ws=ws, tile_class=tile_class)
            results.append((c, status))
    torch.cuda.synchronize()
    for i, (c, status) in enumerate(results):
        st = blas.ft_status_numpy(status)
        assert not st["flag"].any(), (i, st["flag"])
        assert (c - ops[i % 2][2]).abs().max().item() < 1e-3 * (K ** 0.5)
    # a captured call, replayed with the operands it was captured with and then with new ones in the same buffers
    a, b = ops[0][0].clone(), ops[0][1].clone()
    c = torch.empty(M, N, device=dev)
    status = blas.ft_status_alloc(M, N, tile_class=tile_class)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        blas.ft_sgemm(M, N, K, a, b, c, 1.0, 0.0, tau=tau, status=status, ws=ws, tile_class=tile_class)
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=side):
            blas.ft_sgemm(M, N, K, a, b, c, 1.0, 0.0, tau=tau, status=status, ws=ws, tile_class=tile_class)
    torch.cuda.synchronize()
    for replay in range(4):
        src = ops[replay % 2]
        a.copy_(src[0])
        b.copy_(src[1])
        c.fill_(float("nan"))
        status.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        st = blas.ft_status_numpy(status)
        assert not st["flag"].any(), (replay, st["flag"])
        assert (c - src[2]).abs().max().item() < 1e-3 * (K ** 0.5), replay
