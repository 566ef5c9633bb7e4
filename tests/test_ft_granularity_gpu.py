"""GPU parity of the ABFT options against the CPU model: wave-tile checksum granularity (the counterpart of the
reference's warp- / thread-level kernels, ft_sgemm_huge_warp.cuh:111-207, ft_sgemm_huge_thread.cuh:106-177) and the
verification cadence inside the K loop with re-synchronised references (ft_sgemm_huge.cuh:143,263-271).

Decisions (flag, located row and column, bad-line counts per check tile) must equal the model's exactly; values obey
the 1e-5 componentwise criterion once every fault is corrected."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-5
DECISION_FIELDS = ("flag", "row", "col", "n_bad_rows", "n_bad_cols")


def _ws(blas, M, N, K):
    return torch.full((max(blas.ft_workspace_bytes(M, N, K) // 4, 4),), float("nan"), dtype=torch.float32, device="cuda")


def _ws_checksums_only(blas, M, N, K, tile_class=0, granularity=0):
    """A workspace with room for the checksum vectors and nothing else: the call cannot split tiles along K."""
    bm, bn = blas.ft_tile(tile_class)
    cm, cn = blas.ft_check_tile(tile_class, granularity)
    words = (-(-M // bm) * (bm // cm) + -(-N // bn) * (bn // cn)) * ((-(-K // 16) + 2) * 16)
    return torch.full(((words + 3) // 4 * 4,), float("nan"), dtype=torch.float32, device="cuda")


def _problem(oracle_mod, M, N, K, seed, pad=(4, 4, 8)):
    a = oracle_mod.fill_uniform_matrix(M, K, seed, ld=K + pad[0])
    b = oracle_mod.fill_uniform_matrix(K, N, seed + 1, ld=N + pad[1])
    c0 = oracle_mod.fill_uniform_matrix(M, N, seed + 2, ld=N + pad[2])
    return a, b, c0


def _device_run(blas, a, b, c0, M, N, K, alpha, beta, tau, ws, **kw):
    da, db, dc = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda(), torch.from_numpy(c0).cuda()
    status = blas.ft_status_alloc(M, N, tile_class=kw.get("tile_class", 0), granularity=kw.get("granularity", 0))
    blas.ft_sgemm(M, N, K, da, db, dc, alpha, beta, tau=tau, status=status, ws=ws, **kw)
    return dc.cpu().numpy(), blas.ft_status_numpy(status)


def _assert_values(oracle_mod, M, N, K, a, b, c0, c, alpha, beta):
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, a.shape[1], b, b.shape[1], c0, c0.shape[1], alpha, beta)
    err = oracle_mod.gemm_max_err(N, c, c.shape[1], ref, den)
    assert err <= TOL, err
    assert np.all(np.isnan(c[:, N:]))


def test_check_tile_table(blas):
    assert [blas.ft_check_tile(c, blas.FT_GRAN_TILE) for c in range(5)] == [(256, 128), (128, 128), (64, 128), (128, 64), (64, 64)]
    assert [blas.ft_check_tile(c, blas.FT_GRAN_WAVE) for c in range(5)] == [(128, 32), (64, 64), (32, 64), (64, 32), (32, 32)]
    assert blas.ft_num_check_tiles(300, 300, 0, blas.FT_GRAN_WAVE) == 3 * 10
    assert blas.ft_num_check_tiles(300, 300, 0, blas.FT_GRAN_TILE) == blas.ft_num_tiles(300, 300) == 2 * 3


@pytest.mark.parametrize("tile_class", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("tau_kind", ["absolute", "scaled"])
def test_wave_tiles_decisions_equal_the_model(blas, oracle_mod, tile_class, tau_kind):
    """One checksum pair, one verification and one record per wave tile; ragged in every dimension, so edge tiles have
    clipped wave tiles and wave tiles that lie outside the matrix altogether."""
    cm, cn = blas.ft_check_tile(tile_class, blas.FT_GRAN_WAVE)
    M, N, K = 333, 300, 520
    tau = blas.ft_default_tau(K) if tau_kind == "absolute" else -1.0
    ntm, ntn = -(-M // cm), -(-N // cn)
    rng = np.random.default_rng(60 + tile_class)
    ws = _ws(blas, M, N, K)
    for trial in range(8):
        a, b, c0 = _problem(oracle_mod, M, N, K, 900 + 10 * trial)
        fault = None
        if trial:
            tile = int(rng.integers(ntm * ntn))
            tm, tn = min(cm, M - (tile // ntn) * cm), min(cn, N - (tile % ntn) * cn)
            fault = (tile, int(rng.integers(tm)), int(rng.integers(tn)),
                     float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-1.3, 2))))
        c, st = _device_run(blas, a, b, c0, M, N, K, 1.0, 1.0, tau, ws, tile_class=tile_class,
                            granularity=blas.FT_GRAN_WAVE, fault=fault)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 1.0, cm, cn, tau, fault)
        assert len(st) == ntm * ntn
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (tile_class, fault, f, st[f], st_model[f])
        if fault is not None:
            assert st["flag"][fault[0]] == 1 and (st["row"][fault[0]], st["col"][fault[0]]) == fault[1:3]
            assert np.count_nonzero(st["flag"]) == 1
            assert abs(st["row_residual"][fault[0]] + fault[3]) < 2e-3 + 1e-6 * abs(fault[3])
        _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 1.0)


@pytest.mark.parametrize("tile_class,granularity", [(4, 1), (2, 0)])
def test_long_k_and_many_row_groups_in_the_pre_pass(blas, oracle_mod, tile_class, granularity):
    """The pre-pass with 34 row groups, 2 blocks of 128 columns and 62 blocks of k: K is not a multiple of its 64 values
    of k per block, nor of the K step."""
    cm, cn = blas.ft_check_tile(tile_class, granularity)
    M, N, K = 17 * (64 if granularity else 128) - 3, 250, 3900
    tau = blas.ft_default_tau(K)
    ntn = -(-N // cn)
    a, b, c0 = _problem(oracle_mod, M, N, K, 4100 + tile_class)
    fault = (5 * ntn + 1, 7, 9, -2.5)
    c, st = _device_run(blas, a, b, c0, M, N, K, 1.0, 1.0, tau, _ws(blas, M, N, K), tile_class=tile_class, granularity=granularity,
                        fault=fault)
    c_model = c0.copy()
    st_model = oracle_mod.ft_sgemm(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 1.0, cm, cn, tau, fault)
    for f in DECISION_FIELDS:
        assert np.array_equal(st[f], st_model[f]), (f, st[f], st_model[f])
    assert np.count_nonzero(st["flag"]) == 1 and (st["row"][fault[0]], st["col"][fault[0]]) == fault[1:3]
    assert st["max_clean_residual"].max() < 0.6 * tau
    _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 1.0)


def test_two_faults_in_one_workgroup_tile_need_wave_granularity(blas, oracle_mod):
    """Two simultaneous faults in different wave tiles of one 256 x 128 tile: tile granularity sees two bad rows and two
    bad columns and reports the tile uncorrectable; wave-tile granularity corrects both."""
    M, N, K = 512, 256, 512
    tau = blas.ft_default_tau(K)
    a, b, c0 = _problem(oracle_mod, M, N, K, 1200)
    ws = _ws(blas, M, N, K)
    # workgroup tile 3 = rows 256.., columns 128..; the faults sit in its wave tiles (0, 1) and (1, 3)
    f_tile = [(3, 17, 40, 0.5), (3, 200, 100, -3.0)]
    for mode_ws in (ws, None):
        c, st = _device_run(blas, a, b, c0, M, N, K, 1.0, 0.0, tau, mode_ws, faults=f_tile)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 0.0, 256, 128, tau, 0, f_tile)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (f, st[f], st_model[f])
        assert st["flag"].tolist() == [0, 0, 0, 2] and (st["n_bad_rows"][3], st["n_bad_cols"][3]) == (2, 2)
        # uncorrectable: both faults are still in C
        ref, _ = oracle_mod.gemm_f64_rows(M, N, K, a, K + 4, b, N + 4, c0, N + 8, 1.0, 0.0)
        assert abs(c[256 + 17, 128 + 40] - ref[256 + 17, 128 + 40] - 0.5) < 1e-3
        assert abs(c[256 + 200, 128 + 100] - ref[256 + 200, 128 + 100] + 3.0) < 1e-3
    # the same two elements in wave-tile units (128 x 32 wave tiles, 4 x 8 of them): rows 256+17 -> wave row 2, local 17;
    # columns 128+40 -> wave column 5, local 8; rows 256+200 -> wave row 3, local 72; columns 128+100 -> 7, local 4
    f_wave = [(2 * 8 + 5, 17, 8, 0.5), (3 * 8 + 7, 72, 4, -3.0)]
    c, st = _device_run(blas, a, b, c0, M, N, K, 1.0, 0.0, tau, ws, granularity=blas.FT_GRAN_WAVE, faults=f_wave)
    c_model = c0.copy()
    st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 0.0, 128, 32, tau, 0, f_wave)
    for f in DECISION_FIELDS:
        assert np.array_equal(st[f], st_model[f]), (f, st[f], st_model[f])
    assert np.count_nonzero(st["flag"]) == 2 and st["flag"][21] == 1 and st["flag"][31] == 1
    assert (st["row"][21], st["col"][21], st["row"][31], st["col"][31]) == (17, 8, 72, 4)
    _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.0, 0.0)
    # two faults in ONE wave tile are beyond wave granularity too
    f_same = [(21, 17, 8, 0.5), (21, 100, 30, -3.0)]
    c, st = _device_run(blas, a, b, c0, M, N, K, 1.0, 0.0, tau, ws, granularity=blas.FT_GRAN_WAVE, faults=f_same)
    assert st["flag"][21] == 2 and np.count_nonzero(st["flag"]) == 1


@pytest.mark.parametrize("mode", ["fused", "workspace"])
def test_verification_cadence_corrects_one_fault_per_interval(blas, oracle_mod, mode):
    """Verification every 256 k with re-synchronised references: two faults in one tile that fall into different
    intervals are both located and corrected; seen by a single verification after the K loop they are not."""
    M, N, K = 512, 300, 1100     # ragged N and K: 5 verifications (k = 256, 512, 768, 1024, 1100)
    tau = blas.ft_default_tau(K)
    a, b, c0 = _problem(oracle_mod, M, N, K, 1300)
    ws = _ws(blas, M, N, K) if mode == "workspace" else None
    cases = [
        [],
        [(4, 100, 30, 0.75, 0)],
        [(4, 100, 30, 0.75, 1), (4, 7, 2, -12.0, 3)],
        [(1, 255, 127, 5.0, 4), (1, 0, 0, -0.02, 0), (5, 200, 43, 1.0, 2)],   # tile 5 is 44 columns wide
        [(0, 1, 1, 1.0, 2), (0, 2, 2, 1.0, 2)],                                # same interval: uncorrectable
    ]
    for faults in cases:
        c, st = _device_run(blas, a, b, c0, M, N, K, 1.5, -1.0, tau, ws, check_interval=256, faults=faults)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, 256, 128, tau, 256, faults)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (faults, f, st[f], st_model[f])
        assert np.allclose(st["row_residual"], st_model["row_residual"], atol=2e-3)
        assert st["max_clean_residual"].max() < 0.6 * tau
        if not np.any(st["flag"] == 2):
            _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.5, -1.0)
        # one verification after the loop sees all faults of a tile at once
        if len(faults) >= 2:
            c1, st1 = _device_run(blas, a, b, c0, M, N, K, 1.5, -1.0, tau, ws, faults=faults)
            c_model = c0.copy()
            st1_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, 256, 128, tau, 0, faults)
            for f in DECISION_FIELDS:
                assert np.array_equal(st1[f], st1_model[f]), (faults, f, st1[f], st1_model[f])
            assert np.any(st1["flag"] == 2)
    # fault-free: the cadence changes nothing in C (same accumulation order as the plain kernel on this tile)
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    # (with room in the workspace these six tiles would be split along K, which sums in another order)
    c_cad, _ = _device_run(blas, a, b, c0, M, N, K, 1.5, -1.0, tau, ws if ws is None else _ws_checksums_only(blas, M, N, K), check_interval=256)
    plain = torch.from_numpy(c0).cuda()
    blas.sgemm(M, N, K, da, db, plain, 1.5, -1.0, tile=0, split_k=1)
    assert np.array_equal(c_cad[:, :N], plain.cpu().numpy()[:, :N])


@pytest.mark.parametrize("mode", ["fused", "workspace"])
def test_verification_cadence_on_the_128x128_class(blas, oracle_mod, mode):
    """The same on 128 x 128 tiles (tile numbers, rows and columns of the faults are those of that class)."""
    M, N, K = 300, 260, 900      # 3 x 3 tiles, 4 verifications (k = 256, 512, 768, 900)
    tau = blas.ft_default_tau(K)
    a, b, c0 = _problem(oracle_mod, M, N, K, 1350)
    ws = _ws(blas, M, N, K) if mode == "workspace" else None
    for faults in ([], [(4, 100, 30, 0.75, 1), (4, 7, 2, -12.0, 3)], [(8, 43, 3, 2.0, 0), (0, 127, 127, -0.5, 2), (0, 1, 1, 1.0, 2)]):
        c, st = _device_run(blas, a, b, c0, M, N, K, 1.5, -1.0, tau, ws, tile_class=1, check_interval=256, faults=faults)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, 128, 128, tau, 256, faults)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (faults, f, st[f], st_model[f])
        if not np.any(st["flag"] == 2):
            _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.5, -1.0)


@pytest.mark.parametrize("tile_class", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("kind", ["tile-fused", "tile-workspace", "wave-workspace"])
def test_every_class_granularity_and_cadence_equals_the_model(blas, oracle_mod, tile_class, kind):
    """The whole option matrix: every tile class, both granularities, checksum vectors from the main loop or from the
    workspace, with the verification every 256 k (the reference's scheme: every shape of its table has an ABFT kernel
    with the in-loop check, kernel/ft_sgemm/sgemm.cu:186-192, ft_sgemm_large.cuh:337, ft_sgemm_tall.cuh:18) and, for
    comparison, with one verification.  Ragged in every dimension; faults in check-tile units, in different intervals."""
    gran = blas.FT_GRAN_WAVE if kind.startswith("wave") else blas.FT_GRAN_TILE
    cm, cn = blas.ft_check_tile(tile_class, gran)
    M, N, K = 333, 200, 900      # 4 verifications (k = 256, 512, 768, 900)
    tau = blas.ft_default_tau(K)
    a, b, c0 = _problem(oracle_mod, M, N, K, 1500 + tile_class)
    # (no room for K slices: every element is summed by one workgroup, in the order the model below knows)
    ws = _ws_checksums_only(blas, M, N, K, tile_class, gran) if kind.endswith("workspace") else None
    ntm, ntn = -(-M // cm), -(-N // cn)
    rng = np.random.default_rng(70 + tile_class)

    def fault(tile, check):
        tm, tn = min(cm, M - (tile // ntn) * cm), min(cn, N - (tile % ntn) * cn)
        return (tile, int(rng.integers(tm)), int(rng.integers(tn)),
                float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-1.0, 1.5))), check)

    last = ntm * ntn - 1   # the corner check tile, clipped in both directions
    cases = [[], [fault(0, 0)], [fault(last, 1), fault(last, 3)], [fault(1, 2), fault(ntn, 0), fault(ntn, 3)],
             [fault(1, 2), fault(1, 2)]]                                     # same interval: uncorrectable
    for faults in cases:
        for interval in (256, 0):
            c, st = _device_run(blas, a, b, c0, M, N, K, 1.5, -1.0, tau, ws, tile_class=tile_class, granularity=gran,
                                check_interval=interval, faults=faults)
            c_model = c0.copy()
            st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, cm, cn, tau, interval, faults)
            assert len(st) == ntm * ntn
            for f in DECISION_FIELDS:
                assert np.array_equal(st[f], st_model[f]), (tile_class, kind, interval, faults, f, st[f], st_model[f])
            if not np.any(st["flag"] == 2):
                _assert_values(oracle_mod, M, N, K, a, b, c0, c, 1.5, -1.0)
                # corrected or fault-free, C has the bits of the device's summation order
                want = c0.copy()
                oracle_mod.sgemm_device_order(M, N, K, a, K + 4, b, N + 4, want, N + 8, 1.5, -1.0)
                assert np.array_equal(c[:, :N], want[:, :N]), (tile_class, kind, interval, faults)


@pytest.mark.parametrize("tile_class,granularity", [(0, 0), (0, 1), (1, 1), (3, 0), (4, 1)])
def test_partial_last_round_is_split_along_k_under_cadence_and_wave_granularity(blas, oracle_mod, tile_class, granularity):
    """With room in the workspace the tiles of a partial last round of CUs are split along K; under a verification
    cadence every slice is a whole number of intervals and verifies its own, with wave-tile granularity every slice
    keeps one record per wave tile.  Decisions must equal the model's (which knows nothing of slices) and must not
    depend on whether the split happened; C agrees to rounding (a split sums K in another order)."""
    bm, bn = blas.ft_tile(tile_class)
    cm, cn = blas.ft_check_tile(tile_class, granularity)
    M, N, K = 2 * bm + bm // 2 + 3, 2 * bn + 5, 2048      # 3 x 3 workgroup tiles: fewer than half the CUs, all split
    tau = blas.ft_default_tau(K)
    a, b, c0 = _problem(oracle_mod, M, N, K, 1600 + tile_class)
    need = blas.ft_workspace_bytes(M, N, K)
    gm, gn = bm // cm, bn // cn
    enc_only = 4 * (-(-M // bm) * gm + -(-N // bn) * gn) * ((-(-K // 16) + 2) * 16)
    enc_only = (enc_only + 15) // 16 * 16
    assert need > enc_only + 9 * 2 * bm * bn * 4
    ntn = -(-N // cn)
    corner = (-(-M // cm)) * ntn - 1
    for interval, faults in [(0, [(corner, 1, 2, -0.75, 0)]),
                             (128, [(corner, 1, 2, -0.75, 5), (corner, 2, 1, 3.0, 13), (ntn + 1, 17, 9, 12.5, 0)]),
                             (512, [(0, 0, 0, 1.0, 3), (0, 5, 5, -1.0, 1)]),
                             (128, [(1, 3, 3, 1.0, 9), (1, 4, 4, 1.0, 9)])]:      # same interval: uncorrectable
        results = []
        for nbytes in (need, enc_only):   # split, not split
            ws = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
            results.append(_device_run(blas, a, b, c0, M, N, K, 1.5, -1.0, tau, ws, tile_class=tile_class,
                                       granularity=granularity, check_interval=interval, faults=faults))
        (c_split, st_split), (c_whole, st_whole) = results
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.5, -1.0, cm, cn, tau, interval, faults)
        for f in DECISION_FIELDS:
            assert np.array_equal(st_split[f], st_model[f]), (interval, faults, f, st_split[f], st_model[f])
            assert np.array_equal(st_whole[f], st_model[f]), (interval, faults, f, st_whole[f], st_model[f])
        if not np.any(st_model["flag"] == 2):
            _assert_values(oracle_mod, M, N, K, a, b, c0, c_split, 1.5, -1.0)
            _assert_values(oracle_mod, M, N, K, a, b, c0, c_whole, 1.5, -1.0)
            assert not np.array_equal(c_split[:, :N], c_whole[:, :N])   # the split did happen


def test_cadence_with_data_scaled_threshold_and_interval_edge_cases(blas, oracle_mod):
    M, N, K = 300, 200, 700
    a, b, c0 = _problem(oracle_mod, M, N, K, 1400)
    a = (a * np.float32(40.0)).astype(np.float32)
    ws = _ws(blas, M, N, K)
    typical = float(np.abs(a[:64, :K].astype(np.float64) @ b[:, :N].astype(np.float64)).mean())
    faults = [(2, 40, 70, 0.05 * typical, 0), (2, 3, 9, -0.2 * typical, 2)]
    for interval in (256, 16, 688, 704, 4096):   # 704 and above cover all of K: a single verification
        for use_ws in (ws, None):
            c, st = _device_run(blas, a, b, c0, M, N, K, 1.0, 0.0, -1.0, use_ws, check_interval=interval, faults=faults)
            c_model = c0.copy()
            st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 0.0, 256, 128, -1.0, interval, faults)
            for f in DECISION_FIELDS:
                assert np.array_equal(st[f], st_model[f]), (interval, f, st[f], st_model[f])
            assert st["flag"][2] == (1 if interval < 700 else 2)


def test_option_errors(blas):
    t = torch.zeros(256, 256, device="cuda")
    ws = torch.zeros(1 << 20, device="cuda")
    with pytest.raises(blas.HpcdnnError):   # wave-tile checksums come from the workspace
        blas.ft_sgemm(256, 256, 256, t, t, t.clone(), 1.0, 0.0, granularity=blas.FT_GRAN_WAVE)
    with pytest.raises(blas.HpcdnnError):   # five classes
        blas.ft_sgemm(256, 256, 256, t, t, t.clone(), 1.0, 0.0, tile_class=5, check_interval=64, ws=ws)
    with pytest.raises(blas.HpcdnnError):   # a multiple of the K step
        blas.ft_sgemm(256, 256, 256, t, t, t.clone(), 1.0, 0.0, check_interval=100, ws=ws)
    with pytest.raises(blas.HpcdnnError):   # wave tile 128 x 32: column 32 does not exist
        blas.ft_sgemm(256, 256, 256, t, t, t.clone(), 1.0, 0.0, granularity=blas.FT_GRAN_WAVE, ws=ws, faults=[(0, 0, 32, 1.0)])
    with pytest.raises(blas.HpcdnnError):
        blas.ft_sgemm(256, 256, 256, t, t, t.clone(), 1.0, 0.0, granularity=2, ws=ws)


@pytest.mark.parametrize("mode", ["workspace", "fused"])
@pytest.mark.parametrize("tile_class", [0, 1, 3])
def test_columns_screen_and_rows_locate(blas, oracle_mod, mode, tile_class):
    """The column checksums screen (the reference acts only when a column and a row disagree,
    ft_sgemm_huge.cuh:289): two faults of 0.75 tau in one ROW show in no column and leave the tile clean, with both
    faults still in C; the same two faults in one COLUMN add up to 1.5 tau there, are detected and cannot be located
    (no row passes its threshold); with a verification every 256 k each of them is seen alone and absorbed."""
    bm, bn = blas.ft_tile(tile_class)
    M, N, K = 2 * bm + 40, bn + 24, 768
    a, b, c0 = _problem(oracle_mod, M, N, K, 640 + tile_class)
    tau, d = 0.05, 0.0375
    ws = _ws(blas, M, N, K) if mode == "workspace" else None
    clean, _ = _device_run(blas, a, b, c0, M, N, K, 1.0, 0.0, tau, ws, tile_class=tile_class)
    tile = 2  # second tile row, first tile column
    cases = {
        "one row": ([(tile, 9, 4, d, 0), (tile, 9, 61, d, 1)], 0, (0, 0, 0)),
        "one column": ([(tile, 9, 4, d, 0), (tile, 33, 4, d, 1)], 0, (2, 0, 1)),
        "one column, cadence": ([(tile, 9, 4, d, 0), (tile, 33, 4, d, 1)], 256, (0, 0, 0)),
        "row and column": ([(tile, 9, 4, 4 * d, 0)], 0, (1, 1, 1)),
    }
    for name, (faults, interval, want) in cases.items():
        c, st = _device_run(blas, a, b, c0, M, N, K, 1.0, 0.0, tau, ws, tile_class=tile_class, check_interval=interval, faults=faults)
        c_model = c0.copy()
        st_model = oracle_mod.ft_sgemm_checked(M, N, K, a, K + 4, b, N + 4, c_model, N + 8, 1.0, 0.0, bm, bn, tau, interval, faults)
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (name, f, st[f], st_model[f])
        assert (st["flag"][tile], st["n_bad_rows"][tile], st["n_bad_cols"][tile]) == want, name
        assert np.count_nonzero(st["flag"]) == (1 if want[0] else 0), name
        if want[0] == 1:
            assert np.array_equal(c[:, :N], clean[:, :N]), name   # corrected: the bits of the fault-free product
        else:
            # not corrected: the faults are still in C, everything else has the fault-free bits
            diff = np.argwhere(c[:, :N] != clean[:, :N])
            rows0 = (tile // -(-N // bn)) * bm
            assert sorted(map(tuple, diff)) == sorted((rows0 + r, col) for (_, r, col, _, _) in faults), name
