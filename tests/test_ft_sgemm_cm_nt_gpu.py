"""GPU parity of the ABFT SGEMM on the reference family's column-major buffers, ``C = alpha*A*B^T + beta*C`` as
``ft_sgemm_huge<<<...>>>(M, N, K, A, B, C, alpha, beta)`` takes them (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:21,
kernel/ft_sgemm/sgemm.cu:159-165).

Values: the 1e-5 componentwise criterion against the oracle's restatement of the column-major product (after
correction).  Decisions: equal to the CPU model of the checksum logic run on the row-major problem C^T = (B^T)^T A^T,
which is how the entry point numbers its tiles, records and faults; and, fault-free, the same bits as ``ft_sgemm`` on
an explicitly transposed copy of B (the products of an element are added in the same order; the checksum vectors of
the pre-pass are not, so residuals agree to rounding only).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 1e-5
DECISION_FIELDS = ("flag", "row", "col", "n_bad_rows", "n_bad_cols")


@pytest.fixture(params=["fused", "workspace"])
def ft_mode(request):
    """Checksum vectors formed in the main loop (no workspace) or by the pre-pass kernels (with workspace)."""
    return request.param


def _buffers(oracle_mod, M, N, K, pad, seed):
    lda, ldb, ldc = M + pad[0], N + pad[1], M + pad[2]
    abuf = oracle_mod.fill_uniform_matrix(K, M, seed, ld=lda)       # column k of A = row k of the buffer
    bbuf = oracle_mod.fill_uniform_matrix(K, N, seed + 1, ld=ldb)
    cbuf = oracle_mod.fill_uniform_matrix(N, M, seed + 2, ld=ldc)
    return abuf, bbuf, cbuf


def _ws(blas, M, N, K):
    nbytes = blas.ft_cm_nt_workspace_bytes(M, N, K)
    assert nbytes == blas.ft_workspace_bytes(N, M, K)   # the operands are read where they lie: no transposed copy
    return torch.full((max(nbytes // 4, 4),), float("nan"), dtype=torch.float32, device="cuda")   # poisoned


def _run(blas, oracle_mod, M, N, K, alpha, beta, tau, faults=None, pad=(0, 0, 0), seed=600, mode="workspace", values=True, **opts):
    abuf, bbuf, cbuf = _buffers(oracle_mod, M, N, K, pad, seed)
    da, db, dc = torch.from_numpy(abuf).cuda(), torch.from_numpy(bbuf).cuda(), torch.from_numpy(cbuf).cuda()
    tile_class, gran = opts.get("tile_class", 0), opts.get("granularity", 0)
    status = blas.ft_status_alloc(N, M, tile_class=tile_class, granularity=gran)
    ws = _ws(blas, M, N, K) if mode == "workspace" else None
    if mode == "workspace" and opts.pop("no_split", False):
        # room for the checksum vectors only: no tile can be split along K, every element is summed by one workgroup
        bm, bn = blas.ft_tile(tile_class)
        cm, cn = blas.ft_check_tile(tile_class, gran)
        words = (-(-N // bm) * (bm // cm) + -(-M // bn) * (bn // cn)) * ((-(-K // 16) + 2) * 16)
        ws = torch.full(((words + 3) // 4 * 4,), float("nan"), dtype=torch.float32, device="cuda")
    opts.pop("no_split", None)
    blas.ft_sgemm_cm_nt(M, N, K, da, db, dc, alpha, beta, ws, tau=tau, status=status, faults=faults, **opts)
    c = dc.cpu().numpy()
    ref, den = oracle_mod.gemm_cm_nt_f64(M, N, K, abuf, abuf.shape[1], bbuf, bbuf.shape[1], cbuf, cbuf.shape[1], alpha, beta)
    err = oracle_mod.gemm_max_err(M, c, c.shape[1], ref, den)
    assert err <= TOL or not values, err   # (values=False: the caller leaves uncorrectable faults in C)
    assert np.all(np.isnan(c[:, M:]))
    return abuf, bbuf, cbuf, c, blas.ft_status_numpy(status), status


@pytest.mark.parametrize("M,N,K,pad", [(128, 256, 64, (0, 0, 0)), (384, 512, 320, (0, 0, 0)), (200, 300, 100, (4, 8, 12)), (1, 1, 1, (0, 0, 0)),
                                      (129, 257, 17, (3, 1, 2)), (1024, 1024, 1024, (0, 0, 0))])
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (1.0, -1.5)])
def test_fault_free_values_and_clean_records(blas, oracle_mod, ft_mode, M, N, K, pad, alpha, beta):
    tau = blas.ft_default_tau(K)
    *_, st, _ = _run(blas, oracle_mod, M, N, K, alpha, beta, tau, pad=pad, mode=ft_mode)
    assert np.all(st["flag"] == 0) and np.all(st["row"] == -1) and np.all(st["col"] == -1)
    assert st["max_clean_residual"].max() < 0.6 * tau


@pytest.mark.parametrize("fault", [None, (1, 5, 7, 3.0)])
def test_against_the_row_major_call_on_a_transposed_copy(blas, oracle_mod, ft_mode, fault):
    M, N, K = 300, 520, 272
    tau = blas.ft_default_tau(K)
    abuf, bbuf, cbuf, c, st, status = _run(blas, oracle_mod, M, N, K, 1.0, 1.0, tau, faults=[fault] if fault else None, pad=(4, 8, 4),
                                           mode=ft_mode)
    bt = torch.from_numpy(np.ascontiguousarray(bbuf[:, :N].T)).cuda()        # N x K row-major
    dc = torch.from_numpy(cbuf).cuda()
    status2 = blas.ft_status_alloc(N, M)
    ws = torch.full((max(blas.ft_workspace_bytes(N, M, K) // 4, 4),), float("nan"), dtype=torch.float32, device="cuda") if ft_mode == "workspace" else None
    blas.ft_sgemm(N, M, K, bt, torch.from_numpy(abuf).cuda(), dc, 1.0, 1.0, tau=tau, fault=fault, status=status2, ws=ws)
    c2, st2 = dc.cpu().numpy(), blas.ft_status_numpy(status2)
    for f in DECISION_FIELDS:
        assert np.array_equal(st[f], st2[f]), f
    assert np.allclose(st["row_residual"], st2["row_residual"], atol=2e-3) and np.allclose(st["col_residual"], st2["col_residual"], atol=2e-3)
    # same summation order of every element, and a corrected element is computed again in that order
    assert np.array_equal(c2[:, :M], c[:, :M])
    if fault is not None:
        assert st["flag"][1] == 1 and (st["row"][1], st["col"][1]) == (5, 7)


def test_reference_known_answer_plus_one_at_0_1(blas, oracle_mod, ft_mode):
    """The reference's only fault experiment: +1.0 into local element (0, 1) of a tile, threshold 0.1
    (ft_sgemm_huge.cuh:30,40,145) -> located and removed."""
    M, N, K = 256, 512, 256                      # C^T is 512 x 256: two tiles of 256 x 128 down, two across
    for tile in range(4):
        *_, st, _ = _run(blas, oracle_mod, M, N, K, 1.0, 0.0, 0.1, faults=[(tile, 0, 1, 1.0)], mode=ft_mode)
        exp = [0, 0, 0, 0]
        exp[tile] = 1
        assert st["flag"].tolist() == exp
        assert (st["row"][tile], st["col"][tile]) == (0, 1)
        assert abs(st["row_residual"][tile] + 1.0) < 1e-3 and abs(st["col_residual"][tile] + 1.0) < 1e-3


def test_seeded_faults_decisions_equal_cpu_model(blas, oracle_mod, ft_mode):
    M, N, K = 300, 600, 512                       # C^T: 600 x 300 -> 3 x 3 tiles, last row / column of tiles clipped
    tau = blas.ft_default_tau(K)
    rng = np.random.default_rng(17)
    assert blas.ft_num_tiles(N, M) == 9
    for trial in range(12):
        tile = int(rng.integers(9))
        tm = min(blas.FT_TILE_M, N - (tile // 3) * blas.FT_TILE_M)
        tn = min(blas.FT_TILE_N, M - (tile % 3) * blas.FT_TILE_N)
        i, j = int(rng.integers(tm)), int(rng.integers(tn))
        delta = float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-1, 2)))
        abuf, bbuf, cbuf, c, st, _ = _run(blas, oracle_mod, M, N, K, 1.0, 1.0, tau, faults=[(tile, i, j, delta)],
                                          pad=(4, 4, 8), seed=700 + trial, mode=ft_mode)
        # the CPU model on the row-major problem C^T (N x M) = Bt^T (N x K) * At (K x M)
        bt = np.ascontiguousarray(bbuf[:, :N].T)
        c_model = cbuf.copy()
        st_model = oracle_mod.ft_sgemm(N, M, K, bt, K, abuf, abuf.shape[1], c_model, cbuf.shape[1], 1.0, 1.0,
                                       blas.FT_TILE_M, blas.FT_TILE_N, tau, (tile, i, j, delta))
        for f in DECISION_FIELDS:
            assert np.array_equal(st[f], st_model[f]), (trial, f, st[f], st_model[f])
        assert st["flag"][tile] == 1 and (st["row"][tile], st["col"][tile]) == (i, j)


def test_other_classes_granularity_and_cadence(blas, oracle_mod):
    M, N, K = 256, 512, 1024
    tau = blas.ft_default_tau(K)
    *_, st, _ = _run(blas, oracle_mod, M, N, K, 1.0, 0.0, tau, faults=[(0, 3, 4, 2.0)], tile_class=1)
    assert st["flag"][0] == 1 and (st["row"][0], st["col"][0]) == (3, 4)
    *_, st, _ = _run(blas, oracle_mod, M, N, K, 1.0, 0.0, tau, faults=[(1, 3, 4, 2.0)], granularity=blas.FT_GRAN_WAVE)
    assert st["flag"][1] == 1 and (st["row"][1], st["col"][1]) == (3, 4)
    for mode in ("workspace", "fused"):
        *_, st, _ = _run(blas, oracle_mod, M, N, K, 1.0, 0.0, tau, faults=[(0, 3, 4, 2.0, 1)], check_interval=256, mode=mode)
        assert st["flag"][0] == 1 and (st["row"][0], st["col"][0]) == (3, 4)


def test_long_k_and_many_row_groups_in_the_pre_pass(blas, oracle_mod):
    """The pre-pass over the K-major operands with 34 row groups (wave tiles of the 64 x 64 class over the 1085 rows of
    C^T), 2 blocks of 128 columns and 62 blocks of k."""
    M, N, K = 250, 1085, 3900
    tau = blas.ft_default_tau(K)
    *_, st, _ = _run(blas, oracle_mod, M, N, K, 1.0, 1.0, tau, faults=[(41, 3, 4, 2.0)], pad=(4, 8, 4), tile_class=4,
                     granularity=blas.FT_GRAN_WAVE)
    assert np.count_nonzero(st["flag"]) == 1 and st["flag"][41] == 1 and (st["row"][41], st["col"][41]) == (3, 4)
    assert st["max_clean_residual"].max() < 0.6 * tau


@pytest.mark.parametrize("tile_class", [0, 1, 2, 3, 4])
@pytest.mark.parametrize("kind", ["tile-fused", "tile-workspace", "wave-workspace"])
def test_every_class_granularity_and_cadence_equals_the_model(blas, oracle_mod, tile_class, kind):
    """The option matrix on the column-major buffers: every class, both granularities, checksum vectors from the main
    loop or the workspace, with the verification every 256 k and with a single one; decisions equal the CPU model of
    the row-major problem C^T = (B^T)^T A^T, corrected values have the bits of the device's summation order."""
    gran = blas.FT_GRAN_WAVE if kind.startswith("wave") else blas.FT_GRAN_TILE
    cm, cn = blas.ft_check_tile(tile_class, gran)
    M, N, K = 200, 333, 600      # C^T is 333 x 200; 3 verifications (k = 256, 512, 600)
    tau = blas.ft_default_tau(K)
    ntm, ntn = -(-N // cm), -(-M // cn)
    last = ntm * ntn - 1
    rng = np.random.default_rng(90 + tile_class)

    def fault(tile, check):
        tm, tn = min(cm, N - (tile // ntn) * cm), min(cn, M - (tile % ntn) * cn)
        return (tile, int(rng.integers(tm)), int(rng.integers(tn)),
                float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-1.0, 1.5))), check)

    for faults in ([], [fault(last, 0), fault(last, 2)], [fault(0, 1), fault(1, 1), fault(1, 2)], [fault(1, 1), fault(1, 1)]):
        for interval in (256, 0):
            abuf, bbuf, cbuf, c, st, _ = _run(blas, oracle_mod, M, N, K, 1.5, -1.0, tau, faults=faults, pad=(4, 4, 8), seed=1700 + tile_class,
                                              mode="workspace" if kind.endswith("workspace") else "fused", tile_class=tile_class,
                                              granularity=gran, check_interval=interval, no_split=True, values=False)
            bt = np.ascontiguousarray(bbuf[:, :N].T)
            c_model = cbuf.copy()
            st_model = oracle_mod.ft_sgemm_checked(N, M, K, bt, K, abuf, abuf.shape[1], c_model, cbuf.shape[1], 1.5, -1.0,
                                                   cm, cn, tau, interval, faults)
            for f in DECISION_FIELDS:
                assert np.array_equal(st[f], st_model[f]), (tile_class, kind, interval, faults, f, st[f], st_model[f])
            if not np.any(st["flag"] == 2):
                want = cbuf.copy()
                oracle_mod.sgemm_device_order(N, M, K, bt, K, abuf, abuf.shape[1], want, cbuf.shape[1], 1.5, -1.0)
                assert np.array_equal(c[:, :M], want[:, :M]), (tile_class, kind, interval, faults)


def test_workspace_rules(blas, oracle_mod):
    from hpcdeepneuralnetworks_amd.blas import HpcdnnError
    M, N, K = 200, 300, 128
    abuf, bbuf, cbuf = _buffers(oracle_mod, M, N, K, (0, 0, 0), 800)
    da, db = torch.from_numpy(abuf).cuda(), torch.from_numpy(bbuf).cuda()
    with pytest.raises(HpcdnnError):   # a workspace too small for the checksum vectors is an error, not a silent fallback
        blas.ft_sgemm_cm_nt(M, N, K, da, db, torch.from_numpy(cbuf).cuda(), 1.0, 0.0, torch.empty(64, device="cuda"))
    with pytest.raises(HpcdnnError):   # wave-tile checksums come from the pre-pass
        blas.ft_sgemm_cm_nt(M, N, K, da, db, torch.from_numpy(cbuf).cuda(), 1.0, 0.0, None, granularity=blas.FT_GRAN_WAVE)
    # K = 0: C = beta * C, nothing else needed
    dc = torch.full((N, M), 2.0, device="cuda")
    blas.ft_sgemm_cm_nt(M, N, 0, da, db, dc, 1.0, 0.5, None)
    assert torch.equal(dc, torch.full((N, M), 1.0, device="cuda"))


@pytest.mark.parametrize("tile_class", [0, 1, 2, 3, 4])
def test_every_tile_class_on_a_ragged_problem(blas, oracle_mod, ft_mode, tile_class):
    """Ragged in M, N and K with padded leading dimensions: the columns m >= M of the K-major operand (the next row
    or NaN padding) must not reach the column checksums.  One seeded fault per class, located and corrected."""
    M, N, K = 333, 270, 203
    tau = blas.ft_default_tau(K)
    *_, st, _ = _run(blas, oracle_mod, M, N, K, 1.0, -1.5, tau, faults=[(0, 9, 3, -4.0)], pad=(5, 2, 3), tile_class=tile_class, mode=ft_mode)
    assert st["flag"][0] == 1 and (st["row"][0], st["col"][0]) == (9, 3)
    assert np.all(st["flag"][1:] == 0)
