"""Pins the CPU oracle against independent routines (numpy float64, exact rationals, closed forms).

The reference holds no golden vectors for this path, so every check here is
chosen so that a plausible slip in oracle.c (dropped term, transposed operand,
wrong sign or index) fails it.
"""
from fractions import Fraction

import numpy as np
import pytest


def _round_f32(fr: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) float32 of an exact rational."""
    if fr == 0:
        return np.float32(0.0)
    guess = np.float32(float(fr))
    cands = {guess, np.nextafter(guess, np.float32(np.inf)), np.nextafter(guess, np.float32(-np.inf))}
    best = None
    for c in cands:
        d = abs(Fraction(float(c)) - fr)
        key = (d, int(np.float32(c).view(np.uint32)) & 1)  # ties -> even mantissa
        if best is None or key < best[0]:
            best = (key, c)
    return np.float32(best[1])


def test_rng_range_grid_and_independence(oracle_mod):
    v = oracle_mod.fill_uniform(1 << 16, seed=7)
    assert v.dtype == np.float32 and v.min() >= -1.0 and v.max() < 1.0
    # values sit on the 2^-23 grid
    assert np.all(v * 8388608.0 == np.round(v * 8388608.0))
    # first two moments of uniform[-1,1): mean 0, var 1/3
    assert abs(float(v.mean())) < 0.01 and abs(float(v.var()) - 1.0 / 3.0) < 0.01
    w = oracle_mod.fill_uniform(1 << 16, seed=8)
    assert abs(float(np.corrcoef(v, w)[0, 1])) < 0.02
    assert abs(float(np.corrcoef(v[:-1], v[1:])[0, 1])) < 0.02
    # scalar accessor and vector fill agree, counter = index
    assert oracle_mod.uniform(7, 12345) == float(v[12345])


def test_rng_matrix_ignores_leading_dimension(oracle_mod):
    a = oracle_mod.fill_uniform_matrix(5, 7, seed=3)
    b = oracle_mod.fill_uniform_matrix(5, 7, seed=3, ld=11)
    assert np.array_equal(a, b[:, :7]) and np.all(np.isnan(b[:, 7:]))
    assert np.array_equal(a.ravel(), oracle_mod.fill_uniform(35, seed=3))


def test_cpu_gemm_matches_numpy_float64(oracle_mod):
    n = 96
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    b = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    c0 = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    for alpha, beta in [(1.0, 0.0), (1.5, -1.0), (1.0, -1.5), (0.0, 2.0)]:
        c = c0.copy()
        oracle_mod.cpu_gemm(alpha, beta, a, b, n, c)
        ref = alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0.astype(np.float64)
        assert np.max(np.abs(c - ref)) < 5e-5, (alpha, beta)


def test_cpu_gemm_is_not_transposed(oracle_mod):
    # A = permutation-like matrix picks rows of B: C = A@B exactly; A^T@B or B@A would differ
    n = 8
    a = np.zeros((n, n), dtype=np.float32)
    for i in range(n):
        a[i, (3 * i + 1) % n] = 1.0
    b = np.arange(n * n, dtype=np.float32).reshape(n, n)
    c = np.zeros((n, n), dtype=np.float32)
    oracle_mod.cpu_gemm(1.0, 0.0, a, b, n, c)
    assert np.array_equal(c, b[[(3 * i + 1) % n for i in range(n)], :])


def test_cpu_gemm_float_accumulator_order(oracle_mod):
    # float accumulate, k ascending: 2^24 + 1 + 1 stays 2^24 in float, in double it would be 2^24+2
    n = 4
    a = np.zeros((n, n), dtype=np.float32)
    b = np.zeros((n, n), dtype=np.float32)
    a[0, :3] = [16777216.0, 1.0, 1.0]
    b[:3, 0] = 1.0
    c = np.zeros((n, n), dtype=np.float32)
    oracle_mod.cpu_gemm(1.0, 0.0, a, b, n, c)
    assert c[0, 0] == np.float32(16777216.0)


@pytest.mark.parametrize("M,N,K,lda,ldb,ldc", [(17, 9, 33, 40, 12, 10), (32, 32, 32, 32, 32, 32), (1, 1, 1, 1, 1, 1)])
def test_gemm_f64_rows_matches_numpy(oracle_mod, M, N, K, lda, ldb, ldc):
    rng = np.random.default_rng(1)
    a = np.full((M, lda), np.nan, np.float32)
    b = np.full((K, ldb), np.nan, np.float32)
    c0 = np.full((M, ldc), np.nan, np.float32)
    a[:, :K] = rng.uniform(-1, 1, (M, K))
    b[:, :N] = rng.uniform(-1, 1, (K, N))
    c0[:, :N] = rng.uniform(-1, 1, (M, N))
    alpha, beta = 1.5, -0.5
    ref, den = oracle_mod.gemm_f64_rows(M, N, K, a, lda, b, ldb, c0, ldc, alpha, beta)
    a64, b64, c64 = a[:, :K].astype(np.float64), b[:, :N].astype(np.float64), c0[:, :N].astype(np.float64)
    assert np.allclose(ref, alpha * (a64 @ b64) + beta * c64, rtol=0, atol=1e-12)
    assert np.allclose(den, abs(alpha) * (np.abs(a64) @ np.abs(b64)) + abs(beta) * np.abs(c64), rtol=0, atol=1e-12)
    rows = [M - 1, 0]
    ref2, den2 = oracle_mod.gemm_f64_rows(M, N, K, a, lda, b, ldb, c0, ldc, alpha, beta, rows=rows)
    assert np.array_equal(ref2, ref[rows]) and np.array_equal(den2, den[rows])


@pytest.mark.parametrize("M,N,K,lda,ldb,ldc", [(17, 9, 33, 20, 12, 19), (8, 24, 5, 8, 24, 8), (1, 1, 1, 1, 1, 1)])
def test_gemm_cm_nt_matches_numpy_on_column_major_views(oracle_mod, M, N, K, lda, ldb, ldc):
    """The column-major A*B^T of the reference's ft_sgemm family (kernel/ft_sgemm/sgemm.cu:111) against numpy float64 on
    Fortran-ordered views of the same buffers, leading dimensions padded with NaN."""
    rng = np.random.default_rng(4)
    abuf = np.full((K, lda), np.nan, np.float32)   # column k of A is row k of the buffer
    bbuf = np.full((K, ldb), np.nan, np.float32)
    cbuf = np.full((N, ldc), np.nan, np.float32)
    abuf[:, :M] = rng.uniform(-1, 1, (K, M))
    bbuf[:, :N] = rng.uniform(-1, 1, (K, N))
    cbuf[:, :M] = rng.uniform(-1, 1, (N, M))
    A = np.ndarray((M, K), np.float32, abuf, strides=(4, 4 * lda)).astype(np.float64)   # A[m, k] = buffer[m + k*lda]
    B = np.ndarray((N, K), np.float32, bbuf, strides=(4, 4 * ldb)).astype(np.float64)
    C0 = np.ndarray((M, N), np.float32, cbuf, strides=(4, 4 * ldc)).astype(np.float64)
    alpha, beta = 1.5, -0.5
    ref, den = oracle_mod.gemm_cm_nt_f64(M, N, K, abuf, lda, bbuf, ldb, cbuf, ldc, alpha, beta)
    want = alpha * (A @ B.T) + beta * C0                                               # M x N
    assert np.allclose(ref.T, want, rtol=0, atol=1e-12)                                 # ref holds it column-major
    assert np.allclose(den.T, abs(alpha) * (np.abs(A) @ np.abs(B).T) + abs(beta) * np.abs(C0), rtol=0, atol=1e-12)


def test_gemm_cm_nt_hand_case_fails_every_transposition_mistake(oracle_mod):
    """A = [[1,2],[3,4],[5,6]] (3 x 2), B = [[1,0],[0,1],[1,1],[2,0]] (4 x 2): A*B^T = [[1,2,3,2],[3,4,7,6],[5,6,11,10]].
    A*B is not even defined, A^T, B untransposed or a row-major C give other numbers."""
    A = np.array([[1, 2], [3, 4], [5, 6]], np.float32)
    B = np.array([[1, 0], [0, 1], [1, 1], [2, 0]], np.float32)
    abuf = np.asfortranarray(A).ravel(order="K")   # column-major memory
    bbuf = np.asfortranarray(B).ravel(order="K")
    ref, _ = oracle_mod.gemm_cm_nt_f64(3, 4, 2, abuf, 3, bbuf, 4, None, 3, 1.0, 0.0)
    want = np.array([[1, 2, 3, 2], [3, 4, 7, 6], [5, 6, 11, 10]], np.float64)
    assert np.array_equal(ref, want.T)                                                  # memory order: column by column
    assert np.array_equal(ref.ravel(), [1, 3, 5, 2, 4, 6, 3, 7, 11, 2, 6, 10])


def test_gemm_max_err_is_the_componentwise_criterion(oracle_mod):
    M = N = 4
    ref = np.ones((M, N))
    den = np.full((M, N), 2.0)
    c = np.ones((M, 6), dtype=np.float32)
    assert oracle_mod.gemm_max_err(N, c, 6, ref, den) == 0.0
    c[2, 3] = 1.5
    assert oracle_mod.gemm_max_err(N, c, 6, ref, den) == pytest.approx(0.25)
    c[1, 1] = np.nan
    assert not (oracle_mod.gemm_max_err(N, c, 6, ref, den) <= 1.0)  # NaN is never accepted


def test_saxpy_is_one_fused_multiply_add(oracle_mod):
    rng = np.random.default_rng(2)
    n = 2000
    x = rng.uniform(-1, 1, n).astype(np.float32)
    y0 = rng.uniform(-1, 1, n).astype(np.float32)
    alpha = np.float32(2.5)
    y = y0.copy()
    oracle_mod.saxpy(float(alpha), x, y)
    exact = [_round_f32(Fraction(float(alpha)) * Fraction(float(xi)) + Fraction(float(yi))) for xi, yi in zip(x, y0)]
    assert np.array_equal(y, np.array(exact, dtype=np.float32))


def test_saxpy_differs_from_unfused_where_it_must(oracle_mod):
    # a*x rounds in float when unfused; the fused result keeps the low bits: (1+2^-12)^2 - 1
    a = np.float32(1.0 + 2.0**-12)
    x = np.array([a], dtype=np.float32)
    y = np.array([-1.0], dtype=np.float32)
    oracle_mod.saxpy(float(a), x, y)
    assert float(y[0]) == 2.0**-11 + 2.0**-24
    assert np.float32(np.float32(a * a) + np.float32(-1.0)) != y[0]


def test_threaded_saxpy_and_serial_sdot_are_the_same_functions(oracle_mod):
    """The two extra CPU baselines of the benchmark: SAXPY on the OpenMP pool has the bits of the one-thread loop, the
    one-thread double-accumulated dot product agrees with numpy and with the OpenMP form to double rounding."""
    n = (1 << 16) + 7
    x, y = oracle_mod.fill_uniform(n, 5), oracle_mod.fill_uniform(n, 6)
    y1, y2 = y.copy(), y.copy()
    oracle_mod.saxpy(2.5, x, y1)
    oracle_mod.saxpy_omp(2.5, x, y2)
    assert np.array_equal(y1, y2) and not np.array_equal(y1, y)
    want = float(np.dot(x.astype(np.float64), y.astype(np.float64)))
    assert oracle_mod.sdot_f64_serial(x, y) == pytest.approx(want, rel=1e-13, abs=1e-12)
    assert oracle_mod.sdot_f64(x, y) == pytest.approx(oracle_mod.sdot_f64_serial(x, y), rel=1e-13, abs=1e-12)
    assert oracle_mod.sdot_f64_serial(np.array([3.0, 4.0], np.float32), np.array([5.0, -2.0], np.float32)) == 7.0
    assert oracle_mod.sdot_f64_serial(x[:0], y[:0]) == 0.0


def test_sdot_f64_and_f32(oracle_mod):
    rng = np.random.default_rng(3)
    n = 100003
    x = rng.uniform(-1, 1, n).astype(np.float32)
    y = rng.uniform(-1, 1, n).astype(np.float32)
    exact = float(np.dot(x.astype(np.float64), y.astype(np.float64)))
    assert oracle_mod.sdot_f64(x, y) == pytest.approx(exact, rel=0, abs=1e-9)
    assert oracle_mod.sdot_f32(x, y) == pytest.approx(exact, rel=0, abs=0.05)
    # closed forms
    ones = np.ones(1 << 12, dtype=np.float32)
    assert oracle_mod.sdot_f64(ones, ones) == 4096.0 and oracle_mod.sdot_f32(ones, ones) == 4096.0
    k = np.arange(1, 101, dtype=np.float32)
    assert oracle_mod.sdot_f64(k, k) == 338350.0  # sum k^2
    assert oracle_mod.sdot_f64(x[:0], y[:0]) == 0.0


def _tile_problem(tm, tn, K, seed):
    rng = np.random.default_rng(seed)
    a = rng.uniform(-1, 1, (tm, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (K, tn)).astype(np.float32)
    acc = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    return a, b, acc


def test_abft_residuals_follow_the_checksum_algebra(oracle_mod):
    tm, tn, K = 24, 16, 40
    a, b, acc = _tile_problem(tm, tn, K, 4)
    dr, dc = oracle_mod.abft_residuals(a, K, b, tn, acc, tn, tm, tn, K)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    # e^T(AB) = (e^T A)B and (AB)e = A(Be), each computed the "other" way round
    cr_ref = (a64 @ b64).sum(axis=1)
    cc_ref = (a64 @ b64).sum(axis=0)
    assert np.allclose(dr, cr_ref - acc.astype(np.float64).sum(axis=1), atol=1e-10)
    assert np.allclose(dc, cc_ref - acc.astype(np.float64).sum(axis=0), atol=1e-10)
    assert np.max(np.abs(dr)) < 1e-4 and np.max(np.abs(dc)) < 1e-4  # fault-free: rounding only
    # a fault of +delta at (i,j) shows up as -delta in row i and column j only (sign: reference - observed)
    acc2 = acc.copy()
    acc2[5, 9] += np.float32(0.75)
    dr2, dc2 = oracle_mod.abft_residuals(a, K, b, tn, acc2, tn, tm, tn, K)
    assert abs(dr2[5] + 0.75) < 1e-4 and abs(dc2[9] + 0.75) < 1e-4
    mask_r = np.ones(tm, bool); mask_r[5] = False
    mask_c = np.ones(tn, bool); mask_c[9] = False
    assert np.array_equal(dr2[mask_r], dr[mask_r]) and np.array_equal(dc2[mask_c], dc[mask_c])


def test_abft_residuals_not_transposed_for_rectangular_tiles(oracle_mod):
    # rows and columns carry different checksums: make A's rows distinguishable from B's columns
    tm, tn, K = 3, 5, 2
    a = np.array([[1, 0], [0, 1], [2, 2]], dtype=np.float32)
    b = np.array([[1, 2, 3, 4, 5], [10, 20, 30, 40, 50]], dtype=np.float32)
    acc = np.zeros((tm, tn), dtype=np.float32)  # observed = 0 -> residual = reference checksum
    dr, dc = oracle_mod.abft_residuals(a, K, b, tn, acc, tn, tm, tn, K)
    assert dr.tolist() == [15.0, 150.0, 330.0]
    assert dc.tolist() == [33.0, 66.0, 99.0, 132.0, 165.0]  # column sums of A@B


def test_abft_reference_checksums_and_observe_are_the_two_halves_of_the_residuals(oracle_mod):
    """abft_reference_checksums ((e^T A)B and A(Be), through the operands) and abft_observe (reference minus the line
    sums of the accumulators) are what the device campaign calls separately: the first against numpy FP64 on a
    rectangular, padded case that a transposed operand or a swapped output would fail, the second on hand values, and
    the pair against abft_residuals."""
    tm, tn, K, lda, ldb = 5, 7, 11, 13, 9
    rng = np.random.default_rng(77)
    a = rng.standard_normal((tm, lda)).astype(np.float32)
    b = rng.standard_normal((K, ldb)).astype(np.float32)
    a[:, K:] = np.nan   # padding is never read
    b[:, tn:] = np.nan
    cr, cc = oracle_mod.abft_reference_checksums(a, lda, b, ldb, tm, tn, K)
    a64, b64 = a[:, :K].astype(np.float64), b[:, :tn].astype(np.float64)
    assert cr.shape == (tm,) and cc.shape == (tn,)
    assert np.allclose(cr, a64 @ b64.sum(axis=1), rtol=0, atol=1e-12)
    assert np.allclose(cc, a64.sum(axis=0) @ b64, rtol=0, atol=1e-12)
    # observe: residual = reference - observed line sum, rows and columns kept apart, padded accumulator rows
    acc = np.full((3, 6), np.nan, dtype=np.float32)
    acc[:, :4] = np.array([[1, 2, 3, 4], [10, 20, 30, 40], [0.5, 0.25, 0.125, 0]], dtype=np.float32)
    dr, dc = oracle_mod.abft_observe(acc, 6, np.array([10.0, 90.0, 1.0]), np.array([11.5, 22.25, 33.0, 50.0]))
    assert dr.tolist() == [0.0, -10.0, 0.125]
    assert dc.tolist() == [0.0, 0.0, -0.125, 6.0]
    # the composition is abft_residuals
    acc2 = (a64 @ b64).astype(np.float32)
    dr2, dc2 = oracle_mod.abft_observe(acc2, tn, cr, cc)
    dr3, dc3 = oracle_mod.abft_residuals(a, lda, b, ldb, acc2, tn, tm, tn, K)
    assert np.array_equal(dr2, dr3) and np.array_equal(dc2, dc3)


def test_num_threads_reports_the_openmp_pool(oracle_mod):
    import os
    assert 1 <= oracle_mod.num_threads() <= max(os.cpu_count(), 1) * 4


def test_abft_reference_known_answer(oracle_mod):
    """The one case the reference holds: +1.0 at tile-local (m=0, n=1) of a 128x128 tile, threshold 0.1
    -> row 0 and column 1 flagged, magnitude 1 removed (ft_sgemm_huge.cuh:40,145,263,358)."""
    tm = tn = 128
    K = 256
    a, b, acc = _tile_problem(tm, tn, K, 5)
    acc[0, 1] += np.float32(1.0)
    dr, dc = oracle_mod.abft_residuals(a, K, b, tn, acc, tn, tm, tn, K)
    st, fix = oracle_mod.abft_decide(dr, dc, 0.1)
    assert (st["flag"], st["row"], st["col"], st["n_bad_rows"], st["n_bad_cols"]) == (1, 0, 1, 1, 1)
    assert round(-fix) == 1 and abs(fix + 1.0) < 1e-3  # the reference subtracts round(|residual|) = 1
    assert st["max_clean_residual"] < 0.1


def test_abft_decide_cases(oracle_mod):
    tm, tn = 6, 4
    z_r, z_c = np.zeros(tm), np.zeros(tn)
    st, fix = oracle_mod.abft_decide(z_r, z_c, 0.01)
    assert st["flag"] == 0 and fix == 0.0 and st["row"] == -1 and st["col"] == -1
    # below threshold -> clean, recorded as the largest clean residual (of the columns: they are the screen)
    c = z_c.copy(); c[2] = -0.009
    st, fix = oracle_mod.abft_decide(z_r, c, 0.01)
    assert st["flag"] == 0 and st["max_clean_residual"] == pytest.approx(0.009)
    # exactly at the threshold is clean (strict >), as in the reference (fabsf(x) > err_bound)
    c[2] = float(np.float32(0.01))
    assert oracle_mod.abft_decide(z_r, c, np.float32(0.01))[0]["flag"] == 0
    # single fault: correction is the signed row residual
    r = z_r.copy(); c = z_c.copy(); r[4] = -0.5; c[1] = -0.5001
    st, fix = oracle_mod.abft_decide(r, c, 0.01)
    assert (st["flag"], st["row"], st["col"]) == (1, 4, 1) and fix == pytest.approx(-0.5)
    assert st["row_residual"] == pytest.approx(-0.5) and st["col_residual"] == pytest.approx(-0.5001)
    # the columns screen, as in the reference, which acts only when a column AND a row disagree
    # (ft_sgemm_huge.cuh:289): a row without any column is not looked at - not flagged, not counted, and not part of
    # the largest clean residual either
    st, fix = oracle_mod.abft_decide(r, z_c, 0.01)
    assert st["flag"] == 0 and fix == 0.0 and (st["n_bad_rows"], st["n_bad_cols"]) == (0, 0) and st["max_clean_residual"] == 0.0
    # column without row, two rows, or two columns: detected but not correctable
    st, fix = oracle_mod.abft_decide(z_r, c, 0.01)
    assert st["flag"] == 2 and fix == 0.0 and (st["n_bad_rows"], st["n_bad_cols"]) == (0, 1)
    r[0] = 0.3
    st, _ = oracle_mod.abft_decide(r, c, 0.01)
    assert st["flag"] == 2 and (st["n_bad_rows"], st["n_bad_cols"]) == (2, 1)
    c[3] = 0.3
    r[0] = 0.0
    st, _ = oracle_mod.abft_decide(r, c, 0.01)
    assert st["flag"] == 2 and (st["n_bad_rows"], st["n_bad_cols"]) == (1, 2)


def test_tile_acc_matches_numpy_on_a_padded_rectangular_tile(oracle_mod):
    """The accumulator model of the fault campaigns: float accumulators, one fused multiply-add per k, k ascending."""
    tm, tn, K, lda, ldb = 7, 5, 96, 101, 9
    a = oracle_mod.fill_uniform_matrix(tm, K, 41, ld=lda)   # NaN padding: a wrong stride or an over-read shows
    b = oracle_mod.fill_uniform_matrix(K, tn, 42, ld=ldb)
    acc = oracle_mod.tile_acc(a, lda, b, ldb, tm, tn, K)
    ref = a[:, :K].astype(np.float64) @ b[:, :tn].astype(np.float64)
    assert acc.shape == (tm, tn) and acc.dtype == np.float32
    assert np.max(np.abs(acc - ref)) < 4e-6          # float rounding of a 96-term sum of products below 1
    # a sub-block of a larger matrix: pointer + leading dimension select it
    big_a = oracle_mod.fill_uniform_matrix(16, K, 43)
    big_b = oracle_mod.fill_uniform_matrix(K, 24, 44)
    sub = oracle_mod.tile_acc(big_a[8:], K, big_b[:, 16:], 24, 8, 8, K)
    want = big_a[8:].astype(np.float64) @ big_b[:, 16:].astype(np.float64)
    assert np.max(np.abs(sub - want)) < 4e-6


def test_tile_acc_is_not_transposed_and_keeps_float_fma_order(oracle_mod):
    # rectangular hand case: a transposed operand or swapped tm/tn cannot give this
    a = np.array([[1, 2, 3], [4, 5, 6]], dtype=np.float32)                    # 2 x 3
    b = np.array([[1, 0, 2, 0], [0, 1, 0, 2], [1, 1, 1, 1]], dtype=np.float32)  # 3 x 4
    acc = oracle_mod.tile_acc(a, 3, b, 4, 2, 4, 3)
    assert acc.tolist() == [[4.0, 5.0, 5.0, 7.0], [10.0, 11.0, 14.0, 16.0]]
    # float accumulator, k ascending: 2^24 + 1 + 1 stays 2^24 (a double accumulator, or k descending, gives 2^24 + 2)
    a = np.array([[16777216.0, 1.0, 1.0]], dtype=np.float32)
    b = np.ones((3, 1), dtype=np.float32)
    assert oracle_mod.tile_acc(a, 3, b, 1, 1, 1, 3)[0, 0] == np.float32(16777216.0)
    a = np.array([[1.0, 1.0, 16777216.0]], dtype=np.float32)
    assert oracle_mod.tile_acc(a, 3, b, 1, 1, 1, 3)[0, 0] == np.float32(16777218.0)
    # fused: (1 + 2^-12)^2 - 1 keeps the 2^-24 term that a rounded product loses
    h = np.float32(1.0 + 2.0**-12)
    a = np.array([[-1.0, h]], dtype=np.float32)
    b = np.array([[1.0], [h]], dtype=np.float32)
    assert float(oracle_mod.tile_acc(a, 2, b, 1, 1, 1, 2)[0, 0]) == 2.0**-11 + 2.0**-24


def test_decide_lines_uses_each_lines_own_threshold(oracle_mod):
    tm, tn = 5, 4
    dr, dc = np.zeros(tm), np.zeros(tn)
    tau_r = np.array([1.0, 0.1, 1.0, 0.01, 1.0])
    tau_c = np.array([0.5, 0.05, 0.5, 0.5])
    # 0.2 is above column 1's threshold but below its neighbours'; the same residual in column 2 is clean
    dc[1] = -0.2
    st, fix = oracle_mod.abft_decide_lines(dr, dc, tau_r, tau_c)
    assert (st["flag"], st["n_bad_rows"], st["n_bad_cols"]) == (2, 0, 1) and fix == 0.0
    dc[:] = 0.0
    dc[2] = -0.2
    st, fix = oracle_mod.abft_decide_lines(dr, dc, tau_r, tau_c)
    assert st["flag"] == 0 and st["max_clean_residual"] == pytest.approx(0.2)
    # with a flagged column the rows get their own thresholds: 0.2 flags row 1 (0.1) and is clean in row 2 (1.0)
    dc[:] = [0.0, -0.2, 0.0, 0.0]
    dr[:] = [0.0, 0.0, -0.2, 0.0, 0.0]
    st, fix = oracle_mod.abft_decide_lines(dr, dc, tau_r, tau_c)
    assert (st["flag"], st["n_bad_rows"], st["n_bad_cols"]) == (2, 0, 1) and st["max_clean_residual"] == pytest.approx(0.2)
    dr[:] = [0.0, -0.2, 0.0, 0.0, 0.0]
    st, fix = oracle_mod.abft_decide_lines(dr, dc, tau_r, tau_c)
    assert (st["flag"], st["row"], st["col"]) == (1, 1, 1)
    # row 1 and column 1 flagged by their own thresholds, the equally large residuals of row 0 / column 0 are clean
    dr[:] = [0.2, -0.2, 0.0, 0.0, 0.0]
    dc[:] = [0.2, -0.21, 0.0, 0.0]
    st, fix = oracle_mod.abft_decide_lines(dr, dc, tau_r, tau_c)
    assert (st["flag"], st["row"], st["col"], st["n_bad_rows"], st["n_bad_cols"]) == (1, 1, 1, 1, 1)
    assert fix == pytest.approx(-0.2) and st["col_residual"] == pytest.approx(-0.21)
    assert st["max_clean_residual"] == pytest.approx(0.2)
    # rows and columns are not mixed up: tau_c applied to rows would flag row 0 too (0.2 > 0.05 is column 1's threshold)
    st, _ = oracle_mod.abft_decide_lines(dr, dc, tau_r, np.array([0.1, 0.05, 0.5, 0.5]))
    assert (st["flag"], st["n_bad_rows"], st["n_bad_cols"]) == (2, 1, 2)
    # the uniform form is the special case
    st_u, fix_u = oracle_mod.abft_decide(dr, dc, 0.1)
    st_l, fix_l = oracle_mod.abft_decide_lines(dr, dc, np.full(tm, np.float32(0.1), np.float64), np.full(tn, np.float32(0.1), np.float64))
    assert st_u == st_l and fix_u == fix_l


def test_rows_as_the_screen_is_the_same_rule_with_the_sides_exchanged(oracle_mod):
    """The rule for products one tile wide: rows first, columns only when a row is flagged.  Pinned by symmetry (the
    decision on (dr, dc) with the rows as the screen is the decision on (dc, dr) with the columns as the screen, rows
    and columns renamed) and by the patterns that tell the two screens apart."""
    rng = np.random.default_rng(7)
    for _ in range(200):
        tm, tn = int(rng.integers(1, 7)), int(rng.integers(1, 7))
        dr = np.where(rng.random(tm) < 0.25, rng.normal(size=tm), 0.0)
        dc = np.where(rng.random(tn) < 0.25, rng.normal(size=tn), 0.0)
        tau_r, tau_c = rng.uniform(0.05, 0.5, tm), rng.uniform(0.05, 0.5, tn)
        with oracle_mod.rows_screen():
            st, fix = oracle_mod.abft_decide_lines(dr, dc, tau_r, tau_c)
        sw, _ = oracle_mod.abft_decide_lines(dc, dr, tau_c, tau_r)     # columns as the screen, sides exchanged
        assert (st["flag"], st["n_bad_rows"], st["n_bad_cols"], st["row"], st["col"]) == \
               (sw["flag"], sw["n_bad_cols"], sw["n_bad_rows"], sw["col"], sw["row"])
        assert st["max_clean_residual"] == sw["max_clean_residual"]
        assert st["row_residual"] == sw["col_residual"] and st["col_residual"] == sw["row_residual"]
        assert fix == st["row_residual"]
    # a residual pattern in the columns only: unseen with the rows as the screen, "detected" with the columns
    dr, dc, t = np.zeros(4), np.array([0.0, 1.0, -1.0]), np.full(4, 0.1)
    with oracle_mod.rows_screen():
        st, _ = oracle_mod.abft_decide_lines(dr, dc, t, t[:3])
    assert (st["flag"], st["n_bad_rows"], st["n_bad_cols"], st["max_clean_residual"]) == (0, 0, 0, 0.0)
    st, _ = oracle_mod.abft_decide_lines(dr, dc, t, t[:3])
    assert (st["flag"], st["n_bad_rows"], st["n_bad_cols"]) == (2, 0, 2)
    # and the selector does not outlive the block
    st, _ = oracle_mod.abft_decide_lines(np.array([1.0, 0.0, 0.0, 0.0]), np.zeros(3), t, t[:3])
    assert st["flag"] == 0


def _numpy_relative_decision(acc, cr_ref, cc_ref, K):
    """The data-scaled decision of one tile composed in numpy: thresholds rel * sqrt(n) * max(line mean |acc|, tile
    mean |acc|) with rel = 2.56e-7 * sqrt(max(K, 64)), residual = reference - line sum, strict comparison."""
    tm, tn = acc.shape
    a64 = np.abs(acc.astype(np.float64))
    rel = 2.56e-7 * np.sqrt(max(K, 64))
    tau_r = rel * np.sqrt(tn) * np.maximum(a64.mean(axis=1), a64.mean())
    tau_c = rel * np.sqrt(tm) * np.maximum(a64.mean(axis=0), a64.mean())
    dr = cr_ref - acc.astype(np.float64).sum(axis=1)
    dc = cc_ref - acc.astype(np.float64).sum(axis=0)
    bad_r, bad_c = np.flatnonzero(np.abs(dr) > tau_r), np.flatnonzero(np.abs(dc) > tau_c)
    if len(bad_r) == 0 and len(bad_c) == 0:
        flag = 0
    elif len(bad_r) == 1 and len(bad_c) == 1:
        flag = 1
    else:
        flag = 2
    return flag, bad_r, bad_c, tau_r, tau_c, dr, dc


@pytest.mark.parametrize("fault_tile", [None, 0, 1, 4, 5])
@pytest.mark.parametrize("level", ["below both", "between", "above both"])
def test_ft_sgemm_model_with_data_scaled_threshold_against_numpy_composition(oracle_mod, fault_tile, level):
    """oracle_ft_sgemm with tau = -1 on a ragged 3 x 2 tile problem, against the same pipeline composed in numpy
    (float64 accumulators are exact here: small-integer operands, so the fault-free residuals are exactly zero and
    the decision depends only on how the thresholds are composed: clipped tile extents, line mean against tile
    mean, rows against columns).  The fault is sized relative to the two thresholds of its row and column."""
    M, N, K, tm, tn = 20, 12, 70, 8, 8   # tiles: rows 8, 8, 4; columns 8, 4
    rng = np.random.default_rng(17)
    a = rng.integers(-8, 9, (M, K)).astype(np.float32)
    b = rng.integers(-8, 9, (K, N)).astype(np.float32)
    exact = a.astype(np.float64) @ b.astype(np.float64)
    assert np.abs(exact).max() < 2**20   # every partial sum is an exact float
    ntn = 2
    fault = None
    if fault_tile is not None:
        bm, bn = fault_tile // ntn, fault_tile % ntn
        h, w = min(tm, M - bm * tm), min(tn, N - bn * tn)
        blk = exact[bm * tm:bm * tm + h, bn * tn:bn * tn + w].astype(np.float32)
        # thresholds barely move with the fault (it is far below the accumulators): size it from the fault-free ones
        _, _, _, tau_r, tau_c, _, _ = _numpy_relative_decision(blk, blk.astype(np.float64).sum(axis=1), blk.astype(np.float64).sum(axis=0), K)
        # the row with the largest and the column with the smallest threshold: they differ, so a fault can sit between
        i, j = int(np.argmax(tau_r)), int(np.argmin(tau_c))
        lo, hi = sorted((tau_r[i], tau_c[j]))
        assert hi > 1.15 * lo, "row and column thresholds must differ for the in-between case to exist"
        delta = {"below both": 0.85 * lo, "between": 0.5 * (lo + hi), "above both": 1.15 * hi}[level]
        fault = (fault_tile, i, j, float(np.float32(-delta)))
    elif level != "below both":
        pytest.skip("no fault: one case is enough")
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, -1.0, fault)
    for t in range(6):
        bm, bn = t // ntn, t % ntn
        h, w = min(tm, M - bm * tm), min(tn, N - bn * tn)
        blk64 = exact[bm * tm:bm * tm + h, bn * tn:bn * tn + w]
        acc = blk64.astype(np.float32)
        if fault is not None and t == fault[0]:
            acc[fault[1], fault[2]] += np.float32(fault[3])
        flag, bad_r, bad_c, tau_r, tau_c, dr, dc = _numpy_relative_decision(acc, blk64.sum(axis=1), blk64.sum(axis=0), K)
        # the sized fault keeps a clear distance from both thresholds, so float rounding of the thresholds cannot flip it
        for d, tau in ((dr, tau_r), (dc, tau_c)):
            assert np.all(np.abs(np.abs(d) - tau) > 0.05 * tau)
        assert st["flag"][t] == flag, (t, level)
        assert (st["n_bad_rows"][t], st["n_bad_cols"][t]) == (len(bad_r), len(bad_c)), (t, level)
        if flag == 1:
            assert (st["row"][t], st["col"][t]) == (bad_r[0], bad_c[0])
            assert st["row_residual"][t] == np.float32(dr[bad_r[0]])
        else:
            assert (st["row"][t], st["col"][t]) == (-1, -1)
    if fault is not None:
        want = {"below both": 0, "between": 2, "above both": 1}[level]
        assert st["flag"][fault[0]] == want and np.count_nonzero(st["flag"]) == (want != 0)
        if want == 1:   # corrected: C is the exact product again
            assert np.array_equal(c, exact.astype(np.float32))


@pytest.mark.parametrize("fault", [None, (1, 3, 2, 0.5), (2, 7, 0, -20.0)])
def test_ft_sgemm_model_detects_and_corrects(oracle_mod, fault):
    M, N, K, tm, tn = 20, 12, 64, 8, 8   # 3 x 2 tiles, ragged in both directions
    rng = np.random.default_rng(6)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    c0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    c = c0.copy()
    st = oracle_mod.ft_sgemm(M, N, K, a, K, b, N, c, N, 1.0, 1.0, tm, tn, 1e-3, fault)
    ref = a.astype(np.float64) @ b.astype(np.float64) + c0
    assert np.max(np.abs(c - ref)) < 1e-4  # corrected output equals the fault-free product
    flags = st["flag"].tolist()
    if fault is None:
        assert flags == [0] * 6
    else:
        exp = [0] * 6
        exp[fault[0]] = 1
        assert flags == exp
        assert (st["row"][fault[0]], st["col"][fault[0]]) == (fault[1], fault[2])
        assert st["row_residual"][fault[0]] == pytest.approx(-fault[3], abs=1e-4)


@pytest.mark.parametrize("delta", [50.0, -50.0, 1e-2, -3.0e4])
def test_corrected_product_has_the_bits_of_the_fault_free_one(oracle_mod, delta):
    """The correction computes the located accumulator again instead of adding the residual back: with K = 1 (where a
    residual of a whole row of products carries the most noise relative to one element) and with a longer K the
    corrected C equals the fault-free C bit for bit, whatever the fault's size; the record still reports the
    residual, i.e. minus the fault to within the rounding of the line sums."""
    for M, N, K, tm, tn, fault_tile, i, j in [(16, 24, 1, 16, 8, 2, 7, 3), (20, 12, 96, 8, 8, 3, 1, 2)]:
        rng = np.random.default_rng(K)
        a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        c0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
        ntn = -(-N // tn)
        for tau in (1e-3, -1.0):
            clean, hit = c0.copy(), c0.copy()
            st0 = oracle_mod.ft_sgemm(M, N, K, a, K, b, N, clean, N, 1.25, -0.5, tm, tn, tau, None)
            st1 = oracle_mod.ft_sgemm(M, N, K, a, K, b, N, hit, N, 1.25, -0.5, tm, tn, tau, (fault_tile, i, j, delta))
            assert not st0["flag"].any()
            assert st1["flag"][fault_tile] == 1 and (st1["row"][fault_tile], st1["col"][fault_tile]) == (i, j)
            assert np.array_equal(hit, clean)
            assert st1["row_residual"][fault_tile] == pytest.approx(-delta, rel=1e-5, abs=1e-5)
            # the element itself: one fused multiply-add per k, k ascending, from zero
            gi, gj = (fault_tile // ntn) * tm + i, (fault_tile % ntn) * tn + j
            acc = np.float32(0.0)
            for k in range(K):
                acc = np.float32(float(a[gi, k]) * float(b[k, gj]) + float(acc))  # exact in double, rounded once
            assert oracle_mod.recompute_element(a[gi], b[:, gj:], N, 0, K) == float(acc)
            # the cadence model corrects the same way, at whichever verification the fault shows
            for check in range(-(-K // 32)):
                hit2 = c0.copy()
                st2 = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, hit2, N, 1.25, -0.5, tm, tn, tau, 32,
                                                  [(fault_tile, i, j, delta, check)])
                assert st2["flag"][fault_tile] == 1 and np.array_equal(hit2, clean)


def test_recompute_element_covers_exactly_its_k_range(oracle_mod):
    a = np.arange(1, 9, dtype=np.float32)
    b = np.full((8, 3), np.nan, dtype=np.float32)
    b[:, 1] = [1, 10, 100, 1000, 1e4, 1e5, 1e6, 1e7]
    assert oracle_mod.recompute_element(a, b[:, 1:], 3, 0, 8) == 87654321.0 - 1.0  # float(87654321) rounds to ...320
    assert oracle_mod.recompute_element(a, b[:, 1:], 3, 2, 5) == 54300.0
    assert oracle_mod.recompute_element(a, b[:, 1:], 3, 4, 4) == 0.0


def test_sgemm_device_order_matches_numpy_and_keeps_its_k_order(oracle_mod):
    """The model of the device's summation order: float accumulator, one fused multiply-add per k, k taken in the
    order 0,4,1,5,2,6,3,7,8,12,9,13,10,14,11,15 inside each group of 16."""
    M, N, K, lda, ldb, ldc = 9, 7, 53, 60, 11, 8
    a = oracle_mod.fill_uniform_matrix(M, K, 81, ld=lda)
    b = oracle_mod.fill_uniform_matrix(K, N, 82, ld=ldb)
    c0 = oracle_mod.fill_uniform_matrix(M, N, 83, ld=ldc)
    c = c0.copy()
    oracle_mod.sgemm_device_order(M, N, K, a, lda, b, ldb, c, ldc, 1.5, -0.75)
    ref = 1.5 * (a[:, :K].astype(np.float64) @ b[:, :N].astype(np.float64)) - 0.75 * c0[:, :N]
    assert np.max(np.abs(c[:, :N] - ref)) < 5e-6 and np.all(np.isnan(c[:, N:]))
    c = np.full((M, ldc), np.nan, dtype=np.float32)   # beta == 0: C is not read
    oracle_mod.sgemm_device_order(M, N, K, a, lda, b, ldb, c, ldc, 1.0, 0.0)
    assert np.max(np.abs(c[:, :N] - a[:, :K].astype(np.float64) @ b[:, :N].astype(np.float64))) < 5e-6
    # order, by cancellation: +B and -B with B = 2^30 swallow a 1.0 that is added between them and keep one added after
    def run(K, **terms):
        a1 = np.zeros((1, 16), dtype=np.float32)
        for k, v in terms.items():
            a1[0, int(k[1:])] = v
        b1 = np.ones((16, 1), dtype=np.float32)
        c1 = np.full((1, 1), np.nan, dtype=np.float32)
        oracle_mod.sgemm_device_order(1, 1, K, a1, 16, b1, 1, c1, 1, 1.0, 0.0)
        return float(c1[0, 0]), float(oracle_mod.tile_acc(a1, 16, b1, 1, 1, 1, K)[0, 0])
    B = 2.0**30
    assert run(16, k4=B, k5=-B, k2=1.0) == (1.0, 0.0)     # device: 4, 1, 5, 2: the one comes last; ascending: first
    assert run(16, k1=B, k2=-B, k4=1.0) == (0.0, 1.0)     # device: 0, 4, 1, 5, 2: the one sits between them
    assert run(16, k8=B, k9=-B, k12=1.0) == (0.0, 1.0)    # second half of the group: 8, 12, 9
    assert run(16, k3=B, k8=-B, k7=1.0) == (0.0, 0.0)     # 3, 7, 8 in both orders
    assert run(16, k7=B, k8=-B, k3=1.0) == (0.0, 0.0)     # ... 3, 7 | 8: the one precedes both in both orders
    assert run(16, k6=B, k7=-B, k3=1.0) == (0.0, 0.0) and run(16, k2=B, k3=-B, k6=1.0) == (0.0, 1.0)  # 2, 6, 3, 7
    # a ragged last group takes the k that exist, in the same relative order
    assert run(6, k4=B, k5=-B, k2=1.0) == (1.0, 0.0)
    assert run(5, k4=B, k5=-B, k2=1.0) == (B, B)          # k = 5 is outside K


def test_checked_model_with_one_verification_is_the_plain_model(oracle_mod):
    M, N, K, tm, tn = 20, 12, 64, 8, 8
    rng = np.random.default_rng(6)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    c0 = rng.uniform(-1, 1, (M, N)).astype(np.float32)
    for tau in (1e-3, -1.0):
        for fault in (None, (1, 3, 2, 0.5), (5, 3, 1, -20.0)):
            c1, c2 = c0.copy(), c0.copy()
            st1 = oracle_mod.ft_sgemm(M, N, K, a, K, b, N, c1, N, 1.5, -0.5, tm, tn, tau, fault)
            st2 = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c2, N, 1.5, -0.5, tm, tn, tau, 0, [] if fault is None else [fault + (7,)])
            assert np.array_equal(c1, c2) and np.array_equal(st1, st2)
            # an interval of K or more is a single verification too
            c3 = c0.copy()
            st3 = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c3, N, 1.5, -0.5, tm, tn, tau, K, [] if fault is None else [fault + (0,)])
            assert np.array_equal(c1, c3) and np.array_equal(st1, st3)


def _exact_problem(M, N, K, seed):
    rng = np.random.default_rng(seed)
    a = rng.integers(-8, 9, (M, K)).astype(np.float32)
    b = rng.integers(-8, 9, (K, N)).astype(np.float32)
    return a, b, a.astype(np.float64) @ b.astype(np.float64)


def test_checked_model_corrects_one_fault_per_verification(oracle_mod):
    """Small-integer operands: accumulators and checksums are exact, so every expectation below is exact.  Two faults
    in one tile cannot be located by a single verification (two bad rows, two bad columns), but can when they fall
    into different K intervals; the record adds the bad-line counts and keeps the first location."""
    M, N, K, tm, tn = 16, 24, 96, 16, 8   # 1 x 3 tiles, three intervals of 32
    a, b, exact = _exact_problem(M, N, K, 21)
    faults = [(1, 3, 5, 64.0, 0), (1, 9, 2, -32.0, 2)]
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, 32, faults)
    assert np.array_equal(c, exact.astype(np.float32))             # both removed
    assert st["flag"].tolist() == [0, 1, 0]
    assert (st["row"][1], st["col"][1], st["n_bad_rows"][1], st["n_bad_cols"][1]) == (3, 5, 2, 2)
    assert (st["row_residual"][1], st["col_residual"][1]) == (-64.0, -64.0)
    assert st["max_clean_residual"].tolist() == [0.0, 0.0, 0.0]
    # the same two faults seen by one verification: detected, not correctable, left in C
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, 0, faults)
    assert st["flag"].tolist() == [0, 2, 0] and (st["n_bad_rows"][1], st["n_bad_cols"][1]) == (2, 2)
    assert (st["row"][1], st["col"][1]) == (-1, -1)
    want = exact.copy()
    want[3, 8 + 5] += 64.0
    want[9, 8 + 2] -= 32.0
    assert np.array_equal(c, want.astype(np.float32))
    # both in the same interval: that verification fails, the tile stays uncorrectable, later ones find nothing new
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, 32,
                                     [(1, 3, 5, 64.0, 1), (1, 9, 2, -32.0, 1)])
    assert st["flag"][1] == 2 and (st["n_bad_rows"][1], st["n_bad_cols"][1]) == (2, 2)
    assert np.array_equal(c, want.astype(np.float32))
    # an uncorrectable verification followed by a locatable fault: the later fault is still corrected in C
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, 32,
                                     [(1, 3, 5, 64.0, 0), (1, 9, 2, -32.0, 0), (1, 0, 0, 16.0, 2)])
    assert st["flag"][1] == 2 and (st["n_bad_rows"][1], st["n_bad_cols"][1]) == (3, 3)
    assert np.array_equal(c, want.astype(np.float32))


def test_weighted_locator_model_closed_forms(oracle_mod):
    """The reference's second scheme (two row sums of B, weights [1, 1, ...] and [1, 2, ...]; README.md:16-26) on
    small-integer operands, where accumulators and checksums are exact: a fault delta at (m, n) of a tile gives
    d1 = -delta and d2 = -(n + 1) delta, every column of every tile is located (also in the clipped edge tiles), the
    corrected product is the fault-free one, and the record carries the two residuals."""
    M, N, K, tm, tn = 20, 27, 48, 8, 12     # 3 x 3 tiles, the last row of tiles 4 high, the last column 3 wide
    a, b, exact = _exact_problem(M, N, K, 31)
    ntn = -(-N // tn)
    for tile in range(9):
        rows, cols = min(tm, M - (tile // ntn) * tm), min(tn, N - (tile % ntn) * tn)
        for n in range(cols):
            m, delta = (3 * n + tile) % rows, float((-1) ** n * (5 + n))
            c = np.zeros((M, N), np.float32)
            st = oracle_mod.ft_sgemm_weighted(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, [(tile, m, n, delta)])
            want = [0] * 9
            want[tile] = 1
            assert st["flag"].tolist() == want
            assert (st["row"][tile], st["col"][tile], st["n_bad_rows"][tile], st["n_bad_cols"][tile]) == (m, n, 1, 1)
            assert (st["row_residual"][tile], st["col_residual"][tile]) == (-delta, -(n + 1) * delta)
            assert np.array_equal(c, exact.astype(np.float32))
    # fault-free: nothing flagged, exact residuals
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_weighted(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, [])
    assert not st["flag"].any() and st["max_clean_residual"].max() == 0.0 and np.array_equal(c, exact.astype(np.float32))
    # below the threshold: not flagged, left in C
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_weighted(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, [(4, 1, 1, 0.25)])
    assert not st["flag"].any() and st["max_clean_residual"][4] == 0.25 and c[9, 13] == exact[9, 13] + 0.25
    # two equal faults in one row, columns 2 and 6: the ratio points at column 4, which is healthy - computing it again
    # changes nothing, the location is not confirmed, the tile is reported detected and both faults stay
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_weighted(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, [(0, 5, 2, 8.0), (0, 5, 6, 8.0)])
    assert st["flag"][0] == 2 and (st["n_bad_rows"][0], st["n_bad_cols"][0], st["row"][0], st["col"][0]) == (1, 0, -1, -1)
    want = exact.copy()
    want[5, 2] += 8.0
    want[5, 6] += 8.0
    assert np.array_equal(c, want.astype(np.float32))
    # two faults in different rows: two bad rows, nothing located
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_weighted(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 0.5, [(0, 5, 2, 8.0), (0, 6, 2, -4.0)])
    assert st["flag"][0] == 2 and st["n_bad_rows"][0] == 2
    # alpha / beta are applied after the correction
    c0 = np.arange(M * N, dtype=np.float32).reshape(M, N)
    c = c0.copy()
    oracle_mod.ft_sgemm_weighted(M, N, K, a, K, b, N, c, N, 2.0, -1.0, tm, tn, 0.5, [(8, 3, 2, 64.0)])
    assert np.array_equal(c, (2.0 * exact - c0).astype(np.float32))


def test_weighted_locator_model_against_numpy_composition(oracle_mod):
    """Uniform operands, padded leading dimensions: the residuals the record reports equal an independent numpy FP64
    composition (references from A and the two row sums of B, observed sums from the FP32 accumulator model), the
    data-scaled threshold is that of the row x column model's rows, and a fault is located where its size allows."""
    M, N, K, tm, tn, lda, ldb = 24, 40, 96, 16, 32, 100, 43
    a = oracle_mod.fill_uniform_matrix(M, K, 71, ld=lda)
    b = oracle_mod.fill_uniform_matrix(K, N, 72, ld=ldb)
    tile, m, n, delta = 1, 5, 6, 0.5        # tile 1: rows 0..15, columns 32..39 (8 wide)
    for tau in (1e-4, 0.0, -1.0):
        c = np.zeros((M, N), np.float32)
        st = oracle_mod.ft_sgemm_weighted(M, N, K, a, lda, b, ldb, c, N, 1.0, 0.0, tm, tn, tau, [(tile, m, n, delta)])
        assert st["flag"].tolist() == [0, 1, 0, 0] and (st["row"][1], st["col"][1]) == (m, n)
        at, bt = a[:16, :K], b[:, 32:40]
        acc = oracle_mod.tile_acc(at, lda, bt, ldb, 16, 8, K)
        acc[m, n] += np.float32(delta)
        w = np.arange(1, 9, dtype=np.float64)
        r1 = at.astype(np.float64) @ bt.astype(np.float64).sum(axis=1)
        r2 = at.astype(np.float64) @ (bt.astype(np.float64) @ w)
        d1 = r1 - acc.astype(np.float64).sum(axis=1)
        d2 = r2 - acc.astype(np.float64) @ w
        assert st["row_residual"][1] == np.float32(d1[m]) and st["col_residual"][1] == np.float32(d2[m])
        assert st["max_clean_residual"][1] == np.float32(np.abs(np.delete(d1, m)).max())
        assert abs(d1[m] + delta) < 1e-5 and abs(d2[m] + (n + 1) * delta) < 1e-4
        ref = a[:, :K].astype(np.float64) @ b[:, :N].astype(np.float64)
        assert np.max(np.abs(c - ref)) < 5e-6     # corrected: the fault is gone
    # a fault just above the threshold but far below the rounding noise of the weighted sums x the tile width is
    # detected, whether or not the ratio happens to hit its column
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_weighted(M, N, K, a, lda, b, ldb, c, N, 1.0, 0.0, tm, tn, 2e-5, [(0, 3, 17, 4e-5)])
    assert st["flag"][0] in (1, 2) and st["n_bad_rows"][0] == 1 and not st["flag"][1:].any()


def test_checked_model_resynchronises_after_every_verification(oracle_mod):
    """Two faults of 0.75 tau in one column, in different intervals: each verification sees one of them and absorbs it,
    so nothing is ever flagged (and both stay in C); a single verification at the end sees 1.5 tau in that column and
    0.75 tau in two rows.  The residual a verification reports is what happened since the one before."""
    M, N, K, tm, tn = 8, 8, 64, 8, 8
    a, b, exact = _exact_problem(M, N, K, 22)
    tau = 1.0
    faults = [(0, 1, 2, 0.75, 0), (0, 6, 2, 0.75, 1)]
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, tau, 32, faults)
    assert st["flag"][0] == 0 and st["max_clean_residual"][0] == 0.75
    want = exact.copy()
    want[1, 2] += 0.75
    want[6, 2] += 0.75
    assert np.array_equal(c, want.astype(np.float32))
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, tau, 0, faults)
    assert (st["flag"][0], st["n_bad_rows"][0], st["n_bad_cols"][0]) == (2, 0, 1) and st["max_clean_residual"][0] == 0.75
    # (the same two faults in one row would go unnoticed by a single verification: the columns, 0.75 tau each, screen)
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, tau, 0, [(0, 2, 1, 0.75, 0), (0, 2, 6, 0.75, 1)])
    assert (st["flag"][0], st["n_bad_rows"][0], st["n_bad_cols"][0]) == (0, 0, 0)
    # the interval boundaries are k = 32, 64: a fault before verification 1 is seen by verification 1, not 0
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, tau, 32, [(0, 4, 4, 8.0, 1)])
    assert (st["flag"][0], st["row"][0], st["col"][0], st["row_residual"][0]) == (1, 4, 4, -8.0)
    assert np.array_equal(c, exact.astype(np.float32))
    # a ragged last interval (K = 70: verifications after k = 32, 64, 70) and a fault before the last one
    a, b, exact = _exact_problem(M, N, 70, 23)
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, 70, a, 70, b, N, c, N, 1.0, 0.0, tm, tn, tau, 32, [(0, 7, 0, -4.0, 2)])
    assert (st["flag"][0], st["row"][0], st["col"][0]) == (1, 7, 0) and np.array_equal(c, exact.astype(np.float32))
    # a verification index past the last one never happens: the fault is not injected
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, 70, a, 70, b, N, c, N, 1.0, 0.0, tm, tn, tau, 32, [(0, 7, 0, -4.0, 3)])
    assert st["flag"][0] == 0 and np.array_equal(c, exact.astype(np.float32))


def test_checked_model_references_cover_the_k_range_done_so_far(oracle_mod):
    """Float operands: the residuals of every verification are rounding noise, far below a fault; an intermediate
    verification that compared the accumulators of k < 32 with references over all of K (or the other way round)
    would flag every line."""
    M, N, K, tm, tn = 24, 16, 200, 8, 16
    rng = np.random.default_rng(24)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    b = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    c = np.zeros((M, N), np.float32)
    st = oracle_mod.ft_sgemm_checked(M, N, K, a, K, b, N, c, N, 1.0, 0.0, tm, tn, 1e-3, 32, [(2, 1, 9, 0.05, 4)])
    assert st["flag"].tolist() == [0, 0, 1] and (st["row"][2], st["col"][2]) == (1, 9)
    assert st["max_clean_residual"].max() < 5e-5
    assert np.max(np.abs(c - a.astype(np.float64) @ b.astype(np.float64))) < 5e-5


@pytest.mark.parametrize("trans", [False, True])
def test_sgemv_f64_matches_numpy_and_is_not_transposed(oracle_mod, trans):
    M, N, lda = 13, 29, 37
    a = oracle_mod.fill_uniform_matrix(M, N, 71, ld=lda)
    x = oracle_mod.fill_uniform(M if trans else N, 72)
    y = oracle_mod.fill_uniform(N if trans else M, 73)
    a64 = a[:, :N].astype(np.float64)
    out, den = oracle_mod.sgemv_f64(trans, M, N, 1.25, a, lda, x, -0.75, y)
    mat = a64.T if trans else a64
    assert np.allclose(out, 1.25 * (mat @ x.astype(np.float64)) - 0.75 * y.astype(np.float64), rtol=0, atol=1e-12)
    assert np.allclose(den, 1.25 * (np.abs(mat) @ np.abs(x).astype(np.float64)) + 0.75 * np.abs(y).astype(np.float64), rtol=0, atol=1e-12)
    # a non-square matrix with the wrong orientation would not even have matching lengths: check one known entry
    e = np.zeros(M if trans else N, np.float32)
    e[2] = 1.0
    out, _ = oracle_mod.sgemv_f64(trans, M, N, 1.0, a, lda, e, 0.0, None)
    assert np.array_equal(out, (a64[2, :] if trans else a64[:, 2]))


@pytest.mark.parametrize("alpha,beta,panel", [(1.0, 0.0, 256), (1.5, -0.5, 256), (1.0, 1.0, 100)])
def test_offline_ft_model_closed_form(oracle_mod, alpha, beta, panel):
    """Row and column sums of alpha*A*B + beta*C0 equal the checksums carried through the operands, so every
    residual sum is 0 until a fault of size delta enters C and delta from that panel on; C keeps the fault."""
    M, N, K = 37, 23, 700
    a = oracle_mod.fill_uniform_matrix(M, K, 81)
    b = oracle_mod.fill_uniform_matrix(K, N, 82)
    c0 = oracle_mod.fill_uniform_matrix(M, N, 83)
    ref = alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0
    panels = -(-K // panel)
    c = c0.copy()
    res = oracle_mod.offline_ft_sgemm(M, N, K, a, K, b, N, c, N, alpha, beta, panel)
    assert res.shape == (2 * panels,) and np.abs(res).max() < 1e-9
    assert np.abs(c - ref).max() < 1e-5
    for fault_panel in (0, panels - 1):
        c = c0.copy()
        res = oracle_mod.offline_ft_sgemm(M, N, K, a, K, b, N, c, N, alpha, beta, panel, (fault_panel, 5, 7, -3.5))
        expect = np.repeat(np.where(np.arange(panels) >= fault_panel, -3.5, 0.0), 2)
        assert np.abs(res - expect).max() < 1e-9
        diff = c - ref
        assert abs(diff[5, 7] + 3.5) < 1e-5
        diff[5, 7] = 0.0
        assert np.abs(diff).max() < 1e-5


def test_relative_thresholds_closed_forms_and_scaling(oracle_mod):
    """Constant tile: line mean = tile mean = |c|, so a row's threshold is rel * |c| * sqrt(tn) (sqrt(tm) for columns)
    with rel = 2.56e-7 * sqrt(max(K, 64)); a single non-zero entry raises its own row and column above the floor the
    tile mean gives every line; thresholds are linear in the data and in the factor, grow like sqrt(K) from K = 64 up
    and stay put below."""
    tm, tn, K = 48, 20, 400
    rel = 2.56e-7 * np.sqrt(K)
    tr, tc = oracle_mod.abft_relative_thresholds(np.full((tm, tn), -3.0, np.float32), K)
    assert np.allclose(tr, rel * 3.0 * np.sqrt(tn), rtol=1e-6) and np.allclose(tc, rel * 3.0 * np.sqrt(tm), rtol=1e-6)
    one = np.zeros((tm, tn), np.float32)
    one[5, 7] = 2.0
    tr, tc = oracle_mod.abft_relative_thresholds(one, K)
    tile_mean = 2.0 / (tm * tn)
    assert np.isclose(tr[5], rel * 2.0 / np.sqrt(tn), rtol=1e-6) and np.isclose(tc[7], rel * 2.0 / np.sqrt(tm), rtol=1e-6)
    others_r, others_c = np.delete(tr, 5), np.delete(tc, 7)
    assert np.allclose(others_r, rel * np.sqrt(tn) * tile_mean, rtol=1e-6) and np.allclose(others_c, rel * np.sqrt(tm) * tile_mean, rtol=1e-6)
    assert tr[5] > 10 * others_r[0] and tc[7] > 10 * others_c[0]
    rng = np.random.default_rng(3)
    acc = rng.standard_normal((tm, tn)).astype(np.float32)
    tr1, tc1 = oracle_mod.abft_relative_thresholds(acc, K)
    tr2, tc2 = oracle_mod.abft_relative_thresholds(acc * np.float32(8.0), 4 * K, factor=0.5)
    assert np.allclose(tr2, tr1 * 8.0 * 2.0 * 0.5, rtol=1e-6) and np.allclose(tc2, tc1 * 8.0, rtol=1e-6)
    a64 = np.abs(acc.astype(np.float64))
    want = rel * np.sqrt(tn) * np.maximum(a64.mean(axis=1), a64.mean())
    assert np.allclose(tr1, want, rtol=1e-5)
    assert np.any(a64.mean(axis=1) < a64.mean()) and np.any(a64.mean(axis=1) > a64.mean())  # both branches are exercised
    # below K = 64 the rounding of the sums themselves dominates: the threshold stops shrinking
    t1, _ = oracle_mod.abft_relative_thresholds(acc, 1)
    t64, _ = oracle_mod.abft_relative_thresholds(acc, 64)
    t256, _ = oracle_mod.abft_relative_thresholds(acc, 256)
    assert np.array_equal(t1, t64) and np.allclose(t256, 2.0 * t64, rtol=1e-6)
    # a one-element line that cancels to nearly nothing still gets the tile's scale
    thin = np.full((tm, 1), 1.0, np.float32)
    thin[3, 0] = 1e-6
    tr, _ = oracle_mod.abft_relative_thresholds(thin, K)
    assert np.isclose(tr[3], rel * (47.0 + 1e-6) / 48.0, rtol=1e-5) and np.isclose(tr[0], rel * 1.0, rtol=1e-6)


def _fixtures():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures.json")) as f:
        return json.load(f)


def test_golden_fixtures_pin_rng_saxpy_and_the_reference_fault_case(oracle_mod):
    """tests/golden/fixtures.json holds values computed with Python integers / exact fractions
    (tests/golden/make_fixtures.py), independent of the oracle's C code."""
    fx = _fixtures()
    for r in fx["rng"]:
        assert oracle_mod.uniform(r["seed"], r["idx"]) == r["value"], r
    differs = 0
    for c in fx["saxpy"]:
        x, y = np.array([c["x"]], np.float32), np.array([c["y"]], np.float32)
        oracle_mod.saxpy(c["a"], x, y)
        assert float(y[0]) == c["fused"], c
        differs += c["fused"] != c["unfused"]
    assert differs >= 3  # the set does tell a fused multiply-add from a*x rounded, then + y
    k = fx["abft"]
    tm, tn = k["tile_m"], k["tile_n"]
    dr, dc = np.zeros(tm), np.zeros(tn)
    f = k["fault"]
    dr[f["row"]] -= f["delta"]  # residual = reference - observed, the fault sits in the observed sums
    dc[f["col"]] -= f["delta"]
    st, fix = oracle_mod.abft_decide(dr, dc, k["threshold"])
    for name in ("flag", "row", "col", "n_bad_rows", "n_bad_cols"):
        assert st[name] == k["expect"][name], name
    assert fix == k["expect"]["correction"]


def test_offline_scalar_checksum_model(oracle_mod):
    """One scalar checksum per panel: against whole-matrix numpy FP64 sums (a route that shares no loop with the
    model: total of the product so far minus beta * total of C0 minus alpha * (column sums of A) . (row sums of B)
    over the k range done), against the closed form (0 before the faulted panel, delta from it on), and against
    residual [2p] of the row/column model, which it equals."""
    M, N, K, panel = 37, 29, 610, 256
    rng = np.random.default_rng(123)
    a = rng.standard_normal((M, K + 3)).astype(np.float32)
    b = rng.standard_normal((K, N + 5)).astype(np.float32)
    c0 = rng.standard_normal((M, N + 2)).astype(np.float32)
    alpha, beta = 1.25, -0.75
    for fault in (None, (1, 5, 7, 3.5), (2, 36, 28, -2.0)):
        c = c0.copy()
        res = oracle_mod.offline_ft_sgemm_scalar(M, N, K, a, K + 3, b, N + 5, c, N + 2, alpha, beta, panel, fault)
        assert res.shape == (3,)
        a64, b64, c64 = a[:, :K].astype(np.float64), b[:, :N].astype(np.float64), c0[:, :N].astype(np.float64)
        for p in range(3):
            k1 = min(K, (p + 1) * panel)
            total = (beta * c64 + alpha * a64[:, :k1] @ b64[:k1]).sum() + (fault[3] if fault and fault[0] <= p else 0.0)
            ref = beta * c64.sum() + alpha * float(a64[:, :k1].sum(axis=0) @ b64[:k1].sum(axis=1))
            assert abs(res[p] - (total - ref)) < 1e-9
            assert abs(res[p] - (fault[3] if fault and fault[0] <= p else 0.0)) < 1e-9
        c2 = c0.copy()
        both = oracle_mod.offline_ft_sgemm(M, N, K, a, K + 3, b, N + 5, c2, N + 2, alpha, beta, panel, fault)
        assert np.allclose(res, both[0::2], atol=1e-9) and np.array_equal(c, c2)

