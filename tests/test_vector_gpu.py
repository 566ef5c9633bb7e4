"""GPU parity of the fill, SAXPY and SDOT kernels against the CPU oracle, through the C ABI.

SAXPY and the fills are bit-exact; SDOT is within 1e-5 relative of the FP64 sum and reproducible bit for bit.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 3, 4, 5, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4099, (1 << 20) + 7]


def _dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a).cuda()


def test_fill_uniform_matches_oracle_bitwise(blas, oracle_mod):
    for n, seed in [(1, 1), (1000, 2), ((1 << 20) + 7, 3)]:
        d = torch.empty(n, dtype=torch.float32, device="cuda")
        blas.fill_uniform(d, seed)
        assert np.array_equal(d.cpu().numpy(), oracle_mod.fill_uniform(n, seed)), (n, seed)


def test_fill_uniform_matrix_respects_leading_dimension(blas, oracle_mod):
    rows, cols, ld = 37, 29, 40
    d = torch.full((rows, ld), float("nan"), dtype=torch.float32, device="cuda")
    blas.fill_uniform_matrix(d, rows, cols, seed=5)
    h = d.cpu().numpy()
    assert np.array_equal(h[:, :cols], oracle_mod.fill_uniform_matrix(rows, cols, seed=5))
    assert np.all(np.isnan(h[:, cols:]))


@pytest.mark.parametrize("n", SIZES)
def test_saxpy_bit_exact(blas, oracle_mod, n):
    x = oracle_mod.fill_uniform(n, seed=21)
    y = oracle_mod.fill_uniform(n, seed=22)
    dx, dy = _dev(x), _dev(y)
    blas.saxpy(n, 2.5, dx, dy)
    oracle_mod.saxpy(2.5, x, y)
    assert np.array_equal(dy.cpu().numpy(), y)
    assert np.array_equal(dx.cpu().numpy(), x)  # x is read-only


@pytest.mark.parametrize("alpha", [0.0, 1.0, -1.0, 1.0 + 2.0**-12, 3.0e-5, -7.25e4])
def test_saxpy_alpha_values(blas, oracle_mod, alpha):
    n = 10007
    x = oracle_mod.fill_uniform(n, seed=23)
    y = oracle_mod.fill_uniform(n, seed=24)
    dx, dy = _dev(x), _dev(y)
    blas.saxpy(n, alpha, dx, dy)
    oracle_mod.saxpy(alpha, x, y)
    assert np.array_equal(dy.cpu().numpy(), y)


@pytest.mark.parametrize("ox,oy", [(1, 0), (0, 3), (1, 1), (2, 3), (1, 3), (3, 5), (2, 4), (0, 2)])
def test_saxpy_misaligned_base_pointers(blas, oracle_mod, ox, oy):
    n = 5003
    x = oracle_mod.fill_uniform(n + 8, seed=25)
    y = oracle_mod.fill_uniform(n + 8, seed=26)
    dx, dy = _dev(x), _dev(y)
    blas.saxpy(n, 2.5, dx[ox:ox + n], dy[oy:oy + n])
    yo = y.copy()
    oracle_mod.saxpy(2.5, x[ox:ox + n], yo[oy:oy + n])
    assert np.array_equal(dy.cpu().numpy(), yo)  # also checks nothing outside [oy, oy+n) changed


def test_saxpy_full_size_2_pow_28_bit_exact(blas, oracle_mod):
    n = 1 << 28
    dx = torch.empty(n, dtype=torch.float32, device="cuda")
    dy = torch.empty(n, dtype=torch.float32, device="cuda")
    blas.fill_uniform(dx, 31)
    blas.fill_uniform(dy, 32)
    blas.saxpy(n, 2.5, dx, dy)
    # oracle on the whole vector, compared in chunks to bound host memory
    x = oracle_mod.fill_uniform(n, 31)
    y = oracle_mod.fill_uniform(n, 32)
    oracle_mod.saxpy(2.5, x, y)
    chunk = 1 << 26
    for s in range(0, n, chunk):
        assert np.array_equal(dy[s:s + chunk].cpu().numpy(), y[s:s + chunk]), s


def _sdot(blas, n, dx, dy):
    out = torch.full((1,), float("nan"), dtype=torch.float32, device="cuda")
    blas.sdot(n, dx, dy, out)
    return out.cpu().numpy()[0]


@pytest.mark.parametrize("n", SIZES)
def test_sdot_within_tolerance_and_reproducible(blas, oracle_mod, n):
    x = oracle_mod.fill_uniform(n, seed=41)
    y = oracle_mod.fill_uniform(n, seed=42)
    dx, dy = _dev(x), _dev(y)
    got = [_sdot(blas, n, dx, dy) for _ in range(3)]
    assert got[0].tobytes() == got[1].tobytes() == got[2].tobytes()  # deterministic reduction order
    exact = oracle_mod.sdot_f64(x, y)
    scale = float(np.dot(np.abs(x).astype(np.float64), np.abs(y).astype(np.float64)))
    # rel 1e-5 of the result; when the sum cancels, relative to sum|x||y| (the condition-number-free bound)
    assert abs(float(got[0]) - exact) <= 1e-5 * max(abs(exact), 1e-2 * scale) + 1e-30, (got[0], exact)


def test_sdot_closed_forms(blas):
    n = 1 << 16
    ones = torch.ones(n, dtype=torch.float32, device="cuda")
    assert _sdot(blas, n, ones, ones) == np.float32(n)
    k = torch.arange(1, 101, dtype=torch.float32, device="cuda")
    assert _sdot(blas, 100, k, k) == np.float32(338350.0)
    # orthogonal by construction: alternating signs cancel exactly
    alt = torch.ones(n, dtype=torch.float32, device="cuda")
    alt[1::2] = -1.0
    assert _sdot(blas, n, ones, alt) == np.float32(0.0)


def test_sdot_misaligned_and_explicit_workspace(blas, oracle_mod):
    from hpcdeepneuralnetworks_amd import _lib

    n = 7001
    x = oracle_mod.fill_uniform(n + 4, seed=43)
    y = oracle_mod.fill_uniform(n + 4, seed=44)
    dx, dy = _dev(x), _dev(y)
    ws = blas.workspace(int(_lib.lib().hpcdnn_workspace_bytes(_lib.OP_SDOT, 0, 0, 0)))
    out = torch.zeros(1, dtype=torch.float32, device="cuda")
    for ox, oy in [(1, 0), (3, 2)]:
        blas.sdot(n, dx[ox:ox + n], dy[oy:oy + n], out, ws=ws)  # same workspace reused: the ticket resets itself
        exact = oracle_mod.sdot_f64(x[ox:ox + n], y[oy:oy + n])
        assert abs(float(out.cpu()[0]) - exact) <= 1e-5 * abs(exact) + 1e-4


def test_sdot_full_size_2_pow_28(blas, oracle_mod):
    n = 1 << 28
    dx = torch.empty(n, dtype=torch.float32, device="cuda")
    dy = torch.empty(n, dtype=torch.float32, device="cuda")
    blas.fill_uniform(dx, 51)
    blas.fill_uniform(dy, 52)
    got = _sdot(blas, n, dx, dy)
    x = oracle_mod.fill_uniform(n, 51)
    y = oracle_mod.fill_uniform(n, 52)
    exact = oracle_mod.sdot_f64(x, y)
    del y
    assert abs(float(got) - exact) <= 1e-5 * abs(exact), (got, exact)
    # size-independent properties: x.x is the squared norm (n/3 for uniform[-1,1)), and the dot is symmetric
    xx = _sdot(blas, n, dx, dx)
    assert abs(float(xx) - oracle_mod.sdot_f64(x, x)) <= 1e-5 * float(xx)
    assert abs(float(xx) / n - 1.0 / 3.0) < 1e-3
    assert _sdot(blas, n, dy, dx).tobytes() == got.tobytes()


def test_vectors_longer_than_2_pow_31_elements(blas, oracle_mod):
    """Indices past 2^31 (64-bit indexing; the reference's `int N` stops at 2^31 - 1): SAXPY bit-exact on sampled
    elements and on the n % 4 tail, untouched past n; SDOT against an FP64 sum formed chunk by chunk."""
    n = (1 << 31) + (1 << 20) + 3
    dx = torch.empty(n + 5, dtype=torch.float32, device="cuda")
    dy = torch.empty(n + 5, dtype=torch.float32, device="cuda")
    blas.fill_uniform(dx, 61)
    blas.fill_uniform(dy, 62)
    exact = 0.0
    chunk = 1 << 28
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        exact += float((dx[s:e].double() * dy[s:e].double()).sum())
    got = float(_sdot(blas, n, dx, dy))
    assert abs(got - exact) <= 1e-5 * abs(exact) + 1e-2, (got, exact)

    blas.saxpy(n, 2.5, dx, dy)
    rng = np.random.default_rng(5)
    idx = np.unique(np.concatenate([rng.integers(0, n, 4000), np.arange(n - 8, n + 5), np.arange(0, 8),
                                    np.arange((1 << 31) - 8, (1 << 31) + 8), np.arange((1 << 29) - 4, (1 << 29) + 4) * 4]))
    got_y = dy[torch.from_numpy(idx).cuda()].cpu().numpy()
    for i, g in zip(idx.tolist(), got_y.tolist()):
        x0, y0 = np.float32(oracle_mod.uniform(61, i)), np.float32(oracle_mod.uniform(62, i))
        if i < n:
            xs, ys = np.array([x0], np.float32), np.array([y0], np.float32)
            oracle_mod.saxpy(2.5, xs, ys)
            assert np.float32(g) == ys[0], i
        else:
            assert np.float32(g) == y0, i  # past n: untouched


def test_golden_fixtures_on_the_device(blas):
    """The device generator and SAXPY against tests/golden/fixtures.json (values from Python integers and exact
    fractions, tests/golden/make_fixtures.py)."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures.json")) as f:
        fx = json.load(f)
    for seed in sorted({r["seed"] for r in fx["rng"]}):
        want = {r["idx"]: r["value"] for r in fx["rng"] if r["seed"] == seed and r["idx"] < (1 << 20)}
        buf = torch.empty(max(want) + 1, dtype=torch.float32, device="cuda")
        blas.fill_uniform(buf, seed)
        got = buf.cpu().numpy()
        for idx, value in want.items():
            assert float(got[idx]) == value, (seed, idx)
    cases = fx["saxpy"]
    for a in sorted({c["a"] for c in cases}):
        sel = [c for c in cases if c["a"] == a]
        x = torch.tensor([c["x"] for c in sel], dtype=torch.float32, device="cuda")
        y = torch.tensor([c["y"] for c in sel], dtype=torch.float32, device="cuda")
        blas.saxpy(len(sel), a, x, y)
        assert y.cpu().numpy().tolist() == [np.float32(c["fused"]) for c in sel]
