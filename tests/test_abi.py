"""CPU-side checks of the C ABI: the library loads, exports every symbol the header declares,
rejects bad arguments before touching the GPU, and its host validator agrees with the oracle."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def L():
    from hpcdeepneuralnetworks_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return _lib.lib()


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "hpcdnn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hpcdnn_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(L):
    from hpcdeepneuralnetworks_amd import _lib

    declared = _declared_symbols()
    assert len(declared) >= 16
    assert sorted(_lib.EXPORTS) == declared
    for name in declared:
        assert getattr(L, name) is not None


def test_version_and_error_strings(L):
    assert b"gfx950" in L.hpcdnn_version()
    assert L.hpcdnn_error_string(0) == b"success"
    assert b"invalid" in L.hpcdnn_error_string(1)
    assert b"workspace" in L.hpcdnn_error_string(2)


def test_status_and_fault_struct_sizes():
    from hpcdeepneuralnetworks_amd import _lib
    from hpcdeepneuralnetworks_amd.blas import FT_STATUS_DTYPE

    assert C.sizeof(_lib.Fault) == 16 and FT_STATUS_DTYPE.itemsize == 32


def _tile(L, t):
    bm, bn, bk = C.c_int(), C.c_int(), C.c_int()
    assert L.hpcdnn_sgemm_tile_info(t, C.byref(bm), C.byref(bn), C.byref(bk)) == 0
    return bm.value, bn.value, bk.value


def test_bad_arguments_are_rejected_without_a_gpu(L):
    INVALID, WORKSPACE = 1, 2
    dummy = C.c_void_p(0x1000)
    assert L.hpcdnn_saxpy(-1, 1.0, dummy, dummy, None) == INVALID
    assert L.hpcdnn_saxpy(4, 1.0, None, dummy, None) == INVALID
    assert L.hpcdnn_saxpy(4, 1.0, C.c_void_p(0x1002), dummy, None) == INVALID  # not 4-byte aligned
    assert L.hpcdnn_saxpy(0, 1.0, None, None, None) == 0
    assert L.hpcdnn_sdot(4, dummy, dummy, None, dummy, 1 << 20, None) == INVALID
    assert L.hpcdnn_sdot(4, dummy, dummy, dummy, None, 0, None) == WORKSPACE
    assert L.hpcdnn_sdot(4, dummy, dummy, dummy, dummy, 8, None) == WORKSPACE
    assert L.hpcdnn_sdot(4, dummy, dummy, dummy, C.c_void_p(0x1004), 1 << 20, None) == INVALID  # the block partials are doubles
    # GEMM: negative dims, leading dimensions smaller than the row length, null operands
    assert L.hpcdnn_sgemm(-1, 4, 4, dummy, 4, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm(4, 4, 4, dummy, 3, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm(4, 4, 4, dummy, 4, dummy, 3, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm(4, 4, 4, dummy, 4, dummy, 4, dummy, 3, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm(4, 4, 4, None, 4, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm(0, 4, 4, None, 4, None, 4, None, 4, 1.0, 0.0, None, 0, None) == 0  # empty: nothing to do
    # transposed left operand: At is K x M, so its row length must reach M (not K)
    assert L.hpcdnn_sgemm_tn(8, 4, 4, dummy, 7, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm_tn(4, 4, 8, dummy, 4, dummy, 4, dummy, 3, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm_tn(0, 4, 4, None, 1, None, 4, None, 4, 1.0, 0.0, None, 0, None) == 0
    assert L.hpcdnn_sgemm_tn(4, 4, 4, dummy, (1 << 25) - 1023, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    # column-major C = A * B^T: lda >= M, ldb >= N, ldc >= M
    assert L.hpcdnn_sgemm_cm_nt(8, 4, 4, dummy, 7, dummy, 4, dummy, 8, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm_cm_nt(8, 4, 4, dummy, 8, dummy, 3, dummy, 8, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm_cm_nt(8, 4, 4, dummy, 8, dummy, 4, dummy, 7, 1.0, 0.0, None, 0, None) == INVALID
    # ... and its ABFT counterpart (same leading-dimension rules; empty problems need nothing)
    assert L.hpcdnn_ft_sgemm_cm_nt(8, 4, 4, dummy, 7, dummy, 4, dummy, 8, 1.0, 0.0, 0.0, None, None, None, 0, None) == INVALID
    assert L.hpcdnn_ft_sgemm_cm_nt(8, 4, 4, dummy, 8, dummy, 3, dummy, 8, 1.0, 0.0, 0.0, None, None, None, 0, None) == INVALID
    assert L.hpcdnn_ft_sgemm_cm_nt(8, 4, 4, dummy, 8, dummy, 4, dummy, 7, 1.0, 0.0, 0.0, None, None, None, 0, None) == INVALID
    assert L.hpcdnn_ft_sgemm_cm_nt(0, 4, 4, None, 1, None, 4, None, 1, 1.0, 0.0, 0.0, None, None, None, 0, None) == 0
    assert L.hpcdnn_workspace_bytes(5, 300, 200, 100) == L.hpcdnn_workspace_bytes(2, 200, 300, 100) > 0
    assert L.hpcdnn_sgemm_ex(4, 4, 4, dummy, 4, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, 99, 1, None) == INVALID
    assert L.hpcdnn_sgemm_ex(4, 4, 64, dummy, 64, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, 0, 2, None) == WORKSPACE
    # the 32 x 32 tile has no tail split (its waves split K among themselves)
    small = [t for t in range(L.hpcdnn_sgemm_num_tiles()) if _tile(L, t)[:2] == (32, 32)]
    assert L.hpcdnn_sgemm_tn_ex(256, 1056, 256, dummy, 256, dummy, 1056, dummy, 1056, 1.0, 0.0, dummy, 1 << 30, small[0], -2, None) == INVALID
    assert len(small) == 1
    assert L.hpcdnn_sgemm_ex(256, 1056, 256, dummy, 256, dummy, 1056, dummy, 1056, 1.0, 0.0, dummy, 1 << 30, small[0], -2, None) == INVALID
    # leading dimensions beyond the 32-bit tile offsets
    assert L.hpcdnn_sgemm(4, 4, 4, dummy, (1 << 21) - 63, dummy, 4, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm(4, 4, 4, dummy, 4, dummy, (1 << 25) - 1023, dummy, 4, 1.0, 0.0, None, 0, None) == INVALID
    assert L.hpcdnn_sgemm(4, 4, 4, dummy, 4, dummy, 4, dummy, (1 << 21) - 63, 1.0, 0.0, None, 0, None) == INVALID
    from hpcdeepneuralnetworks_amd._lib import Fault

    bad = Fault(5, 0, 0, 1.0)  # only one tile exists
    assert L.hpcdnn_ft_sgemm(4, 4, 4, dummy, 4, dummy, 4, dummy, 4, 1.0, 0.0, 0.0, C.byref(bad), None, None, 0, None) == INVALID
    bad = Fault(0, 256, 0, 1.0)
    assert L.hpcdnn_ft_sgemm(4, 4, 4, dummy, 4, dummy, 4, dummy, 4, 1.0, 0.0, 0.0, C.byref(bad), None, None, 0, None) == INVALID


def test_tile_table_and_workspace_sizes(L):
    n = L.hpcdnn_sgemm_num_tiles()
    assert n >= 4
    bm, bn, bk = C.c_int(), C.c_int(), C.c_int()
    assert L.hpcdnn_sgemm_tile_info(0, C.byref(bm), C.byref(bn), C.byref(bk)) == 0
    assert (bm.value, bn.value) == (256, 128) and bk.value % 8 == 0
    assert L.hpcdnn_sgemm_tile_info(n, None, None, None) == 1
    assert L.hpcdnn_ft_num_tiles(4096, 4096) == 16 * 32
    assert L.hpcdnn_ft_num_tiles(257, 129) == 4
    assert L.hpcdnn_workspace_bytes(1, 0, 0, 0) >= 64 + 8
    # a square compute-bound problem needs no split-K scratch; the deep-K one does
    assert L.hpcdnn_workspace_bytes(0, 4096, 4096, 4096) == 0
    ws = L.hpcdnn_workspace_bytes(0, 128, 128, 65536)
    assert ws > 0 and ws % (128 * 128 * 4) == 0
    assert L.hpcdnn_ft_default_tau(4096) > 0


def test_host_cpu_gemm_matches_oracle_and_numpy(L, oracle_mod):
    n = 64
    a = oracle_mod.fill_uniform_matrix(n, n, seed=11)
    b = oracle_mod.fill_uniform_matrix(n, n, seed=12)
    c0 = oracle_mod.fill_uniform_matrix(n, n, seed=13)
    for alpha, beta in [(1.0, 0.0), (1.5, -1.0)]:
        c_lib, c_orc = c0.copy(), c0.copy()
        L.hpcdnn_cpu_gemm(alpha, beta, a.ctypes.data, b.ctypes.data, n, c_lib.ctypes.data)
        oracle_mod.cpu_gemm(alpha, beta, a, b, n, c_orc)
        assert np.array_equal(c_lib, c_orc)  # same order, same float accumulator -> same bits
        ref = alpha * (a.astype(np.float64) @ b.astype(np.float64)) + beta * c0
        assert np.max(np.abs(c_lib - ref)) < 5e-5


def test_plan_query_without_a_gpu(L):
    """Tile / split choice is host arithmetic on the shape (256 CUs assumed when no device is present)."""
    def plan(M, N, K, ws):
        t, s = C.c_int(-1), C.c_int(0)
        assert L.hpcdnn_sgemm_plan(M, N, K, ws, C.byref(t), C.byref(s)) == 0
        return t.value, s.value

    n_tiles = L.hpcdnn_sgemm_num_tiles()
    for shape in [(1024, 1024, 1024), (4096, 4096, 4096), (6144, 6144, 6144), (3072, 3072, 3072), (2560, 2560, 2560), (128, 128, 65536),
                  (16384, 64, 4096)]:
        t, s = plan(*shape, 0)
        assert 0 <= t < n_tiles and s == 1                      # no workspace: nothing is split
        need = L.hpcdnn_workspace_bytes(0, *shape)
        t, s = plan(*shape, need)
        assert 0 <= t < n_tiles and (s >= 1 or s <= -2)
        if s == 1:
            assert need == 0
        elif s > 1:
            assert need == shape[0] * shape[1] * s * 4           # split-K: one raw copy of C per slice
        else:
            bm, bn = C.c_int(), C.c_int()
            assert L.hpcdnn_sgemm_tile_info(t, C.byref(bm), C.byref(bn), None) == 0
            tiles = -(-shape[0] // bm.value) * -(-shape[1] // bn.value)
            assert 0 < tiles % 256 <= 128 and need == (tiles % 256) * (-s) * bm.value * bn.value * 4
    assert plan(128, 128, 65536, 1 << 30)[1] >= 16               # deep K: split-K
    assert plan(2560, 2560, 2560, 1 << 30)[1] <= -2              # 2560^3: a partial last round whatever the tile, tail split
    assert plan(3072, 3072, 3072, 1 << 30)[1] == 1               # 3072^3: 16 x 16 tiles of 192 x 192 fill one round
    assert plan(4096, 4096, 4096, 1 << 30)[1] == 1               # 4096^3: whole rounds, nothing to split
    assert L.hpcdnn_sgemm_plan(-1, 1, 1, 0, None, None) == 1


def test_plans_fit_their_workspace_for_random_shapes(L):
    """Host arithmetic only: whatever workspace is offered, the plan is valid and never needs more than it was given."""
    import random
    rnd = random.Random(5)
    n_tiles = L.hpcdnn_sgemm_num_tiles()
    dims = [1, 7, 31, 32, 33, 64, 100, 128, 255, 256, 500, 768, 1000, 1024, 1536, 2048, 3001, 4096, 6144, 16384]
    for _ in range(300):
        M, N = rnd.choice(dims), rnd.choice(dims)
        K = rnd.choice(dims + [65536])
        need = L.hpcdnn_workspace_bytes(0, M, N, K)
        for ws in (0, need // 3, need, need + 4096):
            t, s = C.c_int(-1), C.c_int(0)
            assert L.hpcdnn_sgemm_plan(M, N, K, ws, C.byref(t), C.byref(s)) == 0
            assert 0 <= t.value < n_tiles and s.value not in (0, -1)
            bm, bn, bk = C.c_int(), C.c_int(), C.c_int()
            assert L.hpcdnn_sgemm_tile_info(t.value, C.byref(bm), C.byref(bn), C.byref(bk)) == 0
            tiles = -(-M // bm.value) * -(-N // bn.value)
            if s.value > 1:
                assert M * N * s.value * 4 <= ws and K // s.value >= 8 * bk.value
            elif s.value < -1:
                assert 0 < tiles % 256 and (tiles % 256) * (-s.value) * bm.value * bn.value * 4 <= ws
            else:
                assert s.value == 1
            rows, t1, t2 = C.c_int(-1), C.c_int(-2), C.c_int(-2)
            assert L.hpcdnn_sgemm_row_split(M, N, K, ws, C.byref(rows), C.byref(t1), C.byref(t2)) == 0
            if rows.value:
                assert 0 < rows.value < M and 0 <= t1.value < n_tiles and 0 <= t2.value < n_tiles
                assert L.hpcdnn_sgemm_tile_info(t1.value, C.byref(bm), None, None) == 0 and rows.value % bm.value == 0
            else:
                assert (t1.value, t2.value) == (-1, -1)


def test_cpp_header_helpers_compile_and_behave(tmp_path):
    """include/hpcdnn.hpp: the reference's host helpers (verify_matrix, verify_vector, cpu_gemm, CEIL_DIV, the timer;
    utils/utils.cu:60-103, utils.cuh:53-77) compile with a plain C++ compiler against the library and do what the
    reference's do."""
    import os
    import shutil
    import subprocess
    if shutil.which("g++") is None:
        pytest.skip("no host C++ compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    libdir = os.path.join(root, "hpcdeepneuralnetworks_amd", "lib")
    src = tmp_path / "t.cpp"
    src.write_text(r"""
#include <cstdio>
#include <vector>
#include "hpcdnn.hpp"
int main() {
    const int n = 8;
    std::vector<float> a(n * n), b(n * n, 0.f), c(n * n, 1.f), c2;
    for (int i = 0; i < n * n; ++i) a[i] = 0.25f * (i % 7) - 0.5f;
    for (int i = 0; i < n; ++i) b[i * n + i] = 1.f;                    // identity
    hpcdnn::cpu_gemm(2.f, 3.f, a.data(), b.data(), n, c.data());       // c = 2 a + 3
    for (int i = 0; i < n * n; ++i) if (c[i] != 2.f * a[i] + 3.f) return 1;
    c2 = c;
    if (!hpcdnn::verify_matrix(c.data(), c2.data(), n)) return 2;
    c2[5] += 0.009f;
    if (!hpcdnn::verify_matrix(c.data(), c2.data(), n)) return 3;       // within the absolute 1e-2
    c2[5] += 0.002f;
    if (hpcdnn::verify_matrix(c.data(), c2.data(), n)) return 4;        // beyond it
    std::vector<float> v = {1.f, -2.f, 100.f}, w = {1.004f, -2.009f, 100.4f};
    if (!hpcdnn::verify_vector(v.data(), w.data(), 3)) return 5;         // all within 5e-3 relative
    w[1] = -2.02f;
    if (hpcdnn::verify_vector(v.data(), w.data(), 3)) return 6;          // 1 % off on a negative element
    if (hpcdnn::ceil_div(10, 4) != 3 || hpcdnn::ceil_div(8, 4) != 2) return 7;
    hpcdnn::timer t;
    if (t.elapsed() < 0.0 || t.elapsed_msec(true) < 0.0) return 8;
    std::printf("%s\n", hpcdnn_version());
    return 0;
}
""")
    exe = tmp_path / "t"
    subprocess.run(["g++", "-std=c++17", "-O1", "-I", os.path.join(root, "include"), str(src), "-o", str(exe),
                    "-L", libdir, "-lhpcdnn", "-L/opt/rocm/lib", "-lamdhip64", f"-Wl,-rpath,{libdir}", "-Wl,-rpath,/opt/rocm/lib"],
                   check=True, capture_output=True, timeout=120)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, (out.returncode, out.stderr)
    assert out.stdout.startswith("hpcdnn")


def test_python_host_helpers_mirror_the_reference_checks():
    from hpcdeepneuralnetworks_amd import blas
    a = np.arange(16, dtype=np.float32).reshape(4, 4)
    b = a.copy()
    assert blas.verify_matrix(a, b, 4)
    b[1, 2] += 0.009
    assert blas.verify_matrix(a, b, 4)
    b[1, 2] += 0.002
    assert not blas.verify_matrix(a, b, 4)
    v = np.array([1.0, -2.0, 100.0], np.float32)
    assert blas.verify_vector(v, v * np.float32(1.004), 3)
    assert not blas.verify_vector(v, np.array([1.0, -2.02, 100.0], np.float32), 3)
