// C++ convenience layer over the C ABI (hpcdnn.h): the reference's spellings and argument order.
//
// The reference drivers launch `sgemm_k<<<...>>>(N, A, B, C, alpha, beta)` (kernel/sgemm/sgemm.cu:120-141),
// `[ft_]sgemm_<shape><<<...>>>(M, N, K, A, B, C, alpha, beta)` (kernel/ft_sgemm/sgemm.cu:114-165),
// `saxpy<<<...>>>(N, alpha, x, y)` (kernel/saxpy/saxpy.cu:110) and `_sdot<<<...>>>(N, x, y, out)`
// (kernel/sdot/sdot.cu:156), and call `cpu_gemm(alpha, beta, A, B, n, C)` (utils/utils.cuh:97) on the host.
// The overloads below take the same arguments on device pointers (row-major, packed leading dimensions),
// enqueue on the null stream and return the library's status code instead of nothing.
#pragma once

#include <chrono>
#include <cmath>

#include "hpcdnn.h"

namespace hpcdnn {

// kernel/sgemm series: square, ld = N
inline int sgemm(int N, const float* A, const float* B, float* C, float alpha, float beta) {
    return hpcdnn_sgemm(N, N, N, A, N, B, N, C, N, alpha, beta, nullptr, 0, nullptr);
}
// kernel/ft_sgemm family: general M, N, K (row-major here: lda = K, ldb = N, ldc = N)
inline int sgemm(int M, int N, int K, const float* A, const float* B, float* C, float alpha, float beta) {
    return hpcdnn_sgemm(M, N, K, A, K, B, N, C, N, alpha, beta, nullptr, 0, nullptr);
}
// the same family on its own column-major buffers: C (M x N) = alpha * A (M x K) * B (N x K)^T + beta * C with
// lda = M, ldb = N, ldc = M, as the driver hands them to cuBLAS (kernel/ft_sgemm/sgemm.cu:111)
inline int sgemm_cm_nt(int M, int N, int K, const float* A, const float* B, float* C, float alpha, float beta) {
    return hpcdnn_sgemm_cm_nt(M, N, K, A, M, B, N, C, M, alpha, beta, nullptr, 0, nullptr);
}
inline int ft_sgemm(int M, int N, int K, const float* A, const float* B, float* C, float alpha, float beta,
                    hpcdnn_ft_status* status = nullptr, const hpcdnn_fault* inject = nullptr, void* ws = nullptr,
                    size_t ws_bytes = 0) {
    return hpcdnn_ft_sgemm(M, N, K, A, K, B, N, C, N, alpha, beta, 0.0f, inject, status, ws, ws_bytes, nullptr);
}
// ft_sgemm_huge<<<...>>>(M, N, K, A, B, C, alpha, beta) on its own column-major buffers (lda = M, ldb = N, ldc = M;
// kernel/ft_sgemm/sgemm.cu:159-165); status records are those of the row-major N x M matrix C^T
inline int ft_sgemm_cm_nt(int M, int N, int K, const float* A, const float* B, float* C, float alpha, float beta,
                          hpcdnn_ft_status* status = nullptr, void* ws = nullptr, size_t ws_bytes = 0) {
    return hpcdnn_ft_sgemm_cm_nt(M, N, K, A, M, B, N, C, M, alpha, beta, 0.0f, nullptr, status, ws, ws_bytes, nullptr);
}
// the two offline routines of kernel/ft_sgemm/include/baseline_ft_sgemm.cuh (:1-34 and :36-91): their cuBLAS handle and
// eleven scratch vectors become one workspace of hpcdnn_workspace_bytes(HPCDNN_OP_OFFLINE_FT_SGEMM, M, N, K) bytes,
// `residuals` receives what the reference leaves in dRes (2 values per K panel of 256, 1 for the scalar routine)
inline int baseline_ft_sgemm(int M, int N, int K, const float* A, const float* B, float* C, float alpha, float beta,
                             float* residuals, void* ws, size_t ws_bytes) {
    return hpcdnn_offline_ft_sgemm(M, N, K, A, K, B, N, C, N, alpha, beta, nullptr, residuals, ws, ws_bytes, nullptr);
}
inline int offline_ft_sgemm(int M, int N, int K, const float* A, const float* B, float* C, float alpha, float beta,
                            float* residuals, void* ws, size_t ws_bytes) {
    return hpcdnn_offline_ft_sgemm_scalar(M, N, K, A, K, B, N, C, N, alpha, beta, nullptr, residuals, ws, ws_bytes, nullptr);
}
inline int saxpy(int N, float alpha, const float* x, float* y) { return hpcdnn_saxpy(N, alpha, x, y, nullptr); }
// `ws` from hpcdnn_workspace_bytes(HPCDNN_OP_SDOT, ...) / hpcdnn_workspace_init
inline int sdot(int N, const float* x, const float* y, float* out, void* ws, size_t ws_bytes) {
    return hpcdnn_sdot(N, x, y, out, ws, ws_bytes, nullptr);
}
inline void cpu_gemm(float alpha, float beta, const float* mat1, const float* mat2, int n, float* mat3) {
    hpcdnn_cpu_gemm(alpha, beta, mat1, mat2, n, mat3);
}

// The reference's acceptance checks on host arrays (utils/utils.cu:60-91): square n x n matrices agree when every
// element differs by at most 1e-2; vectors agree when every element is within 5e-3 relative.  (The reference
// divides by the signed first argument, so its vector check never fails on negative values; the magnitude is used
// here.)  Silent: the reference also prints the first offending element.
inline bool verify_matrix(const float* mat1, const float* mat2, int n) {
    for (long i = 0; i < static_cast<long>(n) * n; ++i)
        if (!(std::fabs(static_cast<double>(mat1[i]) - static_cast<double>(mat2[i])) <= 1e-2)) return false;
    return true;
}
inline bool verify_vector(const float* vec1, const float* vec2, int n) {
    for (int i = 0; i < n; ++i) {
        const double diff = std::fabs(static_cast<double>(vec1[i]) - static_cast<double>(vec2[i]));
        if (!(diff <= 5e-3 * std::fabs(static_cast<double>(vec1[i])))) return false;
    }
    return true;
}

// utils/utils.cuh:53 and :56-77
constexpr long ceil_div(long m, long n) { return (m + n - 1) / n; }

class timer {
public:
    timer() { reset(); }
    void reset() { t0_ = std::chrono::high_resolution_clock::now(); }
    double elapsed(bool reset_timer = false) {
        const auto t = std::chrono::high_resolution_clock::now();
        const double s = std::chrono::duration<double>(t - t0_).count();
        if (reset_timer) reset();
        return s;
    }
    double elapsed_msec(bool reset_timer = false) { return elapsed(reset_timer) * 1000.0; }

private:
    std::chrono::high_resolution_clock::time_point t0_;
};

}  // namespace hpcdnn
