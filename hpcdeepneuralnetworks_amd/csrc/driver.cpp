// Command-line benchmark driver with the reference drivers' arguments and output format, on top of the C ABI.
//
//   hpcdnn_bench sgemm    <start> <end> <gap>                       kernel/sgemm/sgemm.cu:17-30,367-377
//   hpcdnn_bench ft_sgemm <start> <end> <gap> <first> <last>        kernel/ft_sgemm/sgemm.cu:14-27,186-196,413-422
//   hpcdnn_bench saxpy    [max_exp]                                 kernel/saxpy/saxpy.cu:57-66,122-182
//   hpcdnn_bench sdot     [max_exp]                                 kernel/sdot/sdot.cu:76-85,177-231
//
// sgemm prints the size row, a peak row and one row of GFLOP/s (square sizes, alpha = 1, beta = -1.5 like the
// reference).  ft_sgemm prints one `name = th.as_tensor([...])` line of GFLOP/s per series for M = N = size,
// K = 1024, the form the reference's plotting scripts read; series numbers follow the reference's list where a
// counterpart exists.  saxpy / sdot print the exponent row and a row of GFLOP/s (2 flop per element) for
// n = 2^10 ... 2^max_exp.  Every launch is bracketed by device synchronisation, as in the reference.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "hpcdnn.hpp"

#define HIP_OK(call)                                                                       \
    do {                                                                                   \
        hipError_t e_ = (call);                                                            \
        if (e_ != hipSuccess) {                                                            \
            std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
            std::exit(1);                                                                  \
        }                                                                                  \
    } while (0)
#define LIB_OK(call)                                                                         \
    do {                                                                                     \
        int rc_ = (call);                                                                    \
        if (rc_ != HPCDNN_OK) {                                                              \
            std::fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hpcdnn_error_string(rc_)); \
            std::exit(1);                                                                    \
        }                                                                                    \
    } while (0)

namespace {

constexpr double kPeakGflops = 157300.0;  // FP32 MFMA, MI355X
constexpr int kNumTests = 20;

float* device_floats(size_t n) {
    float* p = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&p), (n ? n : 1) * sizeof(float)));
    return p;
}

template <class F>
double timed_gflops(double flop_per_call, int calls, F&& launch) {
    hipEvent_t beg, end;
    HIP_OK(hipEventCreate(&beg));
    HIP_OK(hipEventCreate(&end));
    launch();  // first call pays for code loading
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipEventRecord(beg, nullptr));
    for (int i = 0; i < calls; ++i) {
        HIP_OK(hipDeviceSynchronize());
        launch();
        HIP_OK(hipDeviceSynchronize());
    }
    HIP_OK(hipEventRecord(end, nullptr));
    HIP_OK(hipEventSynchronize(end));
    float ms = 0.f;
    HIP_OK(hipEventElapsedTime(&ms, beg, end));
    HIP_OK(hipEventDestroy(beg));
    HIP_OK(hipEventDestroy(end));
    return flop_per_call * calls / 1e9 / (ms / 1e3);
}

// max |x - y| over n floats, on the host (the reference's verify_matrix is an absolute 1e-2 test, utils/utils.cu:60-75)
double max_abs_diff(const float* dx, const float* dy, size_t n) {
    std::vector<float> x(n), y(n);
    HIP_OK(hipMemcpy(x.data(), dx, n * sizeof(float), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(y.data(), dy, n * sizeof(float), hipMemcpyDeviceToHost));
    double worst = 0.0;
    for (size_t i = 0; i < n; ++i) {
        const double d = std::fabs(static_cast<double>(x[i]) - static_cast<double>(y[i]));
        if (!(d <= worst)) worst = d;  // NaN propagates
    }
    return worst;
}

void print_sizes(int start, int end, int gap) {
    for (int s = start; s <= end; s += gap) std::printf("%8.2d|", s);
    std::printf("\n");
}

int run_sgemm(int start, int end, int gap) {
    print_sizes(start, end, gap);
    for (int s = start; s <= end; s += gap) std::printf("%8.2f|", kPeakGflops);
    std::printf("\n");
    const size_t nn = static_cast<size_t>(end) * end;
    float *a = device_floats(nn), *b = device_floats(nn), *c = device_floats(nn);
    LIB_OK(hpcdnn_fill_uniform(a, static_cast<int64_t>(nn), 1, nullptr));
    LIB_OK(hpcdnn_fill_uniform(b, static_cast<int64_t>(nn), 2, nullptr));
    LIB_OK(hpcdnn_fill_uniform(c, static_cast<int64_t>(nn), 3, nullptr));
    const float alpha = 1.0f, beta = -1.5f;
    for (int i = 0; i < 40; ++i) LIB_OK(hpcdnn::sgemm(end, a, b, c, alpha, 0.0f));  // clocks up before the first size
    HIP_OK(hipDeviceSynchronize());
    for (int n = start; n <= end; n += gap) {
        // C keeps being rescaled by beta: refill so that it stays finite over the whole run
        LIB_OK(hpcdnn_fill_uniform(c, static_cast<int64_t>(nn), 3, nullptr));
        const double perf = timed_gflops(2.0 * n * n * n, kNumTests, [&] { LIB_OK(hpcdnn::sgemm(n, a, b, c, alpha, beta)); });
        std::printf("%8.2f,", perf);
        std::fflush(stdout);
    }
    std::printf("\n");
    HIP_OK(hipFree(a));
    HIP_OK(hipFree(b));
    HIP_OK(hipFree(c));
    return 0;
}

struct Series {
    int number;        // the reference's kernel_number (kernel/ft_sgemm/sgemm.cu:186)
    const char* name;  // the reference's series name (:187-188) where a counterpart exists
    int kind;          // 0 plain SGEMM, 1 offline ABFT, 2 ABFT without workspace, 3 ABFT with workspace, 4 wave-tile ABFT,
                       // 5 / 6 plain SGEMM / ABFT on column-major operands, 7 a name without a kernel (empty list)
    int tile;          // plain SGEMM: row of the tile table, -1 = chosen by the library; ABFT: tile class
};

// The reference's 16x16 ... 128x128 thread-tile classes map to the MFMA tile classes in the same order of size.
const Series kSeries[] = {
    {0, "hpcdnn_sgemm", 0, -1},        // the reference's vendor-library line (cuBLAS)
    {1, "kernel_sgemm_small", 0, 4},   // 64 x 64
    {2, "kernel_sgemm_medium", 0, 1},  // 128 x 128
    {3, "kernel_sgemm_large", 0, 0},   // 256 x 128
    {4, "kernel_sgemm_tall", 0, 2},    // 128 x 64
    {5, "kernel_sgemm_wide", 0, 3},    // 64 x 128
    {6, "kernel_sgemm_huge", 0, 8},    // 256 x 256
    {10, "abft_baseline", 1, -1},
    {12, "abft_kernel_medium", 2, 4},  // 64 x 64
    {13, "abft_kernel_large", 2, 1},   // 128 x 128
    {14, "abft_kernel_tall", 2, 3},    // 128 x 64
    {15, "abft_kernel_wide", 2, 2},    // 64 x 128
    {16, "abft_kernel_huge", 2, 0},    // 256 x 128
    // the thread-level kernel (kernel/ft_sgemm/sgemm.cu:188) has no counterpart on matrix cores: a matrix-core result
    // is spread over all 64 lanes of a wave, so the finest unit with accumulators of its own is the wave tile.  The
    // series keeps its name with an empty list, so that scripts that look the name up find it.
    {17, "thread_abft_kernel", 7, 0},
    // one checksum pair per wave tile (128 x 32 of the 256 x 128 tile): the matrix-core counterpart of the warp-level
    // kernel
    {18, "warp_abft_kernel", 4, 0},
    // no reference counterpart: checksum vectors from the pre-pass
    {19, "abft_kernel_huge_workspace", 3, 0},
    {20, "abft_kernel_large_workspace", 3, 1},
    {21, "abft_kernel_wide_workspace", 3, 2},
    // the reference's own operand layout, column-major C = A * B^T (kernel/ft_sgemm/sgemm.cu:111): the same device
    // buffers read as the column-major n x K, n x K and n x n matrices
    {22, "hpcdnn_sgemm_column_major", 5, -1},
    {23, "abft_kernel_huge_column_major", 6, 0},
};

int run_ft_sgemm(int start, int end, int gap, int first, int last) {
    for (int s = start; s <= end; s += gap) std::printf("%8.2d|", s);
    const int max_n = end, K = 1024;
    const size_t nn = static_cast<size_t>(max_n) * (max_n > K ? max_n : K);
    float *a = device_floats(nn), *b = device_floats(nn), *c = device_floats(nn), *c_ref = device_floats(nn);
    LIB_OK(hpcdnn_fill_uniform(a, static_cast<int64_t>(nn), 1, nullptr));
    LIB_OK(hpcdnn_fill_uniform(b, static_cast<int64_t>(nn), 2, nullptr));
    const float alpha = 1.0f, beta = -1.5f;
    // neither size grows monotonically with n (K-split room, SGEMV chunking): take the largest need over the sweep
    size_t ft_ws_bytes = 0, off_ws_bytes = 0;
    for (int n = start; n <= end; n += gap) {
        const size_t f = hpcdnn_workspace_bytes(HPCDNN_OP_FT_SGEMM, n, n, K);
        const size_t o = hpcdnn_workspace_bytes(HPCDNN_OP_OFFLINE_FT_SGEMM, n, n, K);
        if (f > ft_ws_bytes) ft_ws_bytes = f;
        if (o > off_ws_bytes) off_ws_bytes = o;
    }
    for (int n = start; n <= end; n += gap) {  // the column-major ABFT series (its query is that of the transposed problem)
        const size_t f = hpcdnn_workspace_bytes(HPCDNN_OP_FT_SGEMM_CM_NT, n, n, K);
        if (f > ft_ws_bytes) ft_ws_bytes = f;
    }
    void *ft_ws = nullptr, *off_ws = nullptr;
    HIP_OK(hipMalloc(&ft_ws, ft_ws_bytes ? ft_ws_bytes : 16));
    HIP_OK(hipMalloc(&off_ws, off_ws_bytes ? off_ws_bytes : 16));
    float* residuals = device_floats(2 * ((K + HPCDNN_OFFLINE_FT_PANEL_K - 1) / HPCDNN_OFFLINE_FT_PANEL_K));
    // optional SGEMM workspace (split-K / tail split), sized for the largest need over the sweep
    size_t gemm_ws_bytes = 16;
    for (int n = start; n <= end; n += gap) {
        const size_t need = hpcdnn_workspace_bytes(HPCDNN_OP_SGEMM, n, n, K);
        if (need > gemm_ws_bytes) gemm_ws_bytes = need;
    }
    void* gemm_ws = nullptr;
    HIP_OK(hipMalloc(&gemm_ws, gemm_ws_bytes));

    // correctness at the largest size, ABFT against plain SGEMM (the reference checks against the vendor library)
    {
        const int n = max_n;
        LIB_OK(hpcdnn_fill_uniform(c, static_cast<int64_t>(nn), 3, nullptr));
        LIB_OK(hpcdnn_fill_uniform(c_ref, static_cast<int64_t>(nn), 3, nullptr));
        LIB_OK(hpcdnn::sgemm(n, n, K, a, b, c_ref, alpha, beta));
        LIB_OK(hpcdnn::ft_sgemm(n, n, K, a, b, c, alpha, beta, nullptr, nullptr, ft_ws, ft_ws_bytes));
        HIP_OK(hipDeviceSynchronize());
        const double d = max_abs_diff(c, c_ref, static_cast<size_t>(n) * n);
        if (!(d <= 1e-2)) {
            std::printf("Failed to pass the correctness verification against plain SGEMM (max |diff| %g). Exited.\n", d);
            return 3;
        }
        // the same on the column-major operands the reference's check uses, cublasSgemm(N, T, ...) against its kernels
        // (kernel/ft_sgemm/sgemm.cu:111): the buffers read as the column-major n x K, n x K and n x n matrices
        LIB_OK(hpcdnn_fill_uniform(c, static_cast<int64_t>(nn), 3, nullptr));
        LIB_OK(hpcdnn_fill_uniform(c_ref, static_cast<int64_t>(nn), 3, nullptr));
        LIB_OK(hpcdnn_sgemm_cm_nt(n, n, K, a, n, b, n, c_ref, n, alpha, beta, nullptr, 0, nullptr));
        LIB_OK(hpcdnn_ft_sgemm_cm_nt(n, n, K, a, n, b, n, c, n, alpha, beta, 0.f, nullptr, nullptr, ft_ws, ft_ws_bytes, nullptr));
        HIP_OK(hipDeviceSynchronize());
        const double d_cm = max_abs_diff(c, c_ref, static_cast<size_t>(n) * n);
        if (!(d_cm <= 1e-2)) {
            std::printf("Failed to pass the correctness verification on column-major operands (max |diff| %g). Exited.\n", d_cm);
            return 3;
        }
        std::printf("finish verified!\n");
    }
    // the device has idled through the host-side comparison: bring its clocks back up before the first series
    for (int i = 0; i < 40; ++i) LIB_OK(hpcdnn::sgemm(max_n, max_n, K, a, b, c, alpha, 0.0f));
    HIP_OK(hipDeviceSynchronize());
    for (const Series& sr : kSeries) {
        if (sr.number < first) continue;
        if (sr.number > last) break;
        std::printf("%s = th.as_tensor([", sr.name);
        if (sr.kind == 7) {
            std::printf("])  # no per-thread checksums on matrix cores: the wave tile is the finest granularity (warp_abft_kernel)\n");
            continue;
        }
        for (int n = start; n <= end; n += gap) {
            LIB_OK(hpcdnn_fill_uniform(c, static_cast<int64_t>(nn), 3, nullptr));
            const double flop = 2.0 * n * static_cast<double>(n) * K;
            double perf = 0.0;
            switch (sr.kind) {
                case 0:
                    perf = timed_gflops(flop, kNumTests, [&] {
                        if (sr.tile < 0)
                            LIB_OK(hpcdnn_sgemm(n, n, K, a, K, b, n, c, n, alpha, beta, gemm_ws, gemm_ws_bytes, nullptr));
                        else
                            LIB_OK(hpcdnn_sgemm_ex(n, n, K, a, K, b, n, c, n, alpha, beta, nullptr, 0, sr.tile, 1, nullptr));
                    });
                    break;
                case 1:
                    perf = timed_gflops(flop, kNumTests, [&] {
                        LIB_OK(hpcdnn_offline_ft_sgemm(n, n, K, a, K, b, n, c, n, alpha, beta, nullptr, residuals, off_ws, off_ws_bytes, nullptr));
                    });
                    break;
                case 2:
                    perf = timed_gflops(flop, kNumTests, [&] {
                        LIB_OK(hpcdnn_ft_sgemm_ex(n, n, K, a, K, b, n, c, n, alpha, beta, 0.f, nullptr, nullptr, nullptr, 0, sr.tile, nullptr));
                    });
                    break;
                case 4: {
                    hpcdnn_ft_options opt{};
                    opt.tile_class = sr.tile;
                    opt.granularity = HPCDNN_FT_GRAN_WAVE;
                    perf = timed_gflops(flop, kNumTests, [&] {
                        LIB_OK(hpcdnn_ft_sgemm_opt(n, n, K, a, K, b, n, c, n, alpha, beta, 0.f, &opt, nullptr, ft_ws, ft_ws_bytes, nullptr));
                    });
                    break;
                }
                case 5:
                    perf = timed_gflops(flop, kNumTests, [&] {
                        LIB_OK(hpcdnn_sgemm_cm_nt(n, n, K, a, n, b, n, c, n, alpha, beta, gemm_ws, gemm_ws_bytes, nullptr));
                    });
                    break;
                case 6: {
                    hpcdnn_ft_options opt{};
                    opt.tile_class = sr.tile;
                    perf = timed_gflops(flop, kNumTests, [&] {
                        LIB_OK(hpcdnn_ft_sgemm_cm_nt(n, n, K, a, n, b, n, c, n, alpha, beta, 0.f, &opt, nullptr, ft_ws, ft_ws_bytes, nullptr));
                    });
                    break;
                }
                default:
                    perf = timed_gflops(flop, kNumTests, [&] {
                        LIB_OK(hpcdnn_ft_sgemm_ex(n, n, K, a, K, b, n, c, n, alpha, beta, 0.f, nullptr, nullptr, ft_ws, ft_ws_bytes, sr.tile, nullptr));
                    });
            }
            std::printf("%8.2f,", perf);
            std::fflush(stdout);
        }
        std::printf("])\n");
    }
    for (void* p : {static_cast<void*>(a), static_cast<void*>(b), static_cast<void*>(c), static_cast<void*>(c_ref), ft_ws,
                    off_ws, gemm_ws, static_cast<void*>(residuals)})
        HIP_OK(hipFree(p));
    return 0;
}

int run_vector(bool dot, int max_exp) {
    constexpr int kVecTests = 100;
    for (int e = 10; e <= max_exp; ++e) std::printf("%8.2d|", e);
    std::printf("\n");
    const size_t ws_bytes = hpcdnn_workspace_bytes(HPCDNN_OP_SDOT, 0, 0, 0);
    void* ws = nullptr;
    HIP_OK(hipMalloc(&ws, ws_bytes));
    LIB_OK(hpcdnn_workspace_init(ws, ws_bytes, nullptr));
    float* out = device_floats(1);
    for (int e = 10; e <= max_exp; ++e) {
        const int64_t n = int64_t{1} << e;
        // like the reference, every call of a series works on its own vectors (up to a 2 GiB cap per operand)
        int64_t copies = kVecTests;
        while (copies > 1 && copies * n > (int64_t{1} << 29)) copies /= 2;
        float *x = device_floats(static_cast<size_t>(copies * n)), *y = device_floats(static_cast<size_t>(copies * n));
        LIB_OK(hpcdnn_fill_uniform(x, copies * n, 1, nullptr));
        LIB_OK(hpcdnn_fill_uniform(y, copies * n, 2, nullptr));
        HIP_OK(hipDeviceSynchronize());
        hpcdnn::timer t;
        for (int i = 0; i < kVecTests; ++i) {
            const int64_t off = (i % copies) * n;
            if (dot)
                LIB_OK(hpcdnn_sdot(n, x + off, y + off, out, ws, ws_bytes, nullptr));
            else
                LIB_OK(hpcdnn_saxpy(n, 2.5f, x + off, y + off, nullptr));
        }
        HIP_OK(hipDeviceSynchronize());
        const double ms = t.elapsed_msec();
        std::printf("%4.2f,", 2.0 * kVecTests * static_cast<double>(n) / 1e9 / (ms / 1e3));
        std::fflush(stdout);
        HIP_OK(hipFree(x));
        HIP_OK(hipFree(y));
    }
    std::printf("\n");
    HIP_OK(hipFree(ws));
    HIP_OK(hipFree(out));
    return 0;
}

int usage() {
    std::fprintf(stderr,
                 "usage: hpcdnn_bench sgemm <start> <end> <gap>\n"
                 "       hpcdnn_bench ft_sgemm <start> <end> <gap> <first_series> <last_series>\n"
                 "       hpcdnn_bench saxpy [max_exp]\n"
                 "       hpcdnn_bench sdot [max_exp]\n");
    return 2;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc < 2) return usage();
    const char* what = argv[1];
    if (!std::strcmp(what, "sgemm") && argc == 5) {
        const int start = std::atoi(argv[2]), end = std::atoi(argv[3]), gap = std::atoi(argv[4]);
        if (start <= 0 || end < start || gap <= 0) return usage();
        return run_sgemm(start, end, gap);
    }
    if (!std::strcmp(what, "ft_sgemm") && argc == 7) {
        const int start = std::atoi(argv[2]), end = std::atoi(argv[3]), gap = std::atoi(argv[4]);
        if (start <= 0 || end < start || gap <= 0) return usage();
        return run_ft_sgemm(start, end, gap, std::atoi(argv[5]), std::atoi(argv[6]));
    }
    if ((!std::strcmp(what, "saxpy") || !std::strcmp(what, "sdot")) && argc <= 3) {
        const int max_exp = argc == 3 ? std::atoi(argv[2]) : 22;
        if (max_exp < 10 || max_exp > 28) return usage();
        return run_vector(what[1] == 'd', max_exp);
    }
    return usage();
}
