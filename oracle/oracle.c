/*
 * CPU oracle for the FP32 BLAS-1/3 + ABFT-SGEMM path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this file; it is the checker the parity tests, the smoke test and the
 * cpu_baseline leg of the benchmark compare the HIP kernels against.
 *
 * Every function names the reference file:line whose behaviour it restates
 * (paths relative to the reference tree).  The reference holds no golden
 * vectors for this path, so each function is pinned by the tests in
 * tests/test_oracle.py against an independent routine (numpy float64 matmul,
 * exact rational arithmetic, closed forms) rather than against itself.
 *
 * Parity status:
 *   oracle_cpu_gemm, oracle_gemm_f64, oracle_saxpy, oracle_sdot_*: pinned.
 *   oracle_gemm_cm_nt_f64 (the column-major A*B^T of the ft_sgemm family):
 *     pinned to numpy float64 on the operands viewed column-major, with
 *     padded leading dimensions, and to a hand case that an untransposed B,
 *     a transposed A or a row-major C each fail.
 *   oracle_sgemv_f64: pinned (numpy float64 matrix-vector products, both
 *     orientations, padded leading dimension).
 *   oracle_offline_ft_sgemm: pinned to the closed form (residual sums are 0
 *     before the faulted panel and delta from it on, for any alpha, beta and
 *     panel width; final C equals the FP64 product plus the uncorrected
 *     fault).  The reference computes these sums and never checks or prints
 *     them (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:26-30), so it holds
 *     no expected values: bit-level agreement with cuBLAS is parity unpinned.
 *   oracle_offline_ft_sgemm_scalar (one scalar checksum per panel,
 *     baseline_ft_sgemm.cuh:36-91): pinned to numpy float64 (total of C minus
 *     the carried scalar, computed from whole-matrix sums) and to the same
 *     closed form.
 *   oracle_abft_*: pinned to the checksum algebra (e^T(AB) = (e^T A)B,
 *     (AB)e = A(Be)) and to the one known-answer case the reference holds
 *     (+1.0 at tile-local (0,1), threshold 0.1 -> row 0, col 1, magnitude 1;
 *     kernel/ft_sgemm/include/ft_sgemm_huge.cuh:40,145,263,358).
 *   oracle_ft_sgemm_weighted (the reference's second scheme, two row sums of
 *     B with weights [1,1,...] and [1,2,...], README.md:16-26): pinned by
 *     closed forms on exact-integer data (d1 = -delta, d2 = -(n+1) delta,
 *     every column of a tile located; two faults in a row detected, not
 *     corrected) and against an independent numpy composition; the reference
 *     only ever ran this scheme offline through cuBLAS and printed nothing,
 *     so it holds no expected values for it.
 *   oracle_recompute_element (the correction: the located accumulator formed
 *     again): pinned by K = 1 and exact-integer cases in which a corrected
 *     product must equal the fault-free one bit for bit.
 *   oracle_sgemm_device_order (a model of this library's own summation
 *     order, no reference counterpart): pinned to numpy float64 within the
 *     FP32 bound and to a hand case that k ascending fails.
 *   oracle_tile_acc (the FP32 accumulator model of the fault campaign):
 *     pinned to numpy float64 on a rectangular padded case, to a float
 *     accumulation-order case and to a hand case a transposed operand fails.
 *   oracle_ft_sgemm with tau < 0, oracle_abft_decide_lines with per-line
 *     thresholds, oracle_ft_sgemm_checked (verification every check_interval
 *     k with resync, ft_sgemm_huge.cuh:143,263-271): pinned to independent
 *     compositions of the pieces above and to closed forms (faults in
 *     different intervals are each located; a corrected fault leaves no trace
 *     in the later intervals).
 *   oracle_abft_set_rows_screen (the decision rule with the sides
 *     exchanged, for products one tile wide): pinned by that symmetry on
 *     random residual patterns and by the patterns that tell the screens apart.
 *   oracle_abft_relative_thresholds (data-scaled thresholds, an addition
 *     with no reference counterpart): pinned to closed forms (constant and
 *     single-entry tiles) and to its scaling laws.  Bit-level
 *     agreement with the reference's CUDA kernels or cuBLAS: parity unpinned
 *     (neither can be built or run without an NVIDIA toolchain, and the
 *     reference's ABFT locate/correct step is unfinished).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ RNG -- */

/* Counter-based generator shared (by definition, not by code) with the
 * device fill kernel: splitmix64 finaliser of seed*golden + index, top 24
 * bits mapped to the grid {-1 + j*2^-23}.  Replaces the reference's libc
 * rand() grid values (utils/utils.cu:28-44); the benchmark configurations ask
 * for seeded i.i.d. uniform[-1,1] inputs instead. */
static inline uint64_t mix64(uint64_t z) {
    z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
    z ^= z >> 27; z *= 0x94D049BB133111EBull;
    z ^= z >> 31;
    return z;
}

float oracle_uniform(uint64_t seed, uint64_t idx) {
    uint64_t z = mix64(seed * 0x9E3779B97F4A7C15ull + idx + 0x632BE59BD9B4E019ull);
    int32_t v = (int32_t)(z >> 40) - (1 << 23);           /* [-2^23, 2^23) */
    return (float)v * (1.0f / 8388608.0f);
}

void oracle_fill_uniform(float* dst, int64_t n, uint64_t seed) {
    for (int64_t i = 0; i < n; ++i) dst[i] = oracle_uniform(seed, (uint64_t)i);
}

/* Element (r,c) takes counter r*cols+c whatever the leading dimension is;
 * padding columns c >= cols are left untouched. */
void oracle_fill_uniform_matrix(float* dst, int rows, int cols, int ld, uint64_t seed) {
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c)
            dst[(size_t)r * ld + c] = oracle_uniform(seed, (uint64_t)r * (uint64_t)cols + (uint64_t)c);
}

int oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ----------------------------------------------------------------- GEMM -- */

/* utils/utils.cu:93-103: naive i-j-k row-major square GEMM with a float
 * accumulator, C = alpha*(A*B) + beta*C, ld = n, single thread. */
void oracle_cpu_gemm(float alpha, float beta, const float* mat1, const float* mat2, int n, float* mat3) {
    for (int i = 0; i < n; ++i) {
        for (int j = 0; j < n; ++j) {
            float temp = 0.0f;
            for (int k = 0; k < n; ++k) temp += mat1[(size_t)i * n + k] * mat2[(size_t)k * n + j];
            mat3[(size_t)i * n + j] = alpha * temp + beta * mat3[(size_t)i * n + j];
        }
    }
}

/* FP64-accumulated validator: for the given rows (rows == NULL means all M),
 *   ref[r][j]   = alpha * sum_k A[i,k]*B[k,j] + beta * C0[i,j]      (double)
 *   denom[r][j] = |alpha| * sum_k |A[i,k]||B[k,j]| + |beta|*|C0[i,j]|
 * with i = rows[r]; outputs are packed nrows x N.  C0 may be NULL when
 * beta == 0.  This is the Cref of the acceptance criterion
 * max |C - Cref| / (|A||B|)_ij <= 1e-5; it replaces the reference's
 * cuBLAS + abs 1e-2 check (utils/utils.cu:75-91). */
void oracle_gemm_f64_rows(int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                          const float* C0, int ldc, float alpha, float beta, const int* rows,
                          int nrows, double* ref, double* denom) {
    (void)M;
    #pragma omp parallel
    {
        double* acc = (double*)malloc(sizeof(double) * (size_t)N * 2);
        double* accabs = acc + N;
        #pragma omp for schedule(dynamic, 1)
        for (int r = 0; r < nrows; ++r) {
            int i = rows ? rows[r] : r;
            for (int j = 0; j < N; ++j) { acc[j] = 0.0; accabs[j] = 0.0; }
            for (int k = 0; k < K; ++k) {
                double a = (double)A[(size_t)i * lda + k];
                double aa = fabs(a);
                const float* brow = B + (size_t)k * ldb;
                for (int j = 0; j < N; ++j) {
                    double b = (double)brow[j];
                    acc[j] += a * b;
                    accabs[j] += aa * fabs(b);
                }
            }
            for (int j = 0; j < N; ++j) {
                double c0 = (beta != 0.0f && C0) ? (double)C0[(size_t)i * ldc + j] : 0.0;
                ref[(size_t)r * N + j] = (double)alpha * acc[j] + (double)beta * c0;
                if (denom) denom[(size_t)r * N + j] = fabs((double)alpha) * accabs[j] + fabs((double)beta) * fabs(c0);
            }
        }
        free(acc);
    }
}

/* The product of the reference's column-major family in FP64:
 *   C[m + n*ldc] = alpha * sum_k A[m + k*lda] * B[n + k*ldb] + beta * C0[m + n*ldc]
 * (C = alpha*A*B^T + beta*C with A M x K, B N x K, C M x N, all column-major:
 * the operand indexing of kernel/ft_sgemm/include/sgemm_huge.cuh:14-60 and the
 * cuBLAS call cublasSgemm(N, T, M, N, K, dA, M, dB, N, dC, M) that the driver
 * checks it against, kernel/ft_sgemm/sgemm.cu:111).  ref and denom are packed
 * column-major M x N (ld = M): ref[m + n*M]; denom as in oracle_gemm_f64_rows. */
void oracle_gemm_cm_nt_f64(int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                           const float* C0, int ldc, float alpha, float beta, double* ref, double* denom) {
    #pragma omp parallel for schedule(static)
    for (int n = 0; n < N; ++n) {
        for (int m = 0; m < M; ++m) {
            double acc = 0.0, accabs = 0.0;
            for (int k = 0; k < K; ++k) {
                double a = (double)A[(size_t)m + (size_t)k * lda], b = (double)B[(size_t)n + (size_t)k * ldb];
                acc += a * b;
                accabs += fabs(a) * fabs(b);
            }
            double c0 = (beta != 0.0f && C0) ? (double)C0[(size_t)m + (size_t)n * ldc] : 0.0;
            ref[(size_t)m + (size_t)n * M] = (double)alpha * acc + (double)beta * c0;
            if (denom) denom[(size_t)m + (size_t)n * M] = fabs((double)alpha) * accabs + fabs((double)beta) * fabs(c0);
        }
    }
}

/* max over the given rows of |C - ref| / denom (0/0 counts as 0, x/0 as inf). */
double oracle_gemm_max_err(int N, const float* C, int ldc, const int* rows, int nrows,
                           const double* ref, const double* denom) {
    double worst = 0.0;
    for (int r = 0; r < nrows; ++r) {
        int i = rows ? rows[r] : r;
        for (int j = 0; j < N; ++j) {
            double d = fabs((double)C[(size_t)i * ldc + j] - ref[(size_t)r * N + j]);
            double q = denom[(size_t)r * N + j];
            double e = (d == 0.0) ? 0.0 : (q > 0.0 ? d / q : INFINITY);
            if (e != e) return NAN;         /* a NaN anywhere is never accepted */
            if (e > worst) worst = e;
        }
    }
    return worst;
}

/* ---------------------------------------------------------- SAXPY / SDOT -- */

/* kernel/saxpy/saxpy.cu:38-48 (b = alpha*a + b) with the contraction nvcc
 * applies made explicit: one fused multiply-add per element. */
void oracle_saxpy(int64_t n, float alpha, const float* x, float* y) {
    for (int64_t i = 0; i < n; ++i) y[i] = fmaf(alpha, x[i], y[i]);
}

/* The same loop spread over the OpenMP pool (element-wise, so the bits do not depend on the thread count); the
 * multi-threaded CPU baseline of the benchmark. */
void oracle_saxpy_omp(int64_t n, float alpha, const float* x, float* y) {
    #pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) y[i] = fmaf(alpha, x[i], y[i]);
}

/* Double-accumulated dot product on one thread, k ascending: the single-thread CPU baseline of the benchmark
 * (oracle_sdot_f64 below is its OpenMP form, whose partial sums are added in thread order). */
double oracle_sdot_f64_serial(int64_t n, const float* x, const float* y) {
    double s = 0.0;
    for (int64_t i = 0; i < n; ++i) s += (double)x[i] * (double)y[i];
    return s;
}

/* Exact-as-possible dot product (double accumulate); the tolerance test for
 * kernel/sdot/sdot.cu:9-36 is relative to this. */
double oracle_sdot_f64(int64_t n, const float* x, const float* y) {
    double s = 0.0;
    #pragma omp parallel for reduction(+ : s) schedule(static)
    for (int64_t i = 0; i < n; ++i) s += (double)x[i] * (double)y[i];
    return s;
}

/* Single-thread float accumulate, the arithmetic of one reference thread
 * (temp += a[tid]*b[tid], kernel/sdot/sdot.cu:15-19) over the whole vector. */
float oracle_sdot_f32(int64_t n, const float* x, const float* y) {
    float s = 0.0f;
    for (int64_t i = 0; i < n; ++i) s = fmaf(x[i], y[i], s);
    return s;
}

/* ----------------------------------------------------------------- ABFT -- */

/* Per-tile status record, same fields as the device record. */
typedef struct {
    int32_t flag;            /* 0 clean, 1 single fault located and corrected, 2 detected, not correctable */
    int32_t row, col;        /* tile-local location of the corrected element, -1 if none */
    int32_t n_bad_rows, n_bad_cols;
    float row_residual;      /* signed residual (reference - observed) of the located row, else 0 */
    float col_residual;      /* same for the located column */
    float max_clean_residual;/* largest |residual| among the lines judged clean */
} oracle_ft_status;

/* Accumulator block of one output tile as the model sees it: float
 * accumulator, one fused multiply-add per k, k ascending (the arithmetic of
 * one reference thread's `tab` FMA chain, kernel_13.cuh:55-81).  acc is
 * tm x tn packed. */
void oracle_tile_acc(int tm, int tn, int K, const float* A, int lda, const float* B, int ldb, float* acc) {
    #pragma omp parallel for schedule(static)
    for (int m = 0; m < tm; ++m) {
        float* arow = acc + (size_t)m * tn;
        for (int n = 0; n < tn; ++n) arow[n] = 0.0f;
        for (int k = 0; k < K; ++k) {
            float a = A[(size_t)m * lda + k];
            const float* brow = B + (size_t)k * ldb;
            for (int n = 0; n < tn; ++n) arow[n] = fmaf(a, brow[n], arow[n]);
        }
    }
}

/* Step 1 (encode) of the online-ABFT scheme for one output tile
 * (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:67-102,442-474; explicit form in
 * ft_sgemm_large.cuh:372-436): reference checksums formed from A and B only,
 *     cc_ref[n] = sum_k (sum_m A[m,k]) * B[k,n]      (= e^T A B)
 *     cr_ref[m] = sum_k A[m,k] * (sum_n B[k,n])      (= A B e)
 * A and B point at the tile's first row / first column. */
void oracle_abft_reference_checksums(int tm, int tn, int K, const float* A, int lda, const float* B,
                                     int ldb, double* cr_ref, double* cc_ref) {
    for (int m = 0; m < tm; ++m) cr_ref[m] = 0.0;
    for (int n = 0; n < tn; ++n) cc_ref[n] = 0.0;
    for (int k = 0; k < K; ++k) {
        double a_c = 0.0, b_r = 0.0;
        for (int m = 0; m < tm; ++m) a_c += (double)A[(size_t)m * lda + k];
        for (int n = 0; n < tn; ++n) b_r += (double)B[(size_t)k * ldb + n];
        for (int n = 0; n < tn; ++n) cc_ref[n] += a_c * (double)B[(size_t)k * ldb + n];
        for (int m = 0; m < tm; ++m) cr_ref[m] += (double)A[(size_t)m * lda + k] * b_r;
    }
}

/* Steps 2-3 (observe, residual; ft_sgemm_huge.cuh:147-171, :200-262):
 * residual = reference checksum minus the line sum of the accumulator block
 * acc (tm x tn, row stride ldacc) taken BEFORE the alpha/beta epilogue. */
void oracle_abft_observe(int tm, int tn, const float* acc, int ldacc, const double* cr_ref,
                         const double* cc_ref, double* dr, double* dc) {
    for (int m = 0; m < tm; ++m) {
        double s = 0.0;
        for (int n = 0; n < tn; ++n) s += (double)acc[(size_t)m * ldacc + n];
        dr[m] = cr_ref[m] - s;
    }
    for (int n = 0; n < tn; ++n) {
        double s = 0.0;
        for (int m = 0; m < tm; ++m) s += (double)acc[(size_t)m * ldacc + n];
        dc[n] = cc_ref[n] - s;
    }
}

/* Steps 1-3 in one call. */
void oracle_abft_residuals(int tm, int tn, int K, const float* A, int lda, const float* B, int ldb,
                           const float* acc, int ldacc, double* dr, double* dc) {
    double* cr_ref = (double*)malloc(sizeof(double) * (size_t)(tm + tn));
    double* cc_ref = cr_ref + tm;
    oracle_abft_reference_checksums(tm, tn, K, A, lda, B, ldb, cr_ref, cc_ref);
    oracle_abft_observe(tm, tn, acc, ldacc, cr_ref, cc_ref, dr, dc);
    free(cr_ref);
}

/* Steps 4-6: threshold each line (|d| > tau marks it faulty,
 * ft_sgemm_huge.cuh:263-271), locate the element where one faulty row meets
 * one faulty column (:273-296) and report the correction to apply.  The
 * reference subtracts round(sum |row residuals|) (:358), which is only right
 * for its +1.0 test fault; the signed row residual measures the fault for any
 * magnitude, but adding it back would leave the row's fault-free rounding
 * noise in one element, so the models below compute the located accumulator
 * again (oracle_recompute_element) and use the residual as a report only.
 * Like the reference, which acts on a tile only when a column checksum AND a
 * row checksum disagree (`if (error > err_bound1 && error1 > err_bound1)`,
 * ft_sgemm_huge.cuh:289), the column checksums screen: a tile none of whose
 * columns exceeds its threshold is clean (flag 0, no bad lines), and its rows
 * are not looked at - neither counted nor part of max_clean_residual.  With a
 * flagged column the rows are thresholded too: one faulty row x one faulty
 * column -> located (flag 1), anything else -> detected only (flag 2).
 * Returns the signed row residual of the located row (0 when nothing is located). */
/* Which side screens.  0 (default): the columns, as described above.  1: the rows - the library's choice for
 * products one tile wide with a workspace, whose operand A is streamed once and gets no checksum vector: there the
 * row checksums (from the small B) are compared every time and the columns only when a row disagrees.  The rule is
 * the same with the two sides exchanged. */
static int g_rows_screen = 0;
void oracle_abft_set_rows_screen(int on) { g_rows_screen = on != 0; }

/* Per-line thresholds: tau_r[m] for row m, tau_c[n] for column n. */
float oracle_abft_decide_lines(int tm, int tn, const double* dr, const double* dc, const double* tau_r,
                               const double* tau_c, oracle_ft_status* st) {
    int nbr = 0, nbc = 0, r = -1, c = -1;
    double clean = 0.0;
    if (g_rows_screen) {
        for (int m = 0; m < tm; ++m) {
            if (fabs(dr[m]) > tau_r[m]) { ++nbr; r = m; }
            else if (fabs(dr[m]) > clean) clean = fabs(dr[m]);
        }
        for (int n = 0; n < tn && nbr > 0; ++n) {
            if (fabs(dc[n]) > tau_c[n]) { ++nbc; c = n; }
            else if (fabs(dc[n]) > clean) clean = fabs(dc[n]);
        }
    } else {
        for (int n = 0; n < tn; ++n) {
            if (fabs(dc[n]) > tau_c[n]) { ++nbc; c = n; }
            else if (fabs(dc[n]) > clean) clean = fabs(dc[n]);
        }
        /* the rows are looked at only when a column checksum disagrees (see the comment above) */
        for (int m = 0; m < tm && nbc > 0; ++m) {
            if (fabs(dr[m]) > tau_r[m]) { ++nbr; r = m; }
            else if (fabs(dr[m]) > clean) clean = fabs(dr[m]);
        }
    }
    st->n_bad_rows = nbr;
    st->n_bad_cols = nbc;
    st->max_clean_residual = (float)clean;
    st->row = -1; st->col = -1; st->row_residual = 0.0f; st->col_residual = 0.0f;
    if (nbr == 0 && nbc == 0) { st->flag = 0; return 0.0f; }
    if (nbr == 1 && nbc == 1) {
        st->flag = 1; st->row = r; st->col = c;
        st->row_residual = (float)dr[r];
        st->col_residual = (float)dc[c];
        return (float)dr[r];
    }
    st->flag = 2;
    return 0.0f;
}

/* One absolute threshold for every line (the reference's scheme: 0.1, kernel/ft_sgemm/include/ft_sgemm_huge.cuh:30,263). */
float oracle_abft_decide(int tm, int tn, const double* dr, const double* dc, float tau,
                         oracle_ft_status* st) {
    double* t = (double*)malloc(sizeof(double) * (size_t)(tm + tn));
    for (int i = 0; i < tm + tn; ++i) t[i] = (double)tau;
    float fix = oracle_abft_decide_lines(tm, tn, dr, dc, t, t + tm, st);
    free(t);
    return fix;
}

/* Data-scaled thresholds (no reference counterpart; the reference's thresholds are constants): a line of n
 * accumulators gets rel * sqrt(n) * max(mean |acc| over the line, mean |acc| over the tile), with
 * rel = factor * 2.56e-7 * sqrt(max(K, 64)) (4.3 units of FP32 rounding per sqrt(K)): the rounding noise of a sum of n
 * accumulators grows like sqrt(n) times their magnitude, and that of one accumulator like sqrt(K) times the rounding
 * unit.  The tile mean keeps a short or cancelling line (whose own |acc| says little about the size of its terms)
 * from getting a threshold below its noise; the floor on K covers the rounding of the sums themselves, which does
 * not shrink with K. */
void oracle_abft_relative_thresholds(int tm, int tn, int K, const float* acc, int ldacc, float factor,
                                     double* tau_r, double* tau_c) {
    float rel = factor * 2.56e-7f * sqrtf((float)(K > 64 ? K : 64));
    float rs = rel / sqrtf((float)tn), cs = rel / sqrtf((float)tm);
    double total = 0.0;
    for (int n = 0; n < tn; ++n) tau_c[n] = 0.0;
    for (int m = 0; m < tm; ++m) {
        double s = 0.0;
        for (int n = 0; n < tn; ++n) {
            double v = fabs((double)acc[(size_t)m * ldacc + n]);
            s += v;
            tau_c[n] += v;
        }
        tau_r[m] = s;
        total += s;
    }
    float mean = (float)total / ((float)tm * (float)tn);
    float row_floor = rel * sqrtf((float)tn) * mean, col_floor = rel * sqrtf((float)tm) * mean;
    for (int m = 0; m < tm; ++m) {
        float t = (float)tau_r[m] * rs;
        tau_r[m] = (double)(t > row_floor ? t : row_floor);
    }
    for (int n = 0; n < tn; ++n) {
        float t = (float)tau_c[n] * cs;
        tau_c[n] = (double)(t > col_floor ? t : col_floor);
    }
}

/* Step 6 (correct): the located accumulator computed again from row `a` of A (stride 1) and column `b` of B
 * (stride ldb) over k0 <= k < k1, in the arithmetic of oracle_tile_acc (float accumulator, one fused multiply-add
 * per k, k ascending).  It replaces the faulty accumulator, so a corrected product has the bits of a fault-free one
 * (the reference's correction site, ft_sgemm_huge.cuh:352-371, subtracts a rounded residual instead). */
float oracle_recompute_element(int k0, int k1, const float* a, const float* b, int ldb) {
    float acc = 0.0f;
    for (int k = k0; k < k1; ++k) acc = fmaf(a[k], b[(size_t)k * ldb], acc);
    return acc;
}

/* Row-major SGEMM in the arithmetic of the device's tile kernels: a float accumulator per element, one fused
 * multiply-add per k, k taken K step by K step (16 values) in the order 0,4,1,5,2,6,3,7,8,12,9,13,10,14,11,15 - the
 * order in which the 32x32x2 FP32 matrix-core instruction (two chained FMAs, lanes 0-31's k first) meets the
 * k-permuted operand fragments -, then C = alpha*acc + beta*C (C is not read when beta == 0).  A model of this
 * library's kernels, not of the reference: it predicts the bits of an unsplit product. */
void oracle_sgemm_device_order(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                               int ldc, float alpha, float beta) {
    static const int order[16] = {0, 4, 1, 5, 2, 6, 3, 7, 8, 12, 9, 13, 10, 14, 11, 15};
    #pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        float* acc = (float*)calloc((size_t)(N > 0 ? N : 1), sizeof(float));
        for (int k0 = 0; k0 < K; k0 += 16)
            for (int o = 0; o < 16; ++o) {
                int k = k0 + order[o];
                if (k >= K) continue;
                float a = A[(size_t)m * lda + k];
                const float* brow = B + (size_t)k * ldb;
                for (int n = 0; n < N; ++n) acc[n] = fmaf(a, brow[n], acc[n]);
            }
        for (int n = 0; n < N; ++n) {
            float* c = &C[(size_t)m * ldc + n];
            float v = alpha * acc[n];
            *c = (beta == 0.0f) ? v : fmaf(beta, *c, v);
        }
        free(acc);
    }
}

/* Whole-matrix model: C = alpha*acc + beta*C with acc = A*B accumulated in
 * float (k ascending), one fault (tile index in row-major tile order,
 * tile-local i, j, delta added to acc before verification) or none
 * (fault_tile < 0), tiles of tile_m x tile_n (edge tiles are clipped), tau > 0
 * absolute or tau <= 0 data-scaled with factor -tau (factor 1 for tau == 0), one
 * status record per tile.  Mirrors the device entry point's contract; used on
 * sizes the CPU finishes in seconds. */
void oracle_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                     int ldc, float alpha, float beta, int tile_m, int tile_n, float tau,
                     int fault_tile, int fault_i, int fault_j, float fault_delta,
                     oracle_ft_status* status) {
    int ntm = (M + tile_m - 1) / tile_m, ntn = (N + tile_n - 1) / tile_n;
    #pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < ntm * ntn; ++t) {
        int bm = t / ntn, bn = t % ntn;
        int m0 = bm * tile_m, n0 = bn * tile_n;
        int tm = (M - m0 < tile_m) ? M - m0 : tile_m;
        int tn = (N - n0 < tile_n) ? N - n0 : tile_n;
        float* acc = (float*)calloc((size_t)tm * tn, sizeof(float));
        double* dr = (double*)malloc(sizeof(double) * (size_t)(tm + tn));
        double* dc = dr + tm;
        for (int m = 0; m < tm; ++m)
            for (int k = 0; k < K; ++k) {
                float a = A[(size_t)(m0 + m) * lda + k];
                const float* brow = B + (size_t)k * ldb + n0;
                float* arow = acc + (size_t)m * tn;
                for (int n = 0; n < tn; ++n) arow[n] = fmaf(a, brow[n], arow[n]);
            }
        if (t == fault_tile && fault_i < tm && fault_j < tn) acc[(size_t)fault_i * tn + fault_j] += fault_delta;
        oracle_abft_residuals(tm, tn, K, A + (size_t)m0 * lda, lda, B + n0, ldb, acc, tn, dr, dc);
        float fix;
        if (tau <= 0.0f) {
            double* thr = (double*)malloc(sizeof(double) * (size_t)(tm + tn));
            oracle_abft_relative_thresholds(tm, tn, K, acc, tn, tau < 0.0f ? -tau : 1.0f, thr, thr + tm);
            fix = oracle_abft_decide_lines(tm, tn, dr, dc, thr, thr + tm, &status[t]);
            free(thr);
        } else {
            fix = oracle_abft_decide(tm, tn, dr, dc, tau, &status[t]);
        }
        (void)fix;
        if (status[t].flag == 1)
            acc[(size_t)status[t].row * tn + status[t].col] =
                oracle_recompute_element(0, K, A + (size_t)(m0 + status[t].row) * lda, B + n0 + status[t].col, ldb);
        for (int m = 0; m < tm; ++m)
            for (int n = 0; n < tn; ++n) {
                float* c = &C[(size_t)(m0 + m) * ldc + n0 + n];
                float v = alpha * acc[(size_t)m * tn + n];
                *c = (beta == 0.0f) ? v : fmaf(beta, *c, v);
            }
        free(acc);
        free(dr);
    }
}

/* One soft error with the verification it precedes: delta is added to accumulator (row, col) of tile `tile` right
 * before verification number `check` of that tile (0 = the first).  A model run that verifies only once, after the
 * whole K loop, injects every fault before that one verification. */
typedef struct {
    int32_t tile, row, col;
    float delta;
    int32_t check;
} oracle_fault_at;

/* The whole-matrix model of the reference's second scheme ("kernel 2", kernel/ft_sgemm/README.md:16-26: double row
 * sums of B with e1 = [1, 1, ...] and e2 = [1, 2, ..., N]; its locator is left in comments at
 * kernel/ft_sgemm/include/ft_sgemm_huge.cuh:299-310): per tile the references r1 = A (B e1), r2 = A (B e2) - weights
 * counted over the tile's columns - are compared with the plain and the weighted row sums of the accumulators.  A row
 * whose plain residual d1 exceeds its threshold is faulty; with one fault delta in column n its residuals are
 * d1 = -delta, d2 = -(n + 1) delta, so the column is round(d2 / d1) - 1 (clamped into the tile).  One faulty row: that
 * element is computed again (oracle_recompute_element); the location is confirmed when that changed the element by d1
 * to within the row's threshold + 2^-20 |d1| -> flag 1, n_bad_cols 1, row/col set, row_residual = d1, col_residual = d2.  Not
 * confirmed (two faults in the row, or a fault lost in the rounding of the weighted sums) or more faulty rows ->
 * flag 2, n_bad_cols 0.  Computing a healthy element again changes nothing, so a wrong column does no harm.
 * tau as for oracle_ft_sgemm; every fault is added before the one verification. */
void oracle_ft_sgemm_weighted(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                              int ldc, float alpha, float beta, int tile_m, int tile_n, float tau,
                              int n_faults, const oracle_fault_at* faults, oracle_ft_status* status) {
    int ntm = (M + tile_m - 1) / tile_m, ntn = (N + tile_n - 1) / tile_n;
    #pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < ntm * ntn; ++t) {
        int bm = t / ntn, bn = t % ntn;
        int m0 = bm * tile_m, n0 = bn * tile_n;
        int tm = (M - m0 < tile_m) ? M - m0 : tile_m;
        int tn = (N - n0 < tile_n) ? N - n0 : tile_n;
        float* acc = (float*)calloc((size_t)tm * tn, sizeof(float));
        double* buf = (double*)calloc((size_t)(3 * tm + tn) + 2 * (size_t)(K > 0 ? K : 1), sizeof(double));
        double *d1 = buf, *d2 = buf + tm, *thr = buf + 2 * tm;      /* thr: tm row thresholds, then tn column ones (unused) */
        double *b1 = buf + 3 * tm + tn, *b2 = b1 + (K > 0 ? K : 1);
        for (int m = 0; m < tm; ++m)
            for (int k = 0; k < K; ++k) {
                float a = A[(size_t)(m0 + m) * lda + k];
                const float* brow = B + (size_t)k * ldb + n0;
                float* arow = acc + (size_t)m * tn;
                for (int n = 0; n < tn; ++n) arow[n] = fmaf(a, brow[n], arow[n]);
            }
        for (int f = 0; f < n_faults; ++f)
            if (faults[f].tile == t && faults[f].row < tm && faults[f].col < tn)
                acc[(size_t)faults[f].row * tn + faults[f].col] += faults[f].delta;
        for (int k = 0; k < K; ++k) {
            double s1 = 0.0, s2 = 0.0;
            for (int n = 0; n < tn; ++n) {
                double v = (double)B[(size_t)k * ldb + n0 + n];
                s1 += v;
                s2 += (double)(n + 1) * v;
            }
            b1[k] = s1;
            b2[k] = s2;
        }
        for (int m = 0; m < tm; ++m) {
            double r1 = 0.0, r2 = 0.0, o1 = 0.0, o2 = 0.0;
            for (int k = 0; k < K; ++k) {
                double a = (double)A[(size_t)(m0 + m) * lda + k];
                r1 += a * b1[k];
                r2 += a * b2[k];
            }
            for (int n = 0; n < tn; ++n) {
                double v = (double)acc[(size_t)m * tn + n];
                o1 += v;
                o2 += (double)(n + 1) * v;
            }
            d1[m] = r1 - o1;
            d2[m] = r2 - o2;
        }
        if (tau <= 0.0f) oracle_abft_relative_thresholds(tm, tn, K, acc, tn, tau < 0.0f ? -tau : 1.0f, thr, thr + tm);
        else for (int m = 0; m < tm; ++m) thr[m] = (double)tau;
        oracle_ft_status st;
        memset(&st, 0, sizeof st);
        st.row = st.col = -1;
        int nbr = 0, r = -1;
        double clean = 0.0;
        for (int m = 0; m < tm; ++m) {
            if (fabs(d1[m]) > thr[m]) { ++nbr; r = m; }
            else if (fabs(d1[m]) > clean) clean = fabs(d1[m]);
        }
        st.n_bad_rows = nbr;
        st.max_clean_residual = (float)clean;
        if (nbr == 1) {
            float f1 = (float)d1[r], f2 = (float)d2[r];
            int c = (int)rintf(f2 / f1) - 1;
            c = c < 0 ? 0 : (c >= tn ? tn - 1 : c);
            float* e = &acc[(size_t)r * tn + c];
            float again = oracle_recompute_element(0, K, A + (size_t)(m0 + r) * lda, B + n0 + c, ldb);
            float change = again - *e;
            *e = again;
            /* (the row's threshold plus sixteen rounding units of the residual: the observed sums of a row that
             * holds a fault of thousands of thresholds are themselves only good to a few units of its size) */
            if (fabsf(change - f1) <= (float)thr[r] + 0x1p-20f * fabsf(f1)) {
                st.flag = 1; st.n_bad_cols = 1; st.row = r; st.col = c;
                st.row_residual = f1; st.col_residual = f2;
            } else {
                st.flag = 2;
            }
        } else if (nbr > 1) {
            st.flag = 2;
        }
        status[t] = st;
        for (int m = 0; m < tm; ++m)
            for (int n = 0; n < tn; ++n) {
                float* c = &C[(size_t)(m0 + m) * ldc + n0 + n];
                float v = alpha * acc[(size_t)m * tn + n];
                *c = (beta == 0.0f) ? v : fmaf(beta, *c, v);
            }
        free(acc);
        free(buf);
    }
}

/* The whole-matrix model with the reference's verification cadence: the accumulators of a tile are verified every
 * check_interval values of k inside the K loop (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:143, `if (k % 256 == 0)`)
 * and once more after the last k, against reference checksums that cover the k range done so far; after every
 * verification the references are re-synchronised with the accumulators (`C_c -= C_c_`, ft_sgemm_huge.cuh:263-271):
 * what is left of each line's residual after the correction is absorbed, so the next verification sees only what
 * happened since this one.  (The reference leaves a line that exceeded the threshold unsynchronised and has no
 * working locate/correct step; here every line that a verification looked at is re-synchronised - the columns always,
 * the rows when a column was flagged, see oracle_abft_decide_lines -, a located element is corrected first, and a
 * verification that could not locate its fault marks the tile uncorrectable for good.)
 * check_interval <= 0: one verification after the K loop (then this is oracle_ft_sgemm with several faults).
 * The tile's record merges its verifications: bad-line counts add up, flag 2 if any verification was
 * uncorrectable, else 1 if any corrected an element; row, col and the residuals are those of the first correction;
 * max_clean_residual is the largest over all verifications. */
void oracle_ft_sgemm_checked(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                             int ldc, float alpha, float beta, int tile_m, int tile_n, float tau,
                             int check_interval, int n_faults, const oracle_fault_at* faults,
                             oracle_ft_status* status) {
    int ntm = (M + tile_m - 1) / tile_m, ntn = (N + tile_n - 1) / tile_n;
    int ci = (check_interval > 0 && check_interval < K) ? check_interval : (K > 0 ? K : 1);
    int checks = (K > 0) ? (K + ci - 1) / ci : 1;
    #pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < ntm * ntn; ++t) {
        int bm = t / ntn, bn = t % ntn;
        int m0 = bm * tile_m, n0 = bn * tile_n;
        int tm = (M - m0 < tile_m) ? M - m0 : tile_m;
        int tn = (N - n0 < tile_n) ? N - n0 : tile_n;
        float* acc = (float*)calloc((size_t)tm * tn, sizeof(float));
        double* buf = (double*)calloc((size_t)(tm + tn) * 5, sizeof(double));
        double *cr_ref = buf, *cc_ref = buf + tm;              /* cumulative references */
        double *off_r = buf + (tm + tn), *off_c = off_r + tm;  /* what re-synchronisation has absorbed so far */
        double *dr = buf + 2 * (tm + tn), *dc = dr + tm;
        double *part_r = buf + 3 * (tm + tn), *part_c = part_r + tm;
        double *thr = buf + 4 * (tm + tn);
        oracle_ft_status rec;
        memset(&rec, 0, sizeof rec);
        rec.row = rec.col = -1;
        for (int c = 0; c < checks; ++c) {
            int k0 = c * ci, k1 = (k0 + ci < K) ? k0 + ci : K;
            for (int m = 0; m < tm; ++m)
                for (int k = k0; k < k1; ++k) {
                    float a = A[(size_t)(m0 + m) * lda + k];
                    const float* brow = B + (size_t)k * ldb + n0;
                    float* arow = acc + (size_t)m * tn;
                    for (int n = 0; n < tn; ++n) arow[n] = fmaf(a, brow[n], arow[n]);
                }
            if (k1 > k0) {
                oracle_abft_reference_checksums(tm, tn, k1 - k0, A + (size_t)m0 * lda + k0, lda,
                                                B + (size_t)k0 * ldb + n0, ldb, part_r, part_c);
                for (int m = 0; m < tm; ++m) cr_ref[m] += part_r[m];
                for (int n = 0; n < tn; ++n) cc_ref[n] += part_c[n];
            }
            for (int f = 0; f < n_faults; ++f)
                if (faults[f].tile == t && (checks == 1 || faults[f].check == c) && faults[f].row < tm && faults[f].col < tn)
                    acc[(size_t)faults[f].row * tn + faults[f].col] += faults[f].delta;
            /* residual against the re-synchronised references */
            for (int m = 0; m < tm; ++m) part_r[m] = cr_ref[m] - off_r[m];
            for (int n = 0; n < tn; ++n) part_c[n] = cc_ref[n] - off_c[n];
            oracle_abft_observe(tm, tn, acc, tn, part_r, part_c, dr, dc);
            oracle_ft_status cur;
            float fix;
            if (tau <= 0.0f) {
                oracle_abft_relative_thresholds(tm, tn, K, acc, tn, tau < 0.0f ? -tau : 1.0f, thr, thr + tm);
                fix = oracle_abft_decide_lines(tm, tn, dr, dc, thr, thr + tm, &cur);
            } else {
                fix = oracle_abft_decide(tm, tn, dr, dc, tau, &cur);
            }
            (void)fix;
            double changed = 0.0;  /* what the correction added to the located accumulator */
            if (cur.flag == 1) {
                float* e = &acc[(size_t)cur.row * tn + cur.col];
                float again = oracle_recompute_element(0, k1, A + (size_t)(m0 + cur.row) * lda, B + n0 + cur.col, ldb);
                changed = (double)again - (double)*e;
                *e = again;
            }
            /* re-synchronise every line that was looked at (the columns; the rows when a column was flagged) with
             * what it shows after the correction */
            for (int m = 0; m < tm && cur.n_bad_cols > 0; ++m) off_r[m] += dr[m] - ((cur.flag == 1 && m == cur.row) ? changed : 0.0);
            for (int n = 0; n < tn; ++n) off_c[n] += dc[n] - ((cur.flag == 1 && n == cur.col) ? changed : 0.0);
            /* merge */
            rec.n_bad_rows += cur.n_bad_rows;
            rec.n_bad_cols += cur.n_bad_cols;
            if (cur.max_clean_residual > rec.max_clean_residual) rec.max_clean_residual = cur.max_clean_residual;
            if (cur.flag == 2) rec.flag = 2;
            else if (cur.flag == 1 && rec.flag == 0) {
                rec.flag = 1; rec.row = cur.row; rec.col = cur.col;
                rec.row_residual = cur.row_residual; rec.col_residual = cur.col_residual;
            }
        }
        if (rec.flag == 2) { rec.row = rec.col = -1; rec.row_residual = rec.col_residual = 0.0f; }
        status[t] = rec;
        for (int m = 0; m < tm; ++m)
            for (int n = 0; n < tn; ++n) {
                float* c = &C[(size_t)(m0 + m) * ldc + n0 + n];
                float v = alpha * acc[(size_t)m * tn + n];
                *c = (beta == 0.0f) ? v : fmaf(beta, *c, v);
            }
        free(acc);
        free(buf);
    }
}

/* ----------------------------------------------- SGEMV / offline ABFT -- */

/* Row-major SGEMV in FP64 on an M x N matrix: trans = 0: out[m] = alpha *
 * sum_n A[m][n] x[n] + beta * y[m]; trans = 1: out[n] = alpha * sum_m A[m][n]
 * x[m] + beta * y[n]; den = the same with absolute values (the scale the
 * componentwise error criterion divides by).  y may be NULL when beta == 0.
 * Restates what the reference asks of cublasSgemv in its offline ABFT baseline
 * (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:8-23), in row-major terms. */
void oracle_sgemv_f64(int trans, int M, int N, float alpha, const float* A, int lda, const float* x,
                      float beta, const float* y, double* out, double* den) {
    int ylen = trans ? N : M;
    for (int i = 0; i < ylen; ++i) {
        double s = 0.0, a = 0.0;
        if (!trans)
            for (int n = 0; n < N; ++n) {
                double p = (double)A[(size_t)i * lda + n] * (double)x[n];
                s += p; a += fabs(p);
            }
        else
            for (int m = 0; m < M; ++m) {
                double p = (double)A[(size_t)m * lda + i] * (double)x[m];
                s += p; a += fabs(p);
            }
        double yv = (beta != 0.0f && y) ? (double)y[i] : 0.0;
        out[i] = (double)alpha * s + (double)beta * yv;
        den[i] = fabs((double)alpha) * a + fabs((double)beta) * fabs(yv);
    }
}

/* Offline (panel-wise) ABFT in FP64: C is formed one K panel at a time; after
 * panel p, res[2p] = sum_n (colsum(C)[n] - ref_col[n]) and res[2p+1] =
 * sum_m (rowsum(C)[m] - ref_row[m]), where the references are carried through
 * the operands: ref_col += alpha * (e^T A_p) B_p, ref_row += alpha * A_p (B_p e),
 * starting from beta * colsum / rowsum of the initial C.  One fault: delta is
 * added to C[row][col] right after panel fault_panel's product (fault_panel
 * < 0: none).  C (float, M x N, ldc) receives the final result rounded to
 * FP32.  Restates the call sequence of baseline_ft_sgemm
 * (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:3-31: gemm, two gemv over C,
 * two gemv over the panels, two gemv carrying them through, two axpy, two
 * dot), with references that accumulate over the panels. */
void oracle_offline_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                             float* C, int ldc, float alpha, float beta, int panel, int fault_panel,
                             int fault_row, int fault_col, float fault_delta, double* res) {
    double* acc = (double*)calloc((size_t)M * N, sizeof(double));
    double* ref_row = (double*)calloc((size_t)M, sizeof(double));
    double* ref_col = (double*)calloc((size_t)N, sizeof(double));
    double* a_col = (double*)malloc(sizeof(double) * (size_t)panel);
    double* b_row = (double*)malloc(sizeof(double) * (size_t)panel);
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double c0 = (beta != 0.0f) ? (double)beta * (double)C[(size_t)m * ldc + n] : 0.0;
            acc[(size_t)m * N + n] = c0;
            ref_row[m] += c0;
            ref_col[n] += c0;
        }
    int panels = (K + panel - 1) / panel;
    for (int p = 0; p < panels; ++p) {
        int k0 = p * panel, kp = (K - k0 < panel) ? K - k0 : panel;
        #pragma omp parallel for schedule(static)
        for (int m = 0; m < M; ++m)
            for (int k = 0; k < kp; ++k) {
                double a = (double)alpha * (double)A[(size_t)m * lda + k0 + k];
                const float* brow = B + (size_t)(k0 + k) * ldb;
                double* crow = acc + (size_t)m * N;
                for (int n = 0; n < N; ++n) crow[n] += a * (double)brow[n];
            }
        if (p == fault_panel) acc[(size_t)fault_row * N + fault_col] += (double)fault_delta;
        for (int k = 0; k < kp; ++k) {
            double s = 0.0, t = 0.0;
            for (int m = 0; m < M; ++m) s += (double)A[(size_t)m * lda + k0 + k];
            for (int n = 0; n < N; ++n) t += (double)B[(size_t)(k0 + k) * ldb + n];
            a_col[k] = s;
            b_row[k] = t;
        }
        for (int n = 0; n < N; ++n) {
            double s = 0.0;
            for (int k = 0; k < kp; ++k) s += a_col[k] * (double)B[(size_t)(k0 + k) * ldb + n];
            ref_col[n] += (double)alpha * s;
        }
        for (int m = 0; m < M; ++m) {
            double s = 0.0;
            for (int k = 0; k < kp; ++k) s += (double)A[(size_t)m * lda + k0 + k] * b_row[k];
            ref_row[m] += (double)alpha * s;
        }
        double rc = 0.0, rr = 0.0;
        for (int n = 0; n < N; ++n) {
            double s = 0.0;
            for (int m = 0; m < M; ++m) s += acc[(size_t)m * N + n];
            rc += s - ref_col[n];
        }
        for (int m = 0; m < M; ++m) {
            double s = 0.0;
            for (int n = 0; n < N; ++n) s += acc[(size_t)m * N + n];
            rr += s - ref_row[m];
        }
        res[2 * p] = rc;
        res[2 * p + 1] = rr;
    }
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) C[(size_t)m * ldc + n] = (float)acc[(size_t)m * N + n];
    free(acc); free(ref_row); free(ref_col); free(a_col); free(b_row);
}

/* Offline ABFT with one scalar checksum per panel: the reference's second offline routine forms, after every panel
 * product, the total of C (row sums of C dotted with ones), the total of the A panel's column sums and the total of
 * the B panel's row sums, twice over, and leaves them unused (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:36-91).
 * The identity that turns those sums into a check is e^T (A_p B_p) e = sum_k (e^T A_p)_k (B_p e)_k:
 *   res[p] = (sum of all of C after panel p) - (beta * sum of C before + alpha * sum over the panels so far of
 *            sum_k a_col[k] * b_row[k]).
 * FP64 throughout; C receives the rounded product (with the uncorrected fault). */
void oracle_offline_ft_sgemm_scalar(int M, int N, int K, const float* A, int lda, const float* B, int ldb,
                                    float* C, int ldc, float alpha, float beta, int panel, int fault_panel,
                                    int fault_row, int fault_col, float fault_delta, double* res) {
    double* acc = (double*)calloc((size_t)M * N, sizeof(double));
    double ref = 0.0;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double c0 = (beta != 0.0f) ? (double)beta * (double)C[(size_t)m * ldc + n] : 0.0;
            acc[(size_t)m * N + n] = c0;
            ref += c0;
        }
    int panels = (K + panel - 1) / panel;
    for (int p = 0; p < panels; ++p) {
        int k0 = p * panel, kp = (K - k0 < panel) ? K - k0 : panel;
        #pragma omp parallel for schedule(static)
        for (int m = 0; m < M; ++m)
            for (int k = 0; k < kp; ++k) {
                double a = (double)alpha * (double)A[(size_t)m * lda + k0 + k];
                const float* brow = B + (size_t)(k0 + k) * ldb;
                double* crow = acc + (size_t)m * N;
                for (int n = 0; n < N; ++n) crow[n] += a * (double)brow[n];
            }
        if (p == fault_panel) acc[(size_t)fault_row * N + fault_col] += (double)fault_delta;
        double carried = 0.0;
        for (int k = 0; k < kp; ++k) {
            double s = 0.0, t = 0.0;
            for (int m = 0; m < M; ++m) s += (double)A[(size_t)m * lda + k0 + k];
            for (int n = 0; n < N; ++n) t += (double)B[(size_t)(k0 + k) * ldb + n];
            carried += s * t;
        }
        ref += (double)alpha * carried;
        double total = 0.0;
        for (size_t i = 0; i < (size_t)M * N; ++i) total += acc[i];
        res[p] = total - ref;
    }
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) C[(size_t)m * ldc + n] = (float)acc[(size_t)m * N + n];
    free(acc);
}

