/*
 * hpcdnn -- FP32 BLAS level-1/3 + ABFT-SGEMM for AMD MI355X (gfx950).
 *
 * C ABI of libhpcdnn.so.  Plain pointers and sizes only; every device pointer
 * is memory the caller allocated on the current HIP device, every `stream` is
 * a hipStream_t passed as void* (NULL = the null stream).  Calls enqueue work
 * on `stream` and return without synchronising.  Nothing here allocates device
 * memory: kernels that need scratch take a caller-provided workspace.
 *
 * The reference (shixun404/HPCDeepNeuralNetworks) exposes no library API: its
 * boundary is "a __global__ function plus the launch geometry its driver
 * hard-codes".  Each entry point below names the reference kernel(s) and the
 * launch site it stands in for; argument order follows the reference
 * (dims, A, B, C, alpha, beta) / (n, alpha, x, y) / (n, x, y, out), with
 * leading dimensions, workspace and stream added.  All matrices are row-major:
 * element (i,j) of A is A[i*lda + j].
 *
 * Return value: 0 on success, otherwise a hipError_t-compatible code
 * (HPCDNN_ERR_INVALID_VALUE = hipErrorInvalidValue for bad arguments, or the
 * launch error reported by the HIP runtime).  The library never exits or
 * prints (the reference's CUDA_CALLER prints and exit(1)s, utils/utils.cuh:7-15).
 */
#ifndef HPCDNN_H
#define HPCDNN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HPCDNN_OK 0
#define HPCDNN_ERR_INVALID_VALUE 1      /* == hipErrorInvalidValue */
#define HPCDNN_ERR_WORKSPACE 2          /* workspace missing or too small (== hipErrorOutOfMemory) */
#define HPCDNN_ERR_NOT_READY 3          /* one-time set-up refused under stream capture (== hipErrorNotInitialized) */

/* Output tile of the ABFT kernel: one checksum pair (256 row sums, 128 column
 * sums) and one status record per tile, tiles numbered row-major:
 * tile = (i / 256) * ceil(N / 128) + (j / 128). */
#define HPCDNN_FT_TILE_M 256
#define HPCDNN_FT_TILE_N 128
/* ABFT tile classes: 0 = 256x128 (above), 1 = 128x128, 2 = 64x128, and for
 * products with few columns 3 = 128x64, 4 = 64x64. */
#define HPCDNN_FT_NUM_CLASSES 5

/* Operation selectors for hpcdnn_workspace_bytes(). */
#define HPCDNN_OP_SGEMM 0
#define HPCDNN_OP_SDOT 1
#define HPCDNN_OP_FT_SGEMM 2
#define HPCDNN_OP_SGEMV 3            /* M, N as passed to hpcdnn_sgemv; only trans = 1 uses a workspace */
#define HPCDNN_OP_OFFLINE_FT_SGEMM 4
#define HPCDNN_OP_FT_SGEMM_CM_NT 5     /* M, N, K as passed to hpcdnn_ft_sgemm_cm_nt */

/* K panel of hpcdnn_offline_ft_sgemm (the reference checks every 256 columns,
 * kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:3). */
#define HPCDNN_OFFLINE_FT_PANEL_K 256

/* One soft error to inject: `delta` is added to the accumulator of element
 * (row, col) of output tile `tile` after the K loop and before verification.
 * Run-time replacement for the reference's compile-time injection
 * (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:40,145: +1.0 into one
 * accumulator of thread 0 of every block). */
typedef struct hpcdnn_fault {
    int32_t tile;
    int32_t row;   /* tile-local, 0 .. HPCDNN_FT_TILE_M-1 */
    int32_t col;   /* tile-local, 0 .. HPCDNN_FT_TILE_N-1 */
    float delta;
} hpcdnn_fault;

/* Verification record of one output tile (32 bytes, device memory).
 * The column checksums screen: a tile none of whose columns exceeds its
 * threshold is clean, and its row checksums are not looked at (the reference
 * acts on a tile only when a column AND a row checksum disagree,
 * kernel/ft_sgemm/include/ft_sgemm_huge.cuh:289).  With a flagged column the
 * rows are thresholded too: one row x one column locates the element.
 * The other way round on a product one tile wide (N <= the tile's columns,
 * 32 tiles or more) that is given a workspace and verified once per tile:
 * its B is small and its A is read exactly once, so the row checksums, which
 * need sums over B only, screen, and the columns are looked at (and counted)
 * only when a row is flagged.  Either way the side that is not the screen
 * costs nothing until it is needed: its references are formed in the
 * verification, from A and B. */
typedef struct hpcdnn_ft_status {
    int32_t flag;             /* 0 clean; 1 single fault located and corrected; 2 detected, not correctable */
    int32_t row, col;         /* tile-local location of the corrected element, -1 if none */
    int32_t n_bad_rows;       /* lines whose |reference - observed| checksum residual exceeded the threshold */
    int32_t n_bad_cols;       /* (the side that is not the screen is counted only when the screen flagged a line) */
    float row_residual;       /* signed residual of the located row (the size of the fault, negated), else 0 */
    float col_residual;       /* signed residual of the located column, else 0 */
    float max_clean_residual; /* largest |residual| among the lines looked at and judged clean */
} hpcdnn_ft_status;

const char* hpcdnn_version(void);
const char* hpcdnn_error_string(int code);

/* C = alpha*A*B + beta*C, A is MxK, B is KxN, C is MxN, any M,N,K >= 0 and any
 * lda >= K, ldb >= N, ldc >= N with lda, ldc <= 2^21 - 64 and ldb <= 2^25 - 1024 (byte
 * offsets inside one tile are 32-bit; larger values return
 * HPCDNN_ERR_INVALID_VALUE).  A, B and C are 4-byte aligned.  C is not read
 * when beta == 0.
 * Replaces sgemm_1..sgemm_14 <<<dim3(ceil(N/bt),ceil(N/bt)),256>>>(N,A,B,C,alpha,beta)
 * (kernel/sgemm/sgemm.cu:70-141, kernel/sgemm/include/kernel_13.cuh:14) and
 * sgemm_{small,medium,large,tall,wide,huge} <<<dim3(ceil(M/ms),ceil(N/ns)),T>>>
 * (M,N,K,A,B,C,alpha,beta) (kernel/ft_sgemm/sgemm.cu:114-157).
 * `ws`/`ws_bytes`: optional split-K scratch (hpcdnn_workspace_bytes); when
 * absent or too small the K dimension is not split (slower for deep-K
 * shapes, same result contract). */
int hpcdnn_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                 float alpha, float beta, void* ws, size_t ws_bytes, void* stream);

/* Same contract with the kernel choice pinned, for tests and sweeps:
 * `tile` indexes the built-in tile table (hpcdnn_sgemm_tile_info), -1 = pick
 * as hpcdnn_sgemm does; `split_k` >= 1 forces that many K slices (needs a
 * workspace of M*N*split_k floats when > 1), 0 = pick; `split_k` = -s (s >= 2)
 * splits only the tiles left over after the last full round of CUs, s ways
 * (workspace: leftover tiles * s * tile size floats, 16-byte aligned; not
 * available for the 32 x 32 tile).  Either way the slices are added in a fixed
 * order.  All tiles but the 32 x 32 one add the products of an element in the
 * same order and give the same bits; in the 32 x 32 tile the four waves of a
 * workgroup split K between them. */
int hpcdnn_sgemm_ex(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                    float alpha, float beta, void* ws, size_t ws_bytes, int tile, int split_k, void* stream);

/* The same product with the left operand given transposed: C (M x N, row-major)
 * = alpha * At^T * B + beta * C, where At is K x M row-major with row length
 * ldat >= M (ldat <= 2^25 - 1024); everything else as hpcdnn_sgemm.  Every
 * element of C sums its products in the order hpcdnn_sgemm uses, so the result
 * has the bits of hpcdnn_sgemm on the explicitly transposed operand.  This is the
 * operand layout of the reference's column-major family (below).  The _ex form
 * pins tile and split as hpcdnn_sgemm_ex does. */
int hpcdnn_sgemm_tn(int M, int N, int K, const float* At, int ldat, const float* B, int ldb, float* C, int ldc,
                    float alpha, float beta, void* ws, size_t ws_bytes, void* stream);
int hpcdnn_sgemm_tn_ex(int M, int N, int K, const float* At, int ldat, const float* B, int ldb, float* C, int ldc,
                       float alpha, float beta, void* ws, size_t ws_bytes, int tile, int split_k, void* stream);

/* COLUMN-MAJOR C (M x N, ldc >= M) = alpha * A (M x K, lda >= M) * B (N x K,
 * ldb >= N)^T + beta * C: the buffers, argument order and meaning of
 * sgemm_{small,medium,large,tall,wide,huge}<<<...>>>(M,N,K,A,B,C,alpha,beta)
 * (kernel/ft_sgemm/include/sgemm_huge.cuh:14, launched at
 * kernel/ft_sgemm/sgemm.cu:114-157) and of the cuBLAS call they are checked
 * against, cublasSgemm(handle, CUBLAS_OP_N, CUBLAS_OP_T, M, N, K, &alpha, dA, M,
 * dB, N, &beta, dC, M) (kernel/ft_sgemm/sgemm.cu:111), taken as they are.  Read
 * row by row the same memory is C^T (N x M) = B^T^T * A^T, which is what runs:
 * hpcdnn_sgemm_tn(N, M, K, B, ldb, A, lda, C, ldc, ...).  Workspace as for
 * hpcdnn_sgemm with M and N exchanged; lda, ldb <= 2^25 - 1024, ldc <= 2^21 - 64. */
int hpcdnn_sgemm_cm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                       float alpha, float beta, void* ws, size_t ws_bytes, void* stream);

/* Number of tile configurations, and the shape of entry `tile` (returns 0, or
 * HPCDNN_ERR_INVALID_VALUE when out of range).  Counterpart of the reference's
 * shape table (kernel/ft_sgemm/code_gen/main.py:8-16). */
int hpcdnn_sgemm_num_tiles(void);
int hpcdnn_sgemm_tile_info(int tile, int* bm, int* bn, int* bk);
/* The (tile, split_k) hpcdnn_sgemm picks for a shape when given a workspace of
 * ws_bytes (0 = none), split_k with the meaning it has for hpcdnn_sgemm_ex: a
 * function of the shape and the device's CU count only. */
int hpcdnn_sgemm_plan(int M, int N, int K, size_t ws_bytes, int* tile, int* split_k);
/* hpcdnn_sgemm may instead cover C with two launches: the first *rows_first rows
 * (whole rounds of tile *tile_first over the CUs) and the remaining rows (tile
 * *tile_rest), when that beats the single plan above by more than 3 %; no
 * workspace is involved and every element of C still sums K in one piece.
 * *rows_first = 0 when it does not. */
int hpcdnn_sgemm_row_split(int M, int N, int K, size_t ws_bytes, int* rows_first, int* tile_first, int* tile_rest);

/* SGEMM with fused online ABFT: row/column checksums of each 256x128 output
 * tile are accumulated from A and B inside the main loop, compared with the
 * line sums of the accumulators in the epilogue, and a single faulty element
 * per tile is located (faulty row x faulty column) and corrected before
 * alpha/beta are applied.  `tau` > 0 is an absolute residual threshold
 * (hpcdnn_ft_default_tau(K) is one calibrated for operands uniform in [-1, 1];
 * on larger or non-zero-mean data a constant flags fault-free products), and
 * `tau` <= 0 scales the threshold to the data: a line of n elements is
 * flagged when its residual exceeds f * 2.56e-7 * sqrt(max(K, 64)) *
 * sqrt(n) * m, m being the larger of the mean |accumulator| of the line and
 * of the whole tile and f = -tau, or 1 for `tau` == 0, the default (f = 1 is
 * calibrated to twice the largest fault-free residual of uniform operands and
 * follows the data when it is scaled or shifted; a check tile that is a single
 * element - the corner of a product ragged in both dimensions - has nothing to
 * take a scale from but that element, and rounding noise flags about 2 % of
 * such tiles when the element is small against its terms: the recomputation
 * then leaves its value unchanged); `inject` is a HOST
 * pointer to one fault or NULL; `status` is DEVICE memory for
 * hpcdnn_ft_num_tiles(M,N) records or NULL.
 * `ws`/`ws_bytes`: optional DEVICE scratch of
 * hpcdnn_workspace_bytes(HPCDNN_OP_FT_SGEMM,M,N,K) bytes, 16-byte aligned, no
 * initialisation needed.  With it the checksum vector of A that the main loop
 * needs (its column sums per tile row) is formed once by a small kernel ahead
 * of the GEMM (faster); with ws == NULL each workgroup forms it in its main
 * loop, as the reference does.  What only a tile with a flagged line needs -
 * the row sums of B and the row references - is formed in that tile's
 * verification, from A and B, either way.  Detection, location and correction
 * are the same in both.
 * The size the query returns also has room for the K slices of a partial last
 * round of tiles: those tiles are then split along K, every slice verifying
 * and correcting its own partial product (the checksums are linear in K), and
 * a second pass adds the slices in order and merges their records into the
 * tile's (bad-line counts add up; the location is that of the first slice that
 * corrected something).  A workspace that only holds the checksum vectors
 * (the size without that room) runs without the split.
 * A corrected element: the located accumulator is computed again from its
 * row of A and column of B, one fused multiply-add per k in the order the
 * matrix cores add them, and replaces the faulty value; a corrected product
 * therefore has exactly the bits of a fault-free one, whatever the size of the
 * fault (the reference subtracts a rounded residual at this point,
 * kernel/ft_sgemm/include/ft_sgemm_huge.cuh:352-371).  The signed residuals of
 * the located row and column are reported in the record (minus the fault, to
 * within the rounding of the line sums).  The recomputation costs a launch
 * that corrects about 3 us per 1024 values of k and a fault-free launch
 * nothing.
 * Replaces ft_sgemm_huge <<<dim3(M/128,N/128),256>>>(M,N,K,A,B,C,alpha,beta)
 * (kernel/ft_sgemm/sgemm.cu:159-165, kernel/ft_sgemm/include/ft_sgemm_huge.cuh:21). */
int hpcdnn_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                    float alpha, float beta, float tau, const hpcdnn_fault* inject, hpcdnn_ft_status* status,
                    void* ws, size_t ws_bytes, void* stream);
int hpcdnn_ft_num_tiles(int M, int N);

/* The same on another tile class (hpcdnn_ft_sgemm is class 0): checksums,
 * verification, status records and `inject` coordinates are per tile of that
 * class, so `status` holds hpcdnn_ft_num_tiles_ex(tile_class, M, N) records.
 * Smaller tiles keep more CUs busy on smaller problems; hpcdnn_ft_pick_class
 * returns the class with the shortest predicted run for a call that passes the
 * workspace (rounds of tiles over the CUs times the tile height, a partial
 * last round counting for what its K split leaves of it).  The workspace
 * size of HPCDNN_OP_FT_SGEMM covers every class.  Counterpart of the reference's
 * abft_kernel_{huge,large,wide,tall,medium} series (kernel/ft_sgemm/sgemm.cu:187-188,
 * kernel/ft_sgemm/code_gen/main.py:8-16; its tall 128x32 and medium 32x32 shapes
 * become 128x64 and 64x64 here: four waves of 32x32 matrix-core blocks). */
int hpcdnn_ft_sgemm_ex(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                       float alpha, float beta, float tau, const hpcdnn_fault* inject, hpcdnn_ft_status* status,
                       void* ws, size_t ws_bytes, int tile_class, void* stream);
int hpcdnn_ft_tile_info(int tile_class, int* bm, int* bn);

/* Checksum granularity and verification cadence (the reference's block- /
 * warp- / thread-level kernels and its in-loop verification:
 * kernel/ft_sgemm/include/ft_sgemm_huge.cuh:143,263-271 verifies every 256 k
 * and re-synchronises; ft_sgemm_huge_warp.cuh:111-207 keeps one checksum pair
 * per warp tile, ft_sgemm_huge_thread.cuh:106-177 one per thread tile).
 *
 * granularity HPCDNN_FT_GRAN_TILE: one checksum pair, one verification and one
 * status record per workgroup tile of the class (what hpcdnn_ft_sgemm_ex does).
 * HPCDNN_FT_GRAN_WAVE: one per wave tile, the part of the workgroup tile one
 * 64-lane wave accumulates on the matrix cores (class 0: 128x32, class 1:
 * 64x64, class 2: 32x64, class 3: 64x32, class 4: 32x32;
 * hpcdnn_ft_check_tile_info): every wave tile is
 * verified, located and corrected on its own, so one fault per wave tile is
 * correctable where tile granularity reports two faults in one 256x128 tile
 * as uncorrectable.  Needs the workspace (HPCDNN_ERR_WORKSPACE without one).
 * Class 1 is the cheapest carrier of this granularity (4096^3: +13 % over plain
 * SGEMM, class 0: +19 %).
 * The wave tile is the finest granularity on this hardware: a matrix-core
 * instruction spreads its 32x32 result over all 64 lanes, so there is no
 * per-thread tile to keep checksums for.
 *
 * check_interval 0: one verification, after the K loop.  > 0 (a multiple of
 * 16; the reference uses 256): also every check_interval values of k inside
 * the K loop, against reference checksums of the k range done so far; after
 * each verification the references are re-synchronised with the (corrected)
 * accumulators, so every verification sees what happened since the one
 * before, and one fault per check tile *per interval* is correctable.  The
 * record of a check tile merges its verifications: bad-line counts add up,
 * flag 2 if any verification could not locate its fault, else 1 if any
 * corrected an element; row, col and the residuals are those of the first
 * correction.  Every class, either granularity, with or without workspace
 * (the reference's kernels all carry the in-loop check,
 * kernel/ft_sgemm/include/ft_sgemm_large.cuh:337, ft_sgemm_tall.cuh:18).
 * Tiles of a partial last round that are split along K (see hpcdnn_ft_sgemm)
 * are cut at multiples of check_interval, every slice verifying its own
 * intervals, so the verifications of a tile are the same with and without
 * the split.
 *
 * locator HPCDNN_FT_LOCATE_ROW_COL: a faulty row and a faulty column of a
 * check tile meet in the faulty element (what everything above describes).
 * HPCDNN_FT_LOCATE_WEIGHTED: the reference's second scheme ("kernel 2",
 * kernel/ft_sgemm/README.md:16-26; its weighted locator is left in comments
 * at kernel/ft_sgemm/include/ft_sgemm_huge.cuh:299-310): two row sums of B,
 * with weights e1 = [1, 1, ...] and e2 = [1, 2, ...] over the tile's columns,
 * and nothing from A.  The references A (B e1), A (B e2) are compared with the
 * plain and the weighted row sums of the accumulators: a row whose plain
 * residual d1 exceeds the threshold is faulty, and with one fault delta in
 * column n of it the residuals are d1 = -delta, d2 = -(n + 1) delta, so the
 * column is round(d2 / d1) - 1.  One faulty row: that element is computed
 * again; if that changed it by d1 (to within the row's threshold + 2^-20 |d1|) the fault is
 * located and corrected (flag 1, n_bad_cols = 1), else - two faults in the
 * row, or a fault too small against the rounding noise of the weighted sums,
 * which is about 0.6 x the tile's width x that of the plain sums - the tile
 * is reported as detected, not corrected (flag 2, n_bad_cols = 0; computing a
 * healthy element again changes nothing, so a wrong guess does no harm).  More
 * faulty rows: flag 2.  The record's col_residual is d2 of the located row.
 * The pre-pass reads B only, which is what a tall product with few columns
 * wants.  Needs the workspace; tile granularity, one verification (the other
 * combinations return HPCDNN_ERR_INVALID_VALUE).
 *
 * Check tiles are numbered row-major over the matrix,
 * t = (i / cm) * ceil(N / cn) + (j / cn); `status` holds
 * hpcdnn_ft_num_check_tiles() records, and the tile / row / col of a fault
 * are in check-tile units.  `check` of a fault is the verification (0 = first)
 * before which it is added; a run that verifies once adds every fault before
 * that verification.  Faults aimed outside the matrix are ignored. */
#define HPCDNN_FT_GRAN_TILE 0
#define HPCDNN_FT_GRAN_WAVE 1
#define HPCDNN_FT_LOCATE_ROW_COL 0
#define HPCDNN_FT_LOCATE_WEIGHTED 1
#define HPCDNN_FT_MAX_FAULTS 4
typedef struct hpcdnn_ft_fault_at {
    int32_t tile;
    int32_t row, col;
    float delta;
    int32_t check;
} hpcdnn_ft_fault_at;
typedef struct hpcdnn_ft_options {
    int32_t tile_class;      /* as for hpcdnn_ft_sgemm_ex */
    int32_t granularity;     /* HPCDNN_FT_GRAN_* */
    int32_t check_interval;  /* 0, or a positive multiple of 16 */
    int32_t n_faults;        /* 0 .. HPCDNN_FT_MAX_FAULTS */
    hpcdnn_ft_fault_at faults[HPCDNN_FT_MAX_FAULTS];
    int32_t locator;         /* HPCDNN_FT_LOCATE_* */
} hpcdnn_ft_options;
/* hpcdnn_ft_sgemm_ex with the options above (`opt` is a HOST pointer, NULL =
 * class 0, tile granularity, one verification, no faults). */
int hpcdnn_ft_sgemm_opt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                        float alpha, float beta, float tau, const hpcdnn_ft_options* opt, hpcdnn_ft_status* status,
                        void* ws, size_t ws_bytes, void* stream);
/* hpcdnn_ft_sgemm_opt on the reference family's own COLUMN-MAJOR buffers:
 * C (M x N, ldc >= M) = alpha * A (M x K, lda >= M) * B (N x K, ldb >= N)^T +
 * beta * C, the buffers, argument order and meaning of
 * ft_sgemm_huge<<<...>>>(M,N,K,A,B,C,alpha,beta)
 * (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:21, launched at
 * kernel/ft_sgemm/sgemm.cu:159-165).  It runs as the row-major problem
 * C^T (N x M) = (B^T)^T * A^T: tiles, check tiles, status records and fault
 * coordinates are those of hpcdnn_ft_sgemm_opt(N, M, K, ...), i.e. `row` counts
 * along N (the columns of the column-major C) and `col` along M; use
 * hpcdnn_ft_num_check_tiles(tile_class, granularity, N, M) records.  Both
 * operands are read where they lie (no transposed copy).  `ws`: optional
 * scratch of hpcdnn_workspace_bytes(HPCDNN_OP_FT_SGEMM_CM_NT, M, N, K) bytes (=
 * that of HPCDNN_OP_FT_SGEMM for N, M, K), with the meaning and rules it has
 * for hpcdnn_ft_sgemm_opt.  `opt` may be NULL. */
int hpcdnn_ft_sgemm_cm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                          float alpha, float beta, float tau, const hpcdnn_ft_options* opt, hpcdnn_ft_status* status,
                          void* ws, size_t ws_bytes, void* stream);
int hpcdnn_ft_check_tile_info(int tile_class, int granularity, int* cm, int* cn);
int hpcdnn_ft_num_check_tiles(int tile_class, int granularity, int M, int N);
int hpcdnn_ft_num_tiles_ex(int tile_class, int M, int N);
int hpcdnn_ft_pick_class(int M, int N, int K);
/* The same for a call that passes a workspace of `ws_bytes` (0: none, the
 * checksum vectors are then formed in the main loop and no tile can be split
 * along K, which favours other classes: at 3072^3 without a workspace the
 * 64x128 class runs 10 % ahead of the 128x128 one that the workspace variant
 * takes).  The status records are those of the class returned.  No counterpart
 * in the reference, which picks its kernel by name. */
int hpcdnn_ft_pick_class_ws(int M, int N, int K, size_t ws_bytes);
/* An absolute threshold for operands uniform in [-1, 1], to be passed as
 * `tau`: 1.1e-6 * max(K, 64), twice the largest fault-free residual measured
 * for such operands (the rounding noise of the FP32 accumulators grows
 * linearly with K).  It is not what tau == 0 selects: that is the data-scaled
 * threshold, which needs no knowledge of the operands. */
float hpcdnn_ft_default_tau(int K);

/* hpcdnn_ft_sgemm for callers that cannot allocate device memory or carry a
 * workspace around (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): same arguments and results as
 * hpcdnn_ft_sgemm called with a workspace, but the scratch (checksum vectors of
 * A and B, K slices of a partial last round when they fit as well) is a fixed
 * array of HPCDNN_FT_STATIC_SCRATCH_BYTES inside the library, one copy per
 * device.  The call allocates and frees nothing.  Problems whose checksum
 * vectors need more than the array,
 *   (ceil(M/256) + ceil(N/128)) * (ceil(K/16) + 2) * 64 bytes > HPCDNN_FT_STATIC_SCRATCH_BYTES,
 * are refused with HPCDNN_ERR_WORKSPACE (e.g. 8192^3 needs 3.0 MiB and fits,
 * 12288^3 does not).  All calls on one device share the array: calls that may
 * overlap in time on one device (different streams, different host threads)
 * race on it and must be serialised by the caller; the array needs no
 * initialisation and keeps nothing between calls.
 * The first call on a device looks the array's address up and raises the LDS
 * limit of its kernels, which does not belong into a stream capture: it
 * returns HPCDNN_ERR_NOT_READY when its stream is capturing.  Make one eager
 * call on the device beforehand (M = 0 is enough and launches nothing); every
 * later call only enqueues kernels and can be captured.
 * No counterpart in the reference, whose driver allocates everything up front
 * (kernel/ft_sgemm/sgemm.cu:60-83). */
#define HPCDNN_FT_STATIC_SCRATCH_BYTES (4u << 20)
int hpcdnn_ft_sgemm_static(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                           float alpha, float beta, float tau, const hpcdnn_fault* inject, hpcdnn_ft_status* status,
                           void* stream);

/* Row-major SGEMV, A is M x N with leading dimension lda >= N:
 *   trans = 0:  y[M] = alpha * A   * x[N] + beta * y
 *   trans = 1:  y[N] = alpha * A^T * x[M] + beta * y
 * beta == 0 never reads y.  `ws`/`ws_bytes`: optional scratch of
 * hpcdnn_workspace_bytes(HPCDNN_OP_SGEMV, M, N, 0) bytes for trans = 1 (rows
 * are then split over more workgroups; the partial sums are added in a fixed
 * order, so results do not depend on timing either way).
 * Stands in for the cublasSgemv calls of the reference's offline ABFT baseline
 * (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:8-23), which are column-major:
 * its CUBLAS_OP_N on an M x N column-major matrix is trans = 1 on the same
 * memory read as an N x M row-major one. */
int hpcdnn_sgemv(int trans, int M, int N, float alpha, const float* A, int lda, const float* x, float beta, float* y,
                 void* ws, size_t ws_bytes, void* stream);

/* Offline (panel-wise) ABFT SGEMM: C = alpha*A*B + beta*C is formed one K panel
 * of HPCDNN_OFFLINE_FT_PANEL_K at a time (hpcdnn_sgemm), and after every panel
 * the row and column sums of C (one pass over C) are compared with checksums
 * carried through the operands, (e^T A_p) B_p and A_p (B_p e), accumulated over
 * the panels (the GEMM and two more launches per panel where the reference
 * issues a GEMM, six SGEMV, two SAXPY and two SDOT calls).
 * `residuals`: DEVICE array of 2*ceil(K/panel) floats; [2p] = sum over the
 * columns of (column sums of C - reference), [2p+1] = the same over the rows,
 * after panel p.  Fault-free both are rounding noise; a soft error of size d
 * in C shows up as d in both from its panel on.  Detection only: like the
 * reference baseline it neither locates nor corrects.
 * `inject`: HOST pointer or NULL; `tile` = panel after whose product `delta`
 * is added to C[row][col] (row, col global).
 * `ws`: DEVICE scratch of hpcdnn_workspace_bytes(HPCDNN_OP_OFFLINE_FT_SGEMM,
 * M,N,K) bytes, 16-byte aligned, no initialisation needed.
 * Replaces baseline_ft_sgemm(num_tests, M, N, K, handle, dA, dB, dC, dE, dRes,
 * dcheck_*..., alpha, beta, negative_1)
 * (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:1-34; call site
 * kernel/ft_sgemm/sgemm.cu:306), whose scratch vectors are the workspace here. */
int hpcdnn_offline_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                            float alpha, float beta, const hpcdnn_fault* inject, float* residuals, void* ws,
                            size_t ws_bytes, void* stream);

/* The same with one scalar checksum per panel: after every panel the total of C
 * is compared with a reference carried through the operands,
 *   e^T (A_p B_p) e = sum_k (e^T A_p)_k (B_p e)_k,
 * accumulated over the panels (no second pass over the panels, a single
 * residual per panel).  `residuals`: DEVICE array of ceil(K/panel) floats,
 * [p] = total of C - reference after panel p; it equals residuals[2p] of
 * hpcdnn_offline_ft_sgemm up to rounding.  Same workspace, `inject` and
 * contract otherwise.
 * Restates offline_ft_sgemm(num_tests, M, N, K, handle, dA, dB, dC, dE, dRes,
 * dcheck_*..., alpha, beta, negative_1)
 * (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:36-91), which forms the total
 * of C, of the A panel's column sums and of the B panel's row sums after each
 * panel product (twice over, each into the same scalar) and uses none of them:
 * the identity above is what makes those sums a check. */
int hpcdnn_offline_ft_sgemm_scalar(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                                   int ldc, float alpha, float beta, const hpcdnn_fault* inject, float* residuals,
                                   void* ws, size_t ws_bytes, void* stream);

/* y = alpha*x + y, one fused multiply-add per element, any n >= 0, any 4-byte
 * aligned x and y.  Replaces saxpy/saxpy3/_saxpy <<<ceil(n/4/tpb),tpb>>>
 * (N,alpha,x,y) (kernel/saxpy/saxpy.cu:15-48, launch :110-114). */
int hpcdnn_saxpy(int64_t n, float alpha, const float* x, float* y, void* stream);

/* *out = sum_i x[i]*y[i] (device scalar, overwritten; deterministic: the same
 * inputs give the same bits on every run).  `ws` must hold
 * hpcdnn_workspace_bytes(HPCDNN_OP_SDOT,...) bytes and have been passed through
 * hpcdnn_workspace_init once (it holds the number of calls completed, by
 * which a call tells the partial sums of its own blocks from older ones);
 * calls sharing a workspace must be stream-ordered, and nothing else may
 * write to it.
 * Replaces _sdot <<<min(1024,ceil(n/tpb)),tpb>>>(N,x,y,out) with its
 * pre-zeroed atomicAdd target, and the sdot + reduction multi-launch chain
 * (kernel/sdot/sdot.cu:9-67, launches :156,:177-187). */
int hpcdnn_sdot(int64_t n, const float* x, const float* y, float* out, void* ws, size_t ws_bytes, void* stream);

/* Scratch size for an operation (SGEMM: split-K partials for the split
 * hpcdnn_sgemm would choose, 0 if none; SDOT: the blocks' tagged partials + the call counter; M,N,K
 * ignored for SDOT). */
size_t hpcdnn_workspace_bytes(int op, int M, int N, int K);
/* Zero a freshly allocated workspace (fill kernel, safe to capture). */
int hpcdnn_workspace_init(void* ws, size_t ws_bytes, void* stream);

/* Seeded i.i.d. uniform values on the grid {-1 + j*2^-23}: element i of a
 * vector takes counter i; element (r,c) of a rows x cols matrix takes counter
 * r*cols + c whatever `ld` is (padding is left untouched).  Device-side
 * replacement for generate_random_vector/matrix (utils/utils.cu:28-44). */
int hpcdnn_fill_uniform(float* dst, int64_t n, uint64_t seed, void* stream);
int hpcdnn_fill_uniform_matrix(float* dst, int rows, int cols, int ld, uint64_t seed, void* stream);

/* Host validator kept from the reference: naive row-major square
 * C = alpha*A*B + beta*C on HOST pointers, float accumulator, one thread
 * (utils/utils.cu:93-103; same argument order). */
void hpcdnn_cpu_gemm(float alpha, float beta, const float* mat1, const float* mat2, int n, float* mat3);

#ifdef __cplusplus
}
#endif
#endif /* HPCDNN_H */
