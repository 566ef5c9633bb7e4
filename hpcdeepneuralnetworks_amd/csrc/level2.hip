// SGEMV (row-major, both orientations; the counterpart of the cublasSgemv calls of the reference's offline ABFT
// baseline) and the offline ABFT baseline itself (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:1-34): the library's
// SGEMM per K panel plus two launches that do what the reference's six SGEMV, two SAXPY and two SDOT calls do.
#include "common.h"

namespace hpcdnn {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;
constexpr int kGemvColsPerBlock = 4 * kWave;  // one 16-byte load per lane
constexpr int kGemvMaxChunks = 128;

// y[m] = alpha * sum_n A[m][n] x[n] + beta * y[m].  One wave per group of kGemvRows rows: the rows are read in 1 KiB
// pieces (one 16-byte load per lane), 8 / kGemvRows pieces of each row in flight, against the same two pieces of x, so x is
// fetched once per four rows; columns >= N read as 0 through the descriptors.  The lane partials are added in a fixed
// order, so the result does not depend on timing.  kGemvRows = 1 (one row per wave, more waves) suits matrices with
// few or short rows.
template <int kGemvRows>
__global__ __launch_bounds__(kGemvThreads) void sgemv_n_kernel(int M, int N, float alpha, const float* __restrict__ A,
                                                               int lda, const float* __restrict__ x, float beta,
                                                               float* __restrict__ y) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const __amdgpu_buffer_rsrc_t xr = make_rsrc(x, static_cast<int64_t>(N) * 4);
    for (int m = kGemvRows * (blockIdx.x * kGemvWaves + wave); m < M; m += kGemvRows * gridDim.x * kGemvWaves) {
        __amdgpu_buffer_rsrc_t ar[kGemvRows];
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r) {
            const bool valid = m + r < M;
            ar[r] = make_rsrc(A + static_cast<int64_t>(valid ? m + r : m) * lda, valid ? static_cast<int64_t>(N) * 4 : 0);
        }
        v4f acc[kGemvRows];
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r) acc[r] = v4f{0.f, 0.f, 0.f, 0.f};
        constexpr int kPieces = 8 / kGemvRows < 4 ? 8 / kGemvRows : 4;
        for (int n0 = 0; n0 < N; n0 += kPieces * kGemvColsPerBlock) {
            v4f a[kGemvRows][kPieces], xv[kPieces];
#pragma unroll
            for (int r = 0; r < kGemvRows; ++r)
#pragma unroll
                for (int u = 0; u < kPieces; ++u) a[r][u] = buffer_load_v4f(ar[r], (n0 + u * kGemvColsPerBlock + lane * 4) * 4);
#pragma unroll
            for (int u = 0; u < kPieces; ++u) xv[u] = buffer_load_v4f(xr, (n0 + u * kGemvColsPerBlock + lane * 4) * 4);
#pragma unroll
            for (int r = 0; r < kGemvRows; ++r)
#pragma unroll
                for (int u = 0; u < kPieces; ++u) {
                    acc[r].x = __builtin_fmaf(a[r][u].x, xv[u].x, acc[r].x);
                    acc[r].y = __builtin_fmaf(a[r][u].y, xv[u].y, acc[r].y);
                    acc[r].z = __builtin_fmaf(a[r][u].z, xv[u].z, acc[r].z);
                    acc[r].w = __builtin_fmaf(a[r][u].w, xv[u].w, acc[r].w);
                }
        }
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r) {
            const float s = wave_sum_lane63((acc[r].x + acc[r].y) + (acc[r].z + acc[r].w));
            if (lane == kWave - 1 && m + r < M) y[m + r] = (beta == 0.f) ? alpha * s : __builtin_fmaf(beta, y[m + r], alpha * s);
        }
    }
}

// The same product for matrices with rows of 2048 ... 16384 elements: x is copied to LDS once per workgroup (zeros
// behind its end), every wave walks one row at a time in pieces of 16 KiB (sixteen 16-byte loads per lane in flight)
// and multiplies them with x from LDS, so the only traffic to memory is the stream of A.  Workgroup b owns the
// contiguous rows [b * rows_per_block, ...), wave w every fourth of them.  Measured 6.97 TB/s at 16384^2 against
// 6.4 for the kernel above, whose x comes from L2 with every piece.
constexpr int kGemvLdsMaxN = 16384;
constexpr int kGemvLdsLoads = 16;
constexpr int kGemvLdsStep = kGemvLdsLoads * kGemvColsPerBlock;  // 4096 columns per wave and pass

__global__ __launch_bounds__(kGemvThreads) void sgemv_n_lds_kernel(int M, int N, int rows_per_block, float alpha,
                                                                   const float* __restrict__ A, int lda,
                                                                   const float* __restrict__ x, float beta,
                                                                   float* __restrict__ y) {
    extern __shared__ __align__(16) float xs[];  // N rounded up to a multiple of kGemvLdsStep
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int padded = (N + kGemvLdsStep - 1) / kGemvLdsStep * kGemvLdsStep;
    // 16-byte groups through a descriptor over x (zeros behind its end), eight in flight per thread
    {
        const __amdgpu_buffer_rsrc_t xr = make_rsrc(x, static_cast<int64_t>(N) * 4);
        constexpr int kBatch = 8;
        for (int i = threadIdx.x * 4; i < padded; i += kBatch * kGemvThreads * 4) {
            v4f t[kBatch];
#pragma unroll
            for (int u = 0; u < kBatch; ++u) t[u] = buffer_load_v4f(xr, (i + u * kGemvThreads * 4) * 4);
#pragma unroll
            for (int u = 0; u < kBatch; ++u)
                if (i + u * kGemvThreads * 4 < padded) *reinterpret_cast<v4f*>(xs + i + u * kGemvThreads * 4) = t[u];
        }
    }
    __syncthreads();
    const int first = blockIdx.x * rows_per_block;
    const int last = (M - first < rows_per_block) ? M : first + rows_per_block;
    for (int m = first + wave; m < last; m += kGemvWaves) {
        const __amdgpu_buffer_rsrc_t ar = make_rsrc(A + static_cast<int64_t>(m) * lda, static_cast<int64_t>(N) * 4);
        float acc[kGemvLdsLoads];
#pragma unroll
        for (int u = 0; u < kGemvLdsLoads; ++u) acc[u] = 0.f;
        for (int n0 = 0; n0 < N; n0 += kGemvLdsStep) {
            v4f a[kGemvLdsLoads];
#pragma unroll
            for (int u = 0; u < kGemvLdsLoads; ++u) a[u] = buffer_load_v4f_nt(ar, (n0 + u * kGemvColsPerBlock + lane * 4) * 4);
#pragma unroll
            for (int u = 0; u < kGemvLdsLoads; ++u) {
                const v4f xv = *reinterpret_cast<const v4f*>(xs + n0 + u * kGemvColsPerBlock + lane * 4);
                acc[u] = __builtin_fmaf(a[u].x, xv.x, acc[u]);
                acc[u] = __builtin_fmaf(a[u].y, xv.y, acc[u]);
                acc[u] = __builtin_fmaf(a[u].z, xv.z, acc[u]);
                acc[u] = __builtin_fmaf(a[u].w, xv.w, acc[u]);
            }
        }
        float s = acc[0];
#pragma unroll
        for (int u = 1; u < kGemvLdsLoads; ++u) s += acc[u];
        s = wave_sum_lane63(s);
        if (lane == kWave - 1) y[m] = (beta == 0.f) ? alpha * s : __builtin_fmaf(beta, y[m], alpha * s);
    }
}

// out[n] = sum over the rows m of one chunk of A[m][n] x[m], for the 256 columns of one block.  Wave w takes rows
// first + w, first + w + 4, ... (U of them in flight): every load is one 1 KiB piece of a row; the four wave partials are added in wave
// order.  With partial == nullptr (a single chunk) the block finishes y itself; otherwise it writes its chunk's
// partial sums and sgemv_t_finish_kernel adds the chunks in order.
template <int U>
__global__ __launch_bounds__(kGemvThreads) void sgemv_t_kernel(int M, int N, int rows_per_chunk, float alpha,
                                                               const float* __restrict__ A, int lda,
                                                               const float* __restrict__ x, float beta,
                                                               float* __restrict__ y, float* __restrict__ partial) {
    __shared__ v4f part[kGemvWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int n0 = blockIdx.x * kGemvColsPerBlock;
    const int first = blockIdx.y * rows_per_chunk;
    const int last = (M - first < rows_per_chunk) ? M : first + rows_per_chunk;
    const int64_t row_bytes = static_cast<int64_t>(N - n0) * 4;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    for (int m = first + wave; m < last; m += U * kGemvWaves) {
        v4f a[U];
        float xm[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int mm = m + u * kGemvWaves;
            const bool valid = mm < last;
            const int mc = valid ? mm : first;
            a[u] = buffer_load_v4f(make_rsrc(A + static_cast<int64_t>(mc) * lda + n0, valid ? row_bytes : 0), lane * 16);
            xm[u] = valid ? x[mc] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            acc.x = __builtin_fmaf(a[u].x, xm[u], acc.x);
            acc.y = __builtin_fmaf(a[u].y, xm[u], acc.y);
            acc.z = __builtin_fmaf(a[u].z, xm[u], acc.z);
            acc.w = __builtin_fmaf(a[u].w, xm[u], acc.w);
        }
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    v4f t = part[0][lane];
#pragma unroll
    for (int w = 1; w < kGemvWaves; ++w) t += part[w][lane];
    const float tv[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const int n = n0 + lane * 4 + e;
        if (n >= N) break;
        if (partial)
            partial[static_cast<int64_t>(blockIdx.y) * N + n] = tv[e];
        else
            y[n] = (beta == 0.f) ? alpha * tv[e] : __builtin_fmaf(beta, y[n], alpha * tv[e]);
    }
}

// The transposed product for wide matrices: every *wave* owns a strip of 2048 columns and a chunk of rows, keeps
// the strip's 2048 partial sums in registers (8 x 4 per lane) and walks its rows two at a time (sixteen 16-byte
// loads in flight, each row 8 KiB of contiguous memory); no LDS, no barrier.  Partial sums go to
// partial[chunk][n] and sgemv_t_finish_kernel adds the chunks in order; with a single chunk the wave finishes y.
// Measured 6.7 TB/s at 16384^2 with 128 chunks (finish included) against 6.1 for the kernel above.
constexpr int kGemvStripLoads = 8;
constexpr int kGemvStripCols = kGemvStripLoads * kGemvColsPerBlock;  // 2048

__global__ __launch_bounds__(kGemvThreads) void sgemv_t_strip_kernel(int M, int N, int rows_per_chunk, int strips, int waves,
                                                                     float alpha, const float* __restrict__ A, int lda,
                                                                     const float* __restrict__ x, float beta,
                                                                     float* __restrict__ y, float* __restrict__ partial) {
    const int lane = threadIdx.x & (kWave - 1);
    const int gw = __builtin_amdgcn_readfirstlane(blockIdx.x * kGemvWaves + threadIdx.x / kWave);
    if (gw >= waves) return;
    const int strip = gw % strips, chunk = gw / strips;
    const int c0 = strip * kGemvStripCols;
    const int first = chunk * rows_per_chunk;
    const int last = (M - first < rows_per_chunk) ? M : first + rows_per_chunk;
    const int64_t row_bytes = static_cast<int64_t>(N - c0) * 4;
    v4f acc[kGemvStripLoads];
#pragma unroll
    for (int u = 0; u < kGemvStripLoads; ++u) acc[u] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int m = first; m < last; m += 2) {
        v4f a[2][kGemvStripLoads];
        float xm[2];
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const bool valid = m + q < last;
            const int mc = valid ? m + q : first;
            const __amdgpu_buffer_rsrc_t ar = make_rsrc(A + static_cast<int64_t>(mc) * lda + c0, valid ? row_bytes : 0);
            xm[q] = valid ? x[mc] : 0.f;
#pragma unroll
            for (int u = 0; u < kGemvStripLoads; ++u) a[q][u] = buffer_load_v4f_nt(ar, (u * kGemvColsPerBlock + lane * 4) * 4);
        }
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int u = 0; u < kGemvStripLoads; ++u) {
                acc[u].x = __builtin_fmaf(a[q][u].x, xm[q], acc[u].x);
                acc[u].y = __builtin_fmaf(a[q][u].y, xm[q], acc[u].y);
                acc[u].z = __builtin_fmaf(a[q][u].z, xm[q], acc[u].z);
                acc[u].w = __builtin_fmaf(a[q][u].w, xm[q], acc[u].w);
            }
    }
#pragma unroll
    for (int u = 0; u < kGemvStripLoads; ++u) {
        const float tv[4] = {acc[u].x, acc[u].y, acc[u].z, acc[u].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int n = c0 + u * kGemvColsPerBlock + lane * 4 + e;
            if (n < N) {
                if (partial)
                    partial[static_cast<int64_t>(chunk) * N + n] = tv[e];
                else
                    y[n] = (beta == 0.f) ? alpha * tv[e] : __builtin_fmaf(beta, y[n], alpha * tv[e]);
            }
        }
    }
}

__global__ __launch_bounds__(kGemvThreads) void sgemv_t_finish_kernel(int N, int chunks, float alpha,
                                                                      const float* __restrict__ partial, float beta,
                                                                      float* __restrict__ y) {
    const int n = blockIdx.x * kGemvThreads + threadIdx.x;
    if (n >= N) return;
    // chunk partials of column n, added in chunk order; eight loads in flight
    float s = 0.f;
    for (int c = 0; c < chunks; c += 8) {
        float t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) t[u] = (c + u < chunks) ? partial[static_cast<int64_t>(c + u) * N + n] : 0.f;
#pragma unroll
        for (int u = 0; u < 8; ++u) s += t[u];
    }
    y[n] = (beta == 0.f) ? alpha * s : __builtin_fmaf(beta, y[n], alpha * s);
}

__global__ __launch_bounds__(kGemvThreads) void fill_const_kernel(float* __restrict__ dst, int64_t n, float value) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kGemvThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kGemvThreads + threadIdx.x; i < n; i += stride) dst[i] = value;
}

__global__ void add_to_element_kernel(float* __restrict__ p, float delta) { *p += delta; }

// Row chunks of the transposed product: enough workgroups (narrow matrices, 256-column blocks) or waves (wide ones,
// 2048-column strips) to fill the device, at least 32 rows each.  A function of the shape only.
static bool gemv_t_wide(int N) { return N >= kGemvStripCols; }

static int gemv_t_chunks(int M, int N) {
    int64_t want;
    if (gemv_t_wide(N))
        want = ceil_div(4 * 256, ceil_div(N, kGemvStripCols));  // about four waves per CU of an MI355X
    else
        want = ceil_div(2 * 256, ceil_div(N, kGemvColsPerBlock));  // about two blocks per CU
    const int64_t most = ceil_div(M, 32);
    if (want > most) want = most;
    if (want > kGemvMaxChunks) want = kGemvMaxChunks;
    return want < 1 ? 1 : static_cast<int>(want);
}

size_t sgemv_workspace_bytes(int M, int N) {
    if (M <= 0 || N <= 0) return 0;
    const int chunks = gemv_t_chunks(M, N);
    return chunks > 1 ? static_cast<size_t>(chunks) * N * sizeof(float) : 0;
}

static int run_sgemv(int trans, int M, int N, float alpha, const float* A, int lda, const float* x, float beta, float* y,
                     void* ws, size_t ws_bytes, hipStream_t s) {
    if (M < 0 || N < 0 || (trans != 0 && trans != 1)) return HPCDNN_ERR_INVALID_VALUE;
    const int ylen = trans ? N : M, xlen = trans ? M : N;
    if (ylen == 0) return HPCDNN_OK;
    if (!y || (xlen > 0 && (!A || !x || lda < N))) return HPCDNN_ERR_INVALID_VALUE;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 3u)
        return HPCDNN_ERR_INVALID_VALUE;
    if (!trans) {
        if (N >= 2048 && N <= kGemvLdsMaxN && M >= kGemvWaves) {
            // x in LDS, one contiguous range of rows per workgroup, one workgroup per CU when there are enough rows
            int rows_per_block = static_cast<int>(ceil_div(ceil_div(M, device_cus()), kGemvWaves)) * kGemvWaves;
            const int grid = static_cast<int>(ceil_div(M, rows_per_block));
            const size_t lds = static_cast<size_t>(ceil_div(N, kGemvLdsStep)) * kGemvLdsStep * sizeof(float);
            sgemv_n_lds_kernel<<<grid, kGemvThreads, lds, s>>>(M, N, rows_per_block, alpha, A, lda, x, beta, y);
            return launch_status();
        }
        const bool grouped = N >= 4096 && M >= 8192;  // long rows and enough of them: share x between four rows
        int64_t grid = ceil_div(M, (grouped ? 4 : 1) * kGemvWaves);
        const int64_t cap = static_cast<int64_t>(device_cus()) * 16;
        if (grid > cap) grid = cap;
        if (grouped)
            sgemv_n_kernel<4><<<static_cast<int>(grid), kGemvThreads, 0, s>>>(M, N, alpha, A, lda, x, beta, y);
        else
            sgemv_n_kernel<1><<<static_cast<int>(grid), kGemvThreads, 0, s>>>(M, N, alpha, A, lda, x, beta, y);
        return launch_status();
    }
    int chunks = gemv_t_chunks(M, N);
    if (chunks > 1 && (!ws || ws_bytes < static_cast<size_t>(chunks) * N * sizeof(float))) chunks = 1;  // slower, same contract
    if (M == 0) chunks = 1;
    const int rows_per_chunk = M > 0 ? static_cast<int>(ceil_div(M, chunks)) : 1;
    chunks = M > 0 ? static_cast<int>(ceil_div(M, rows_per_chunk)) : 1;
    float* partial = chunks > 1 ? static_cast<float*>(ws) : nullptr;
    if (gemv_t_wide(N)) {
        const int strips = static_cast<int>(ceil_div(N, kGemvStripCols)), waves = strips * chunks;
        sgemv_t_strip_kernel<<<static_cast<int>(ceil_div(waves, kGemvWaves)), kGemvThreads, 0, s>>>(M, N, rows_per_chunk, strips, waves,
                                                                                                   alpha, A, lda, x, beta, y, partial);
    } else {
        const dim3 grid(static_cast<unsigned>(ceil_div(N, kGemvColsPerBlock)), chunks);
        sgemv_t_kernel<8><<<grid, kGemvThreads, 0, s>>>(M, N, rows_per_chunk, alpha, A, lda, x, beta, y, partial);
    }
    if (chunks > 8 && N % 4 == 0 && (reinterpret_cast<uintptr_t>(partial) & 15u) == 0)
        // many chunks: the reduction that keeps all of a lane's slices in flight (y as a 1 x N matrix)
        launch_splitk_reduce_wide(1, N, chunks, partial, y, N, alpha, beta, device_cus(), s);
    else if (chunks > 1)
        sgemv_t_finish_kernel<<<static_cast<int>(ceil_div(N, kGemvThreads)), kGemvThreads, 0, s>>>(N, chunks, alpha, partial,
                                                                                                  beta, y);
    return launch_status();
}

// ---- offline ABFT (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:3-31), two launches per K panel behind the GEMM:
//   sums    one grid whose blocks (a) pass over C once for its row *and* column sums (partial per 512-column /
//           64-row block), (b) form the column sums of the A panel and the row sums of the B panel of the *next* K
//           panel (they depend on nothing the GEMM computes, so they are ready a launch ahead), (c) carry this panel's
//           sums through its operands: rowcarry[m] = sum_k A_p[m][k] b_row[k], colcarry[chunk][n] = sum over a chunk
//           of 64 k of a_col[k] B_p[k][n], and (d) one block that adds up the residual block sums of the panel before;
//   finish  one thread per row and per column: running reference += alpha * carried value, sum of C's row / column
//           from its block partials, residual, block sum of the residuals.
// A last small launch after the loop adds up the last panel's block sums.  Every sum is formed in a fixed order: lanes,
// then waves, then blocks by index.
constexpr int kSumRows = 64;            // rows of one block of the sums pass: 16 per wave
constexpr int kSumPieceCols = 4 * kWave;  // one 16-byte load per lane
constexpr int kSumPieces = 2;           // 1 KiB pieces of a row per block: 512 columns
constexpr int kSumCols = kSumPieces * kSumPieceCols;
constexpr int kCarryCols = 256;         // columns per block of the carried column checksum and of the finish launch
constexpr int kCarryChunk = 64;         // k values per block of the carried column checksum
constexpr int kCarryChunks = HPCDNN_OFFLINE_FT_PANEL_K / kCarryChunk;

// rows [r0, r0 + 64) x columns [c0, c0 + PIECES * 256) of a row-major matrix: rowsum[r] = sum over the block's
// columns of row r (lane partials combined by DPP), colsum[c] = sum over the block's rows of column c (in-lane over
// the rows of a wave, then the four waves in order).  Wave w takes rows r0 + w, r0 + w + 4, ..., four of them in
// flight.  Rows >= rows and columns >= cols read as zeros through the descriptors and are not written.  Plain
// loads on purpose: C stays in the memory-side cache for the next panel's GEMM, which reads it again (with the
// non-temporal hint that GEMM ran 4 % slower).
template <int PIECES, bool WANT_ROW, bool WANT_COL>
__device__ __forceinline__ void sums_block(const float* __restrict__ mat, int ld, int rows, int cols, int r0, int c0,
                                           float* __restrict__ rowsum, float* __restrict__ colsum,
                                           v4f (*part)[kSumPieces][kWave]) {
    constexpr int kUnroll = 8;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int64_t row_bytes = static_cast<int64_t>(cols - c0) * 4;
    v4f acc[PIECES];
#pragma unroll
    for (int pc = 0; pc < PIECES; ++pc) acc[pc] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < kSumRows / kGemvWaves; i += kUnroll) {
        v4f a[kUnroll][PIECES];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int r = r0 + wave + kGemvWaves * (i + u);
            const bool valid = r < rows;
            const __amdgpu_buffer_rsrc_t rs = make_rsrc(mat + static_cast<int64_t>(valid ? r : r0) * ld + c0, valid ? row_bytes : 0);
#pragma unroll
            for (int pc = 0; pc < PIECES; ++pc) a[u][pc] = buffer_load_v4f(rs, (pc * kSumPieceCols + lane * 4) * 4);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if constexpr (WANT_COL) {
#pragma unroll
                for (int pc = 0; pc < PIECES; ++pc) acc[pc] += a[u][pc];
            }
            if constexpr (WANT_ROW) {
                float s = (a[u][0].x + a[u][0].y) + (a[u][0].z + a[u][0].w);
#pragma unroll
                for (int pc = 1; pc < PIECES; ++pc) s += (a[u][pc].x + a[u][pc].y) + (a[u][pc].z + a[u][pc].w);
                s = wave_sum_lane63(s);
                const int r = r0 + wave + kGemvWaves * (i + u);
                if (lane == kWave - 1 && r < rows) rowsum[r] = s;
            }
        }
    }
    if constexpr (WANT_COL) {
#pragma unroll
        for (int pc = 0; pc < PIECES; ++pc) part[wave][pc][lane] = acc[pc];
        __syncthreads();
        const int pc = threadIdx.x / kWave, l = lane;  // 256 threads = 4 pieces x 64 lanes
        if (pc < PIECES) {
            v4f t = part[0][pc][l];
#pragma unroll
            for (int w = 1; w < kGemvWaves; ++w) t += part[w][pc][l];
            const float tv[4] = {t.x, t.y, t.z, t.w};
            const int c = c0 + pc * kSumPieceCols + l * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (c + e < cols) colsum[c + e] = tv[e];
        }
    }
}

// base[0] + base[stride] + ... (count terms, added in index order): 32 loads are in flight before the first
// addition waits, instead of one trip to memory per term
__device__ __forceinline__ float strided_sum(const float* __restrict__ base, size_t stride, int count) {
    constexpr int kBatch = 32;
    float s = 0.f;
    int i = 0;
    for (; i + kBatch <= count; i += kBatch) {
        float t[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) t[u] = base[static_cast<size_t>(i + u) * stride];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) s += t[u];
    }
    float t[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) t[u] = (i + u < count) ? base[static_cast<size_t>(i + u) * stride] : 0.f;
#pragma unroll
    for (int u = 0; u < kBatch; ++u) s += t[u];
    return s;
}

struct OfflineArgs {
    int M, N, kp;  // kp: columns of the A panel = rows of the B panel (<= HPCDNN_OFFLINE_FT_PANEL_K)
    const float* C;
    int ldc;
    const float* Ap;  // this panel's operands (carry roles)
    int lda;
    const float* Bp;
    int ldb;
    const float* An;  // the next panel's operands (panel-sum roles) and its width, 0 when there is none
    const float* Bn;
    int kn;
    float alpha;
    float* rowpart;     // [col blocks of C][M]   row sums of C per 512-column block
    float* colpart;     // [row blocks of C][N]   column sums of C per 64-row block
    float* apart;       // [row blocks][panel]    column sums of this panel of A per 64-row block
    float* bpart;       // [col blocks][panel]    row sums of this panel of B per 512-column block
    float* apart_next;  // the same for the next panel, written by the sums launch
    float* bpart_next;
    float* rowcarry;    // [M]                    sum_k A_p[m][k] * b_row[k]
    float* colcarry;    // [kCarryChunks][N]      sum over 64 k of a_col[k] * B_p[k][n]
    float* ref_row;     // [M] running reference row checksum
    float* ref_col;     // [N] running reference column checksum
    double* row_slots;  // residual block sums of the finish launch (256 rows each); scalar variant: totals of C per 64 rows
    double* col_slots;  // [N / 256]           the same for the column sums; scalar variant: [0] = the carried scalar
    float* res_out;     // where the residuals of the panel before this one go (sums launch), or nullptr
    // roles of the sums launch, in this order; one more block when res_out is set
    int c_blocks, a_blocks, b_blocks, rc_blocks, cc_blocks;
    int row_blocks, col_blocks;        // 64-row blocks of C, 512-column blocks of C
    int fin_row_blocks, fin_col_blocks;  // 256-row / 256-column blocks of the finish launch
    // one scalar checksum per panel (hpcdnn_offline_ft_sgemm_scalar): the running reference total
    double* scalar_ref;
    int scalar;
};

// residual sums of a panel: the block partials added in block order
__device__ __forceinline__ void finish_residuals(const OfflineArgs& p) {
    if (threadIdx.x != 0) return;
    if (p.scalar) {
        // total of C (block partials in block order) against the reference carried through the operands
        double total = 0.0;
        for (int b = 0; b < p.row_blocks; ++b) total += p.row_slots[b];
        const double ref = *p.scalar_ref + p.col_slots[0];
        *p.scalar_ref = ref;
        p.res_out[0] = static_cast<float>(total - ref);
        return;
    }
    double sc = 0.0, sr = 0.0;
    for (int b = 0; b < p.fin_col_blocks; ++b) sc += p.col_slots[b];
    for (int b = 0; b < p.fin_row_blocks; ++b) sr += p.row_slots[b];
    p.res_out[0] = static_cast<float>(sc);
    p.res_out[1] = static_cast<float>(sr);
}

// sum of a double over the block, valid in thread 0 (wave partials added in wave order)
__device__ __forceinline__ double block_sum_f64(double v, double* lds) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = v;
    __syncthreads();
    double s = 0.0;
    if (threadIdx.x == 0)
        for (int w = 0; w < kGemvWaves; ++w) s += lds[w];
    return s;
}

// rowcarry[m] = sum_k A_p[m][k] * b_row[k] for the 64 rows of block rb (b_row = the B panel's row sums, its
// column-block partials added in order): one wave per row, the row's 256 values in one load.  (baseline_ft_sgemm.cuh:23)
__device__ __forceinline__ void carry_rows_block(const OfflineArgs& p, int rb, float* vec) {
    constexpr int pk = HPCDNN_OFFLINE_FT_PANEL_K;
    static_assert(pk == kGemvThreads && pk == kSumPieceCols, "one thread per k of a panel, one piece per panel row of A");
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    vec[tid] = tid < p.kp ? strided_sum(p.bpart + tid, pk, p.col_blocks) : 0.f;
    __syncthreads();
    const v4f bv = *reinterpret_cast<const v4f*>(vec + lane * 4);
    const int r0 = rb * kSumRows;
    constexpr int kUnroll = 16;
    static_assert(kSumRows / kGemvWaves == kUnroll, "all rows of a wave in one batch");
    v4f a[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int r = r0 + wave + kGemvWaves * u;
        const bool valid = r < p.M;
        a[u] = buffer_load_v4f(make_rsrc(p.Ap + static_cast<int64_t>(valid ? r : r0) * p.lda, valid ? static_cast<int64_t>(p.kp) * 4 : 0), lane * 16);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int r = r0 + wave + kGemvWaves * u;
        float s = __builtin_fmaf(a[u].x, bv.x, 0.f);
        s = __builtin_fmaf(a[u].y, bv.y, s);
        s = __builtin_fmaf(a[u].z, bv.z, s);
        s = __builtin_fmaf(a[u].w, bv.w, s);
        s = wave_sum_lane63(s);
        if (lane == kWave - 1 && r < p.M) p.rowcarry[r] = s;
    }
}

// colcarry[chunk][n] = sum over the 64 k of the chunk of a_col[k] * B_p[k][n] for the 256 columns of block cbk (a_col
// from its row-block partials): wave w takes rows w, w + 4, ... of the chunk, all sixteen in flight; the four wave
// partials are added in wave order.  (baseline_ft_sgemm.cuh:20)
__device__ __forceinline__ void carry_cols_block(const OfflineArgs& p, int cbk, int chunk, float* vec, v4f (*part)[kWave]) {
    constexpr int pk = HPCDNN_OFFLINE_FT_PANEL_K;
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int c0 = cbk * kCarryCols, k0 = chunk * kCarryChunk;
    if (tid < kCarryChunk) vec[tid] = (k0 + tid < p.kp) ? strided_sum(p.apart + k0 + tid, pk, p.row_blocks) : 0.f;
    __syncthreads();
    const int64_t row_bytes = static_cast<int64_t>(p.N - c0) * 4;
    constexpr int kUnroll = kCarryChunk / kGemvWaves;
    v4f bq[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const int kk = k0 + wave + u * kGemvWaves;
        const bool valid = kk < p.kp;
        bq[u] = buffer_load_v4f(make_rsrc(p.Bp + static_cast<int64_t>(valid ? kk : 0) * p.ldb + c0, valid ? row_bytes : 0), lane * 16);
    }
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
        const float av = vec[wave + u * kGemvWaves];
        acc.x = __builtin_fmaf(bq[u].x, av, acc.x);
        acc.y = __builtin_fmaf(bq[u].y, av, acc.y);
        acc.z = __builtin_fmaf(bq[u].z, av, acc.z);
        acc.w = __builtin_fmaf(bq[u].w, av, acc.w);
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0) {
        v4f t = part[0][lane];
#pragma unroll
        for (int w = 1; w < kGemvWaves; ++w) t += part[w][lane];
        const float tv[4] = {t.x, t.y, t.z, t.w};
        float* dst = p.colcarry + static_cast<size_t>(chunk) * p.N;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (c0 + lane * 4 + e < p.N) dst[c0 + lane * 4 + e] = tv[e];
    }
}

__global__ __launch_bounds__(kGemvThreads) void offline_sums_kernel(const OfflineArgs p) {
    __shared__ v4f part[kGemvWaves][kSumPieces][kWave];
    __shared__ float vec[HPCDNN_OFFLINE_FT_PANEL_K];
    int b = blockIdx.x;
    if (b < p.c_blocks) {
        const int rb = b / p.col_blocks, cb = b % p.col_blocks;
        sums_block<kSumPieces, true, true>(p.C, p.ldc, p.M, p.N, rb * kSumRows, cb * kSumCols, p.rowpart + static_cast<size_t>(cb) * p.M,
                                           p.colpart + static_cast<size_t>(rb) * p.N, part);
        return;
    }
    b -= p.c_blocks;
    if (b < p.a_blocks) {  // column sums of the next A panel (M x kn): one 256-column piece
        sums_block<1, false, true>(p.An, p.lda, p.M, p.kn, b * kSumRows, 0, nullptr, p.apart_next + static_cast<size_t>(b) * HPCDNN_OFFLINE_FT_PANEL_K, part);
        return;
    }
    b -= p.a_blocks;
    if (b < p.b_blocks) {  // row sums of the next B panel (kn x N)
        const int rb = b / p.col_blocks, cb = b % p.col_blocks;
        sums_block<kSumPieces, true, false>(p.Bn, p.ldb, p.kn, p.N, rb * kSumRows, cb * kSumCols,
                                            p.bpart_next + static_cast<size_t>(cb) * HPCDNN_OFFLINE_FT_PANEL_K, nullptr, part);
        return;
    }
    b -= p.b_blocks;
    if (b < p.rc_blocks) {
        carry_rows_block(p, b, vec);
        return;
    }
    b -= p.rc_blocks;
    if (b < p.cc_blocks) {
        carry_cols_block(p, b / kCarryChunks, b % kCarryChunks, vec, reinterpret_cast<v4f(*)[kWave]>(&part[0][0][0]));
        return;
    }
    finish_residuals(p);
}

// One thread per row (blocks 0 .. fin_row_blocks-1) or per column: the carried value goes into the running reference,
// the row / column sum of C is put together from its block partials, and the residuals of the block's 256 lines are
// summed.  (baseline_ft_sgemm.cuh:26-30)
__global__ __launch_bounds__(kGemvThreads) void offline_finish_lines_kernel(const OfflineArgs p) {
    __shared__ double red[kGemvWaves];
    const int tid = threadIdx.x;
    double d = 0.0;
    if (static_cast<int>(blockIdx.x) < p.fin_row_blocks) {
        const int r = blockIdx.x * kGemvThreads + tid;
        if (r < p.M) {
            const float ref = __builtin_fmaf(p.alpha, p.rowcarry[r], p.ref_row[r]);
            p.ref_row[r] = ref;
            d = static_cast<double>(strided_sum(p.rowpart + r, p.M, p.col_blocks) - ref);
        }
        const double s = block_sum_f64(d, red);
        if (tid == 0) p.row_slots[blockIdx.x] = s;
        return;
    }
    const int cb = blockIdx.x - p.fin_row_blocks, n = cb * kCarryCols + tid;
    if (n < p.N) {
        float carried = p.colcarry[n];
#pragma unroll
        for (int ch = 1; ch < kCarryChunks; ++ch) carried += p.colcarry[static_cast<size_t>(ch) * p.N + n];
        const float ref = __builtin_fmaf(p.alpha, carried, p.ref_col[n]);
        p.ref_col[n] = ref;
        d = static_cast<double>(strided_sum(p.colpart + n, p.N, p.row_blocks) - ref);
    }
    const double s = block_sum_f64(d, red);
    if (tid == 0) p.col_slots[cb] = s;
}

// One scalar checksum per panel.  Blocks 0 .. row_blocks-1: the sum of C over 64 rows, from the row sums of the sums
// pass (column-block partials in order, rows in order within a thread, threads by block_sum_f64).  The last block:
// alpha * sum_k a_col[k] * b_row[k], the panel's contribution to e^T (A B) e.
__global__ __launch_bounds__(kGemvThreads) void offline_scalar_kernel(const OfflineArgs p) {
    constexpr int pk = HPCDNN_OFFLINE_FT_PANEL_K;
    __shared__ double red[kGemvWaves];
    const int tid = threadIdx.x;
    if (static_cast<int>(blockIdx.x) < p.row_blocks) {
        const int r = blockIdx.x * kSumRows + tid;
        double d = 0.0;
        if (tid < kSumRows && r < p.M) d = static_cast<double>(strided_sum(p.rowpart + r, p.M, p.col_blocks));
        const double s = block_sum_f64(d, red);
        if (tid == 0) p.row_slots[blockIdx.x] = s;
        return;
    }
    double d = 0.0;
    if (tid < p.kp) {
        const float ak = strided_sum(p.apart + tid, pk, p.row_blocks), bk = strided_sum(p.bpart + tid, pk, p.col_blocks);
        d = static_cast<double>(ak) * static_cast<double>(bk);
    }
    const double s = block_sum_f64(d, red);
    if (tid == 0) p.col_slots[0] = static_cast<double>(p.alpha) * s;
}

// the running scalar reference before the first panel: beta times the total of the C that is there (its row sums
// from a sums pass), or zero
__global__ __launch_bounds__(kGemvThreads) void offline_scalar_init_kernel(const OfflineArgs p, float beta) {
    __shared__ double red[kGemvWaves];
    double d = 0.0;
    if (beta != 0.f)
        for (int r = threadIdx.x; r < p.M; r += kGemvThreads) d += static_cast<double>(strided_sum(p.rowpart + r, p.M, p.col_blocks));
    const double s = block_sum_f64(d, red);
    if (threadIdx.x == 0) *p.scalar_ref = static_cast<double>(beta) * s;
}

// running references before the first panel: beta times the sums of the C that is there, or zeros
__global__ __launch_bounds__(kGemvThreads) void offline_init_kernel(const OfflineArgs p, float beta) {
    const int i = blockIdx.x * kGemvThreads + threadIdx.x;
    if (i < p.M) {
        p.ref_row[i] = beta != 0.f ? beta * strided_sum(p.rowpart + i, p.M, p.col_blocks) : 0.f;
    }
    if (i < p.N) {
        p.ref_col[i] = beta != 0.f ? beta * strided_sum(p.colpart + i, p.N, p.row_blocks) : 0.f;
    }
}

__global__ void offline_finish_kernel(const OfflineArgs p) { finish_residuals(p); }

// ---- workspace carving (sizes in floats, each region 64-float aligned)
struct OfflineWs {
    size_t rowpart, colpart, apart, bpart, rowcarry, colcarry, ref_row, ref_col, slots, total;
    size_t apart_len, bpart_len;  // one of the two panel-sum buffers each
};

static size_t align64(size_t v) { return (v + 63) & ~static_cast<size_t>(63); }

static OfflineWs offline_layout(int M, int N) {
    constexpr size_t pk = HPCDNN_OFFLINE_FT_PANEL_K;
    const size_t rb = static_cast<size_t>(ceil_div(M, kSumRows)), cb = static_cast<size_t>(ceil_div(N, kSumCols));
    OfflineWs w{};
    size_t off = 0;
    w.rowpart = off; off += align64(cb * M);
    w.colpart = off; off += align64(rb * N);
    w.apart_len = align64(rb * pk);
    w.bpart_len = align64(cb * pk);
    w.apart = off; off += 2 * w.apart_len;  // this panel's and the next one's
    w.bpart = off; off += 2 * w.bpart_len;
    w.rowcarry = off; off += align64(M);
    w.colcarry = off; off += align64(static_cast<size_t>(kCarryChunks) * N);
    w.ref_row = off; off += align64(M);
    w.ref_col = off; off += align64(N);
    w.slots = off; off += align64(2 * (rb + static_cast<size_t>(ceil_div(N, kCarryCols)) + 1));  // doubles; the last one is the scalar reference
    w.total = off;
    return w;
}

size_t offline_ft_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return offline_layout(M, N).total * sizeof(float);
}

}  // namespace hpcdnn

using namespace hpcdnn;

extern "C" int hpcdnn_sgemv(int trans, int M, int N, float alpha, const float* A, int lda, const float* x, float beta,
                            float* y, void* ws, size_t ws_bytes, void* stream) {
    return run_sgemv(trans, M, N, alpha, A, lda, x, beta, y, ws, ws_bytes, static_cast<hipStream_t>(stream));
}

static int run_offline_ft_sgemm(bool scalar, int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                                int ldc, float alpha, float beta, const hpcdnn_fault* inject, float* residuals, void* ws,
                                size_t ws_bytes, void* stream) {
    if (M < 0 || N < 0 || K < 0) return HPCDNN_ERR_INVALID_VALUE;
    if (M == 0 || N == 0) return HPCDNN_OK;
    constexpr int pk = HPCDNN_OFFLINE_FT_PANEL_K;
    const int panels = K > 0 ? static_cast<int>(ceil_div(K, pk)) : 0;
    const int per_panel = scalar ? 1 : 2;  // residuals per panel
    if (panels > 0 && !residuals) return HPCDNN_ERR_INVALID_VALUE;
    if (inject && (inject->tile < 0 || inject->tile >= panels || inject->row < 0 || inject->row >= M || inject->col < 0 ||
                   inject->col >= N))
        return HPCDNN_ERR_INVALID_VALUE;
    const OfflineWs w = offline_layout(M, N);
    if (K > 0 && (!ws || ws_bytes < w.total * sizeof(float) || (reinterpret_cast<uintptr_t>(ws) & 15u)))
        return HPCDNN_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (K == 0)  // nothing to check: C = beta * C
        return hpcdnn_sgemm(M, N, 0, A, lda, B, ldb, C, ldc, alpha, beta, nullptr, 0, stream);

    float* base = static_cast<float*>(ws);
    OfflineArgs a{};
    a.M = M; a.N = N;
    a.C = C; a.ldc = ldc; a.lda = lda; a.ldb = ldb;
    a.alpha = alpha;
    a.rowpart = base + w.rowpart; a.colpart = base + w.colpart;
    a.rowcarry = base + w.rowcarry; a.colcarry = base + w.colcarry;
    a.ref_row = base + w.ref_row; a.ref_col = base + w.ref_col;
    a.row_blocks = static_cast<int>(ceil_div(M, kSumRows));
    a.col_blocks = static_cast<int>(ceil_div(N, kSumCols));
    a.fin_row_blocks = static_cast<int>(ceil_div(M, kGemvThreads));
    a.fin_col_blocks = static_cast<int>(ceil_div(N, kCarryCols));
    a.row_slots = reinterpret_cast<double*>(base + w.slots);
    a.col_slots = a.row_slots + a.row_blocks;
    a.scalar_ref = a.col_slots + a.fin_col_blocks;
    a.scalar = scalar ? 1 : 0;
    float* apart[2] = {base + w.apart, base + w.apart + w.apart_len};
    float* bpart[2] = {base + w.bpart, base + w.bpart + w.bpart_len};
    int rc = HPCDNN_OK;
    // running reference checksums start from what C already holds (nothing when beta == 0: C is not read then); the
    // same launch forms the sums of the first panels of A and B
    {
        OfflineArgs first = a;
        first.c_blocks = beta != 0.f ? a.row_blocks * a.col_blocks : 0;
        first.An = A;
        first.Bn = B;
        first.kn = K < pk ? K : pk;
        first.apart_next = apart[0];
        first.bpart_next = bpart[0];
        first.a_blocks = a.row_blocks;
        first.b_blocks = static_cast<int>(ceil_div(first.kn, kSumRows)) * a.col_blocks;
        offline_sums_kernel<<<first.c_blocks + first.a_blocks + first.b_blocks, kGemvThreads, 0, s>>>(first);
    }
    if (scalar) {
        offline_scalar_init_kernel<<<1, kGemvThreads, 0, s>>>(a, beta);
    } else {
        const int most = M > N ? M : N;
        offline_init_kernel<<<static_cast<int>(ceil_div(most, kGemvThreads)), kGemvThreads, 0, s>>>(a, beta);
    }
    rc = launch_status();
    if (rc != HPCDNN_OK) return rc;
    a.c_blocks = a.row_blocks * a.col_blocks;
    for (int p = 0; p < panels; ++p) {
        const int k0 = p * pk, kp = (K - k0 < pk) ? K - k0 : pk;
        a.kp = kp;
        a.Ap = A + k0;
        a.Bp = B + static_cast<int64_t>(k0) * ldb;
        a.apart = apart[p & 1];
        a.bpart = bpart[p & 1];
        // the panel's product (baseline_ft_sgemm.cuh:5)
        rc = hpcdnn_sgemm(M, N, kp, a.Ap, lda, a.Bp, ldb, C, ldc, alpha, p == 0 ? beta : 1.f, nullptr, 0, stream);
        if (rc != HPCDNN_OK) return rc;
        if (inject && inject->tile == p)
            add_to_element_kernel<<<1, 1, 0, s>>>(C + static_cast<int64_t>(inject->row) * ldc + inject->col, inject->delta);
        // row and column sums of C (:8-11), the next panel's sums (:14-17), this panel's sums carried through its
        // operands (:20-23); one more block finishes the residuals of the panel before
        const int kn = p + 1 < panels ? ((K - k0 - pk < pk) ? K - k0 - pk : pk) : 0;
        a.kn = kn;
        a.An = A + k0 + pk;
        a.Bn = B + static_cast<int64_t>(k0 + pk) * ldb;
        a.apart_next = apart[(p + 1) & 1];
        a.bpart_next = bpart[(p + 1) & 1];
        a.a_blocks = kn > 0 ? a.row_blocks : 0;
        a.b_blocks = kn > 0 ? static_cast<int>(ceil_div(kn, kSumRows)) * a.col_blocks : 0;
        a.rc_blocks = scalar ? 0 : a.row_blocks;
        a.cc_blocks = scalar ? 0 : a.fin_col_blocks * kCarryChunks;
        a.res_out = p > 0 ? residuals + per_panel * (p - 1) : nullptr;
        offline_sums_kernel<<<a.c_blocks + a.a_blocks + a.b_blocks + a.rc_blocks + a.cc_blocks + (p > 0 ? 1 : 0), kGemvThreads, 0, s>>>(a);
        if (scalar) {
            // the total of C and the panel's carried scalar (:42-54)
            offline_scalar_kernel<<<a.row_blocks + 1, kGemvThreads, 0, s>>>(a);
        } else {
            // running references, residual vectors and their block sums (:26-30)
            offline_finish_lines_kernel<<<a.fin_row_blocks + a.fin_col_blocks, kGemvThreads, 0, s>>>(a);
        }
        rc = launch_status();
        if (rc != HPCDNN_OK) return rc;
    }
    a.res_out = residuals + per_panel * (panels - 1);
    offline_finish_kernel<<<1, kWave, 0, s>>>(a);
    return launch_status();
}

extern "C" int hpcdnn_offline_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                                       int ldc, float alpha, float beta, const hpcdnn_fault* inject, float* residuals,
                                       void* ws, size_t ws_bytes, void* stream) {
    return run_offline_ft_sgemm(false, M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, inject, residuals, ws, ws_bytes, stream);
}

extern "C" int hpcdnn_offline_ft_sgemm_scalar(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                                              int ldc, float alpha, float beta, const hpcdnn_fault* inject, float* residuals,
                                              void* ws, size_t ws_bytes, void* stream) {
    return run_offline_ft_sgemm(true, M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, inject, residuals, ws, ws_bytes, stream);
}
