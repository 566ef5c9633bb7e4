// SGEMV (row-major, both orientations) and the offline ABFT baseline composed from the library's own
// SGEMM + SGEMV + SAXPY + SDOT, the way the reference composes its baseline from cuBLAS calls
// (kernel/ft_sgemm/include/baseline_ft_sgemm.cuh:1-34).
#include "common.h"

namespace hpcdnn {

constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;
constexpr int kGemvColsPerBlock = 4 * kWave;  // one 16-byte load per lane
constexpr int kGemvMaxChunks = 64;

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

__global__ __launch_bounds__(kGemvThreads) void sgemv_t_finish_kernel(int N, int chunks, float alpha,
                                                                      const float* __restrict__ partial, float beta,
                                                                      float* __restrict__ y) {
    const int n = blockIdx.x * kGemvThreads + threadIdx.x;
    if (n >= N) return;
    float s = partial[n];
    for (int c = 1; c < chunks; ++c) s += partial[static_cast<int64_t>(c) * N + n];
    y[n] = (beta == 0.f) ? alpha * s : __builtin_fmaf(beta, y[n], alpha * s);
}

__global__ __launch_bounds__(kGemvThreads) void fill_const_kernel(float* __restrict__ dst, int64_t n, float value) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kGemvThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kGemvThreads + threadIdx.x; i < n; i += stride) dst[i] = value;
}

__global__ void add_to_element_kernel(float* __restrict__ p, float delta) { *p += delta; }

// Row chunks of the transposed product: enough blocks to fill the device, at least 32 rows each.
static int gemv_t_chunks(int M, int N) {
    const int64_t col_blocks = ceil_div(N, kGemvColsPerBlock);
    int64_t want = ceil_div(2 * 256, col_blocks);  // about two blocks per CU of an MI355X; a function of the shape only
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
    const dim3 grid(static_cast<unsigned>(ceil_div(N, kGemvColsPerBlock)), chunks);
    float* partial = chunks > 1 ? static_cast<float*>(ws) : nullptr;
    sgemv_t_kernel<8><<<grid, kGemvThreads, 0, s>>>(M, N, rows_per_chunk, alpha, A, lda, x, beta, y, partial);
    if (chunks > 1)
        sgemv_t_finish_kernel<<<static_cast<int>(ceil_div(N, kGemvThreads)), kGemvThreads, 0, s>>>(N, chunks, alpha, partial,
                                                                                                  beta, y);
    return launch_status();
}

// ---- offline ABFT: workspace carving (all sizes in floats, each region 64-float aligned)
struct OfflineWs {
    size_t ones, c_row, c_col, ref_row, ref_col, a_col, b_row, gemv, sdot, total;
};

static size_t align64(size_t v) { return (v + 63) & ~static_cast<size_t>(63); }

size_t sdot_workspace_bytes();

static OfflineWs offline_layout(int M, int N, int panel_k) {
    OfflineWs w{};
    const size_t mx = static_cast<size_t>(M > N ? M : N);
    size_t off = 0;
    w.ones = off; off += align64(mx > static_cast<size_t>(panel_k) ? mx : panel_k);
    w.c_row = off; off += align64(M);
    w.c_col = off; off += align64(N);
    w.ref_row = off; off += align64(M);
    w.ref_col = off; off += align64(N);
    w.a_col = off; off += align64(panel_k);
    w.b_row = off; off += align64(panel_k);
    size_t g = sgemv_workspace_bytes(M, N);
    const size_t g2 = sgemv_workspace_bytes(M, panel_k), g3 = sgemv_workspace_bytes(panel_k, N);
    if (g2 > g) g = g2;
    if (g3 > g) g = g3;
    w.gemv = off; off += align64(g / sizeof(float));
    w.sdot = off; off += align64(sdot_workspace_bytes() / sizeof(float));
    w.total = off;
    return w;
}

size_t offline_ft_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    return offline_layout(M, N, HPCDNN_OFFLINE_FT_PANEL_K).total * sizeof(float);
}

}  // namespace hpcdnn

using namespace hpcdnn;

extern "C" int hpcdnn_sgemv(int trans, int M, int N, float alpha, const float* A, int lda, const float* x, float beta,
                            float* y, void* ws, size_t ws_bytes, void* stream) {
    return run_sgemv(trans, M, N, alpha, A, lda, x, beta, y, ws, ws_bytes, static_cast<hipStream_t>(stream));
}

extern "C" int hpcdnn_offline_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                                       int ldc, float alpha, float beta, const hpcdnn_fault* inject, float* residuals,
                                       void* ws, size_t ws_bytes, void* stream) {
    if (M < 0 || N < 0 || K < 0) return HPCDNN_ERR_INVALID_VALUE;
    if (M == 0 || N == 0) return HPCDNN_OK;
    constexpr int pk = HPCDNN_OFFLINE_FT_PANEL_K;
    const int panels = K > 0 ? static_cast<int>(ceil_div(K, pk)) : 0;
    if (panels > 0 && !residuals) return HPCDNN_ERR_INVALID_VALUE;
    if (inject && (inject->tile < 0 || inject->tile >= panels || inject->row < 0 || inject->row >= M || inject->col < 0 ||
                   inject->col >= N))
        return HPCDNN_ERR_INVALID_VALUE;
    const OfflineWs w = offline_layout(M, N, pk);
    if (K > 0 && (!ws || ws_bytes < w.total * sizeof(float) || (reinterpret_cast<uintptr_t>(ws) & 15u)))
        return HPCDNN_ERR_WORKSPACE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (K == 0)  // nothing to check: C = beta * C
        return hpcdnn_sgemm(M, N, 0, A, lda, B, ldb, C, ldc, alpha, beta, nullptr, 0, stream);

    float* base = static_cast<float*>(ws);
    float *ones = base + w.ones, *c_row = base + w.c_row, *c_col = base + w.c_col, *ref_row = base + w.ref_row,
          *ref_col = base + w.ref_col, *a_col = base + w.a_col, *b_row = base + w.b_row;
    void* gws = base + w.gemv;
    const size_t gws_bytes = (w.sdot - w.gemv) * sizeof(float);
    void* dws = base + w.sdot;
    const size_t dws_bytes = (w.total - w.sdot) * sizeof(float);
    const int64_t n_ones = static_cast<int64_t>(w.c_row - w.ones);
    fill_const_kernel<<<static_cast<int>(ceil_div(n_ones, kGemvThreads)), kGemvThreads, 0, s>>>(ones, n_ones, 1.0f);
    int rc = hpcdnn_workspace_init(dws, dws_bytes, stream);
    if (rc != HPCDNN_OK) return rc;
#define HPCDNN_TRY(call)              \
    do {                              \
        rc = (call);                  \
        if (rc != HPCDNN_OK) return rc; \
    } while (0)
    // running reference checksums start from what C already holds (nothing when beta == 0: C is not read then)
    if (beta != 0.f) {
        HPCDNN_TRY(run_sgemv(0, M, N, beta, C, ldc, ones, 0.f, ref_row, nullptr, 0, s));
        HPCDNN_TRY(run_sgemv(1, M, N, beta, C, ldc, ones, 0.f, ref_col, gws, gws_bytes, s));
    } else {
        fill_const_kernel<<<static_cast<int>(ceil_div(M, kGemvThreads)), kGemvThreads, 0, s>>>(ref_row, M, 0.f);
        fill_const_kernel<<<static_cast<int>(ceil_div(N, kGemvThreads)), kGemvThreads, 0, s>>>(ref_col, N, 0.f);
    }
    for (int p = 0; p < panels; ++p) {
        const int k0 = p * pk, kp = (K - k0 < pk) ? K - k0 : pk;
        const float* Ap = A + k0;
        const float* Bp = B + static_cast<int64_t>(k0) * ldb;
        // the panel's product (baseline_ft_sgemm.cuh:5)
        HPCDNN_TRY(hpcdnn_sgemm(M, N, kp, Ap, lda, Bp, ldb, C, ldc, alpha, p == 0 ? beta : 1.f, nullptr, 0, stream));
        if (inject && inject->tile == p)
            add_to_element_kernel<<<1, 1, 0, s>>>(C + static_cast<int64_t>(inject->row) * ldc + inject->col, inject->delta);
        // row and column sums of C (:8,:11)
        HPCDNN_TRY(run_sgemv(0, M, N, 1.f, C, ldc, ones, 0.f, c_row, nullptr, 0, s));
        HPCDNN_TRY(run_sgemv(1, M, N, 1.f, C, ldc, ones, 0.f, c_col, gws, gws_bytes, s));
        // column sums of the A panel, row sums of the B panel (:14,:17)
        HPCDNN_TRY(run_sgemv(1, M, kp, 1.f, Ap, lda, ones, 0.f, a_col, gws, gws_bytes, s));
        HPCDNN_TRY(run_sgemv(0, kp, N, 1.f, Bp, ldb, ones, 0.f, b_row, nullptr, 0, s));
        // checksums carried through the operands, added to the running references (:20,:23)
        HPCDNN_TRY(run_sgemv(1, kp, N, alpha, Bp, ldb, a_col, 1.f, ref_col, gws, gws_bytes, s));
        HPCDNN_TRY(run_sgemv(0, M, kp, alpha, Ap, lda, b_row, 1.f, ref_row, nullptr, 0, s));
        // residual vectors and their sums (:26-30)
        HPCDNN_TRY(hpcdnn_saxpy(N, -1.f, ref_col, c_col, stream));
        HPCDNN_TRY(hpcdnn_sdot(N, c_col, ones, residuals + 2 * p, dws, dws_bytes, stream));
        HPCDNN_TRY(hpcdnn_saxpy(M, -1.f, ref_row, c_row, stream));
        HPCDNN_TRY(hpcdnn_sdot(M, c_row, ones, residuals + 2 * p + 1, dws, dws_bytes, stream));
    }
#undef HPCDNN_TRY
    return launch_status();
}
