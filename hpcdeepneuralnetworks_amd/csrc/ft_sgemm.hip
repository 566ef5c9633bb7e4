// ABFT-SGEMM entry points: tile classes, checksum granularity, verification cadence, workspace layout, launch.
#include "gemm_host.h"

namespace hpcdnn {


// row length of the pre-encoded checksum vectors: K rounded up to the K step, plus two K steps of zeros for the
// fetches that run ahead of the main loop
static int ft_enc_ld(int K) { return (static_cast<int>(ceil_div(K, kGemmBK)) + 2) * kGemmBK; }
size_t ft_workspace_bytes(int M, int N, int K);

// ABFT tile classes (the counterpart of the reference's abft_kernel_{huge,large,wide,...} family,
// kernel/ft_sgemm/sgemm.cu:187-188): class 0 is the 256 x 128 tile of HPCDNN_FT_TILE_M/N; the smaller classes keep
// more CUs busy on smaller problems, the 64-column classes (the reference's tall 128 x 32 and medium 32 x 32 shapes,
// kernel/ft_sgemm/code_gen/main.py:8-16, at the size of four waves of 32 x 32 matrix-core blocks) serve products with
// few columns.  Geometry in gemm_host.h (kFtGeom), kernels in ft_kernels.hip, one translation unit per class and
// operand layout.
//
// Without a workspace (FT = 1) four waves: on this part every VALU instruction takes its issue cycles away from the
// FP32 matrix pipe of the same SIMD, whichever wave it comes from, so more waves do not hide the checksum arithmetic;
// fewer, fatter threads need the fewest VALU instructions per K step.  With the operands' checksum vectors read from
// a workspace (FT = 2) no cross-lane reductions are left in the loop, the thread count no longer changes the VALU
// work per SIMD, and eight waves (two per SIMD) hide each other's barriers and LDS latency: measured 2 % faster.
//
// Wave-tile granularity (the counterpart of ft_sgemm_huge_warp.cuh / ft_sgemm_huge_thread.cuh) runs the FT = 2 kernel
// with one checksum pair per wave tile: the tile a wave of the workspace kernel owns, (bm / wgm) x (bn / wgn).
typedef FtGeom FtClass;
static const FtClass* const kFtClasses = kFtGeom;

static FtKernel ft_kernel(int tile_class, bool ta, int kind) {
    switch (tile_class * 2 + (ta ? 1 : 0)) {
        case 0: return ft_kernel_c0_ta0(kind);
        case 1: return ft_kernel_c0_ta1(kind);
        case 2: return ft_kernel_c1_ta0(kind);
        case 3: return ft_kernel_c1_ta1(kind);
        case 4: return ft_kernel_c2_ta0(kind);
        case 5: return ft_kernel_c2_ta1(kind);
        case 6: return ft_kernel_c3_ta0(kind);
        case 7: return ft_kernel_c3_ta1(kind);
        case 8: return ft_kernel_c4_ta0(kind);
        case 9: return ft_kernel_c4_ta1(kind);
        default: return FtKernel{nullptr, nullptr, 0, 0};
    }
}
static EncodeFn ft_encode(int tile_class, bool ta, bool wave) {
    switch (tile_class * 2 + (ta ? 1 : 0)) {
        case 0: return ft_encode_c0_ta0(wave);
        case 1: return ft_encode_c0_ta1(wave);
        case 2: return ft_encode_c1_ta0(wave);
        case 3: return ft_encode_c1_ta1(wave);
        case 4: return ft_encode_c2_ta0(wave);
        case 5: return ft_encode_c2_ta1(wave);
        case 6: return ft_encode_c3_ta0(wave);
        case 7: return ft_encode_c3_ta1(wave);
        case 8: return ft_encode_c4_ta0(wave);
        case 9: return ft_encode_c4_ta1(wave);
        default: return nullptr;
    }
}

// check tile of a class at a granularity: the unit that has a checksum pair, a verification and a status record
static void check_tile(const FtClass& fc, int granularity, int* cm, int* cn) {
    *cm = granularity == HPCDNN_FT_GRAN_WAVE ? fc.bm / fc.wgm : fc.bm;
    *cn = granularity == HPCDNN_FT_GRAN_WAVE ? fc.bn / fc.wgn : fc.bn;
}

// ABFT with a workspace splits the tiles of a partial last round of CUs along K, like plain SGEMM's tail split: every
// slice is a workgroup that verifies (and corrects) its own partial product - the checksums are linear in K - and
// writes it raw; tail_reduce_kernel adds the slices and merges their records.  With fewer tiles
// than half the CUs every tile is split.  A slice is a multiple of `unit` values of k long: the K step, or the
// verification interval, so that every slice of a cadence kernel verifies whole intervals of the K range.  Returns
// the number of ways (1: no split), the tiles it applies to and the slice length.
struct FtTail {
    int ways, tiles, k_chunk;
};
static FtTail ft_tail_plan(const FtClass& fc, int M, int N, int K, int unit = kGemmBK) {
    const FtTail none{1, 0, 0};
    const int cus = device_cus();
    const int64_t tiles = ceil_div(M, fc.bm) * ceil_div(N, fc.bn);
    const int64_t r = tiles % cus;
    if (r == 0 || 2 * r > cus) return none;
    int64_t s = cus / r;
    const int64_t most = K / (16 * kGemmBK);  // at least 16 K steps per slice: each slice pays a verification
    if (s > most) s = most;
    if (s > 8) s = 8;
    if (s < 2) return none;
    const int k_chunk = static_cast<int>(ceil_div(ceil_div(K, s), unit)) * unit;
    s = ceil_div(K, k_chunk);  // drop empty slices
    if (s < 2) return none;
    return FtTail{static_cast<int>(s), static_cast<int>(r), k_chunk};
}
// A product one tile wide or high streams an operand that no other workgroup shares: all its tiles are split along K
// until two workgroups per CU keep enough bytes on their way from memory (at most eight ways, at least 16 K steps per
// slice, slices a multiple of `unit` long).
static FtTail ft_split_all_plan(int tiles, int K, int unit) {
    int64_t ways = ceil_div(2 * device_cus(), tiles);
    const int64_t most = K / (16 * kGemmBK);
    if (ways > most) ways = most;
    if (ways > 8) ways = 8;
    if (ways < 2) return FtTail{1, 0, 0};
    const int k_chunk = static_cast<int>(ceil_div(ceil_div(K, ways), unit)) * unit;
    ways = ceil_div(K, k_chunk);
    if (ways < 2) return FtTail{1, 0, 0};
    return FtTail{static_cast<int>(ways), tiles, k_chunk};
}
// checksum vectors: one row per row group and per column group of the granularity
static size_t ft_enc_bytes(const FtClass& fc, int granularity, int M, int N, int K) {
    const int gm = granularity == HPCDNN_FT_GRAN_WAVE ? fc.wgm : 1, gn = granularity == HPCDNN_FT_GRAN_WAVE ? fc.wgn : 1;
    const size_t b = static_cast<size_t>(ceil_div(M, fc.bm) * gm + ceil_div(N, fc.bn) * gn) * ft_enc_ld(K) * sizeof(float);
    return (b + 15) & ~static_cast<size_t>(15);
}
// the weighted locator's vectors: two rows (plain and weighted row sums of B) per tile column
static size_t ft_weighted_enc_bytes(const FtClass& fc, int N, int K) {
    const size_t b = static_cast<size_t>(2 * ceil_div(N, fc.bn)) * ft_enc_ld(K) * sizeof(float);
    return (b + 15) & ~static_cast<size_t>(15);
}
// the raw tile images of the K slices and their records (one per check tile of the workgroup tile)
static size_t ft_tail_bytes(const FtClass& fc, int granularity, const FtTail& t) {
    const int nct = granularity == HPCDNN_FT_GRAN_WAVE ? fc.wgm * fc.wgn : 1;
    return t.ways < 2 ? 0
                      : static_cast<size_t>(t.tiles) * t.ways * (static_cast<size_t>(fc.bm) * fc.bn * sizeof(float) + nct * sizeof(hpcdnn_ft_status));
}

static size_t ft_class_workspace_bytes(int tile_class, int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const FtClass& fc = kFtClasses[tile_class];
    // (a cadence kernel's slices are at most as many as these, and as long or longer: they fit as well)
    const FtTail tail = ft_tail_plan(fc, M, N, K);
    const size_t tile_mode = ft_enc_bytes(fc, HPCDNN_FT_GRAN_TILE, M, N, K) + ft_tail_bytes(fc, HPCDNN_FT_GRAN_TILE, tail);
    const size_t wave_mode = ft_enc_bytes(fc, HPCDNN_FT_GRAN_WAVE, M, N, K) + ft_tail_bytes(fc, HPCDNN_FT_GRAN_WAVE, tail);
    size_t most = tile_mode > wave_mode ? tile_mode : wave_mode;
    const size_t weighted_mode = ft_weighted_enc_bytes(fc, N, K) + ft_tail_bytes(fc, HPCDNN_FT_GRAN_TILE, tail);
    if (weighted_mode > most) most = weighted_mode;
    // a product one tile wide or high: every tile split up to eight ways by the kernels that need no pre-pass
    const int64_t tiles = ceil_div(M, fc.bm) * ceil_div(N, fc.bn);
    if (ceil_div(M, fc.bm) == 1 || ceil_div(N, fc.bn) == 1) {
        const size_t all = ft_weighted_enc_bytes(fc, N, K) + ft_tail_bytes(fc, HPCDNN_FT_GRAN_TILE, FtTail{8, static_cast<int>(tiles), 0});
        if (all > most) most = all;
    }
    return most;
}

// K == 0 with wave-tile granularity: there is nothing to verify, every check tile gets a clean record
__global__ __launch_bounds__(256) void ft_clean_status_kernel(hpcdnn_ft_status* __restrict__ status, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    hpcdnn_ft_status st;
    st.flag = 0; st.row = -1; st.col = -1; st.n_bad_rows = 0; st.n_bad_cols = 0;
    st.row_residual = 0.f; st.col_residual = 0.f; st.max_clean_residual = 0.f;
    status[i] = st;
}

// ta: A is given transposed (K x M row-major, lda >= M)
static int run_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                        float alpha, float beta, float tau, const hpcdnn_ft_options& opt, hpcdnn_ft_status* status, void* ws,
                        size_t ws_bytes, hipStream_t s, bool ta = false) {
    int rc = check_gemm_args(M, N, K, A, lda, B, ldb, C, ldc, ta);
    if (rc != HPCDNN_OK) return rc;
    if (opt.tile_class < 0 || opt.tile_class >= HPCDNN_FT_NUM_CLASSES) return HPCDNN_ERR_INVALID_VALUE;
    if (opt.granularity != HPCDNN_FT_GRAN_TILE && opt.granularity != HPCDNN_FT_GRAN_WAVE) return HPCDNN_ERR_INVALID_VALUE;
    if (opt.check_interval < 0 || opt.check_interval % kGemmBK != 0) return HPCDNN_ERR_INVALID_VALUE;
    if (opt.n_faults < 0 || opt.n_faults > HPCDNN_FT_MAX_FAULTS) return HPCDNN_ERR_INVALID_VALUE;
    if (opt.locator != HPCDNN_FT_LOCATE_ROW_COL && opt.locator != HPCDNN_FT_LOCATE_WEIGHTED) return HPCDNN_ERR_INVALID_VALUE;
    const FtClass& fc = kFtClasses[opt.tile_class];
    const bool wave = opt.granularity == HPCDNN_FT_GRAN_WAVE;
    const bool user_weighted = opt.locator == HPCDNN_FT_LOCATE_WEIGHTED;
    bool weighted = user_weighted;
    // an interval that covers all of K is a single verification after the loop
    const bool cadence = opt.check_interval > 0 && opt.check_interval < K;
    if (weighted && (wave || cadence)) return HPCDNN_ERR_INVALID_VALUE;  // one pair of checksums per workgroup tile, verified once
    if (M == 0 || N == 0) return HPCDNN_OK;
    if ((wave || weighted) && K > 0 && !ws) return HPCDNN_ERR_WORKSPACE;

    GemmArgs a = make_args(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, fc.bm, fc.bn);
    // tau > 0: absolute; tau <= 0: scaled to the data, the threshold of a line of n elements being f * 4.3 FP32
    // rounding units * sqrt(max(K, 64)) * sqrt(n) * the larger of the line's and the check tile's mean |accumulator|,
    // with f = -tau, or 1 for tau == 0 (the default: a threshold that follows the size and the mean of the operands
    // cannot flag a fault-free product the way a constant calibrated for unit-range data does)
    a.tau = (tau > 0.f) ? tau : 0.f;
    a.tau_rel = (tau > 0.f) ? 0.f : (tau < 0.f ? -tau : 1.f) * 2.56e-7f * sqrtf(static_cast<float>(K > 64 ? K : 64));
    a.status = status;
    a.check_interval = cadence ? opt.check_interval : 0;
    int cm = 0, cn = 0;
    check_tile(fc, opt.granularity, &cm, &cn);
    const int gm = fc.bm / cm, gn = fc.bn / cn;
    a.status_rows = static_cast<int>(ceil_div(M, cm));
    a.status_ld = static_cast<int>(ceil_div(N, cn));
    // faults come in check-tile units; the kernel takes them per workgroup tile
    a.n_faults = opt.n_faults;
    for (int f = 0; f < opt.n_faults; ++f) {
        const hpcdnn_ft_fault_at& in = opt.faults[f];
        if (in.tile < 0 || in.tile >= a.status_rows * a.status_ld || in.row < 0 || in.row >= cm || in.col < 0 ||
            in.col >= cn || in.check < 0)
            return HPCDNN_ERR_INVALID_VALUE;
        const int srow = in.tile / a.status_ld, scol = in.tile % a.status_ld;
        a.faults[f].tile = (srow / gm) * a.tiles_n + scol / gn;
        a.faults[f].row = (srow % gm) * cm + in.row;
        a.faults[f].col = (scol % gn) * cn + in.col;
        a.faults[f].delta = in.delta;
        a.faults[f].check = in.check;
    }
    if (K == 0 && wave) {
        // an empty product: C = beta * C through the workgroup-tile kernel below, which would lay its records out per
        // workgroup tile, so the wave-tile records are written here (all clean; faults have nothing to hit)
        if (status) {
            const int n = a.status_rows * a.status_ld;
            ft_clean_status_kernel<<<static_cast<int>(ceil_div(n, 256)), 256, 0, s>>>(status, n);
            rc = launch_status();
            if (rc != HPCDNN_OK) return rc;
        }
        a.status = nullptr;
        a.n_faults = 0;
    }
    const bool edge = needs_edge(a, fc.bm, fc.bn, kGemmBK);
    dim3 grid(a.tiles_m * a.tiles_n, 1, 1);
    // A product that is one tile wide (or one tile high) reads each row panel of A (column panel of B) in exactly one
    // workgroup: a pre-pass would read that operand a second time for checksum vectors nobody shares, and on a tall
    // product with few columns the operand is all the traffic there is.  Those products run the kernels that form the
    // vectors in their main loop, and use the workspace only to split every tile along K until two workgroups per CU
    // keep enough bytes on their way from memory.
    const bool one_wide = K > 0 && (a.tiles_n == 1 || a.tiles_m == 1) && a.tiles_m * a.tiles_n >= device_cus() / 8;
    // One tile wide, one verification per tile, row x column locator: the kernels of the weighted locator (row sums of B
    // from a pre-pass over B, which is small here; the plain row checksum as the screen) with the column references
    // formed when a row is flagged (locate_rc) - nothing of A is summed in the loop at all.
    const bool row_screen = ws && one_wide && a.tiles_n == 1 && !wave && !cadence && !user_weighted &&
                            ws_bytes >= ft_weighted_enc_bytes(fc, N, K) && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
    if (row_screen) {
        weighted = true;
        a.locate_rc = 1;
    }
    const bool fused_split = ws && one_wide && !wave && !weighted;
    if (fused_split) {
        if (reinterpret_cast<uintptr_t>(ws) & 15u) return HPCDNN_ERR_WORKSPACE;
        const int tiles = a.tiles_m * a.tiles_n;
        FtTail tail = ft_split_all_plan(tiles, K, cadence ? opt.check_interval : kGemmBK);
        if (ws_bytes < ft_tail_bytes(fc, opt.granularity, tail)) tail = FtTail{1, 0, 0};
        const FtKernel k = ft_kernel(opt.tile_class, ta, cadence ? kFtFusedCad : kFtFused);
        if (!k.plain) return HPCDNN_ERR_INVALID_VALUE;
        void (*fn)(const GemmArgs) = edge ? k.edge : k.plain;
        rc = enable_lds(fn, k.lds);
        if (rc != HPCDNN_OK) return rc;
        if (tail.ways >= 2) {
            a.tail_k_chunk = tail.k_chunk;
            a.full_tiles = 0;
            a.tail_split = tail.ways;
            a.tail_partial = static_cast<float*>(ws);
            a.tail_status = reinterpret_cast<hpcdnn_ft_status*>(a.tail_partial + static_cast<size_t>(tiles) * tail.ways * fc.bm * fc.bn);
            grid = dim3(tiles * tail.ways, 1, 1);
        }
        hipLaunchKernelGGL(fn, grid, dim3(k.threads), k.lds, s, a);
        rc = launch_status();
        if (rc != HPCDNN_OK || a.tail_split < 2) return rc;
        tail_reduce_kernel<><<<dim3(tiles, fc.bm / 32), 256, 0, s>>>(M, N, fc.bm, fc.bn, a.tiles_m, a.tiles_n, 0, a.tail_split,
                                                                    a.tail_partial, C, ldc, alpha, beta, a.tail_status, status, 1, 1,
                                                                    a.status_rows, a.status_ld);
        return launch_status();
    }
    // With a workspace the checksum vectors of A and B are formed once per row group / column group by a small
    // bandwidth-bound kernel and the main loop only reads them; without one every workgroup forms them itself.
    if (ws && K > 0) {
        const size_t enc_bytes = weighted ? ft_weighted_enc_bytes(fc, N, K) : ft_enc_bytes(fc, opt.granularity, M, N, K);
        if (ws_bytes < enc_bytes || (reinterpret_cast<uintptr_t>(ws) & 15u)) return HPCDNN_ERR_WORKSPACE;
        // the K split of a partial last round is taken when the workspace has room for it
        FtTail tail = ft_tail_plan(fc, M, N, K, cadence ? opt.check_interval : kGemmBK);
        // (the weighted locator on a product one tile wide or high: every tile split, as the kernels without a pre-pass do)
        if (weighted && (a.tiles_n == 1 || a.tiles_m == 1) && a.tiles_m * a.tiles_n >= device_cus() / 8)
            tail = ft_split_all_plan(a.tiles_m * a.tiles_n, K, kGemmBK);
        if (ws_bytes < enc_bytes + ft_tail_bytes(fc, opt.granularity, tail)) tail = FtTail{1, 0, 0};
        a.enc_ld = ft_enc_ld(K);
        const int row_groups = a.tiles_m * gm, col_groups = a.tiles_n * gn;
        float* enc_a = static_cast<float*>(ws);
        float* enc_b = enc_a + static_cast<size_t>(row_groups) * a.enc_ld;
        a.enc_a = enc_a;
        a.enc_b = enc_b;
        const int k_blocks = static_cast<int>(ceil_div(a.enc_ld, kEncodeKB));
        const int b_blocks = static_cast<int>(ceil_div(N, 128));  // the pre-pass walks B in blocks of 128 columns
        // (ta: the same launch, with the blocks of the A half walking A^T)
        if (weighted) {
            // the two row sums of B per tile column; nothing of A (enc_a carries the weighted vectors to the kernel)
            a.enc_b = static_cast<float*>(ws);
            a.enc_a = a.enc_b + static_cast<size_t>(col_groups) * a.enc_ld;
            float* const wb = static_cast<float*>(ws);
            if (fc.bn == 128)
                abft_encode_weighted_kernel<128><<<dim3(k_blocks * b_blocks), dim3(kEncodeKB * 4), 0, s>>>(N, K, B, ldb, wb, wb + static_cast<size_t>(col_groups) * a.enc_ld,
                                                                                             a.enc_ld, k_blocks, col_groups);
            else
                abft_encode_weighted_kernel<64><<<dim3(k_blocks * b_blocks), dim3(kEncodeKB * 4), 0, s>>>(N, K, B, ldb, wb, wb + static_cast<size_t>(col_groups) * a.enc_ld,
                                                                                            a.enc_ld, k_blocks, col_groups);
        } else {
            const EncodeFn encode = ft_encode(opt.tile_class, ta, wave);
            if (!encode) return HPCDNN_ERR_INVALID_VALUE;
            // (one checksum pair per workgroup tile: the kernels need the column sums of A only - the row sums of B are
            // formed in a verification that has flagged a column - so the blocks of the B half are not launched)
            hipLaunchKernelGGL(encode, dim3(k_blocks * (row_groups + (wave ? b_blocks : 0))), dim3(kEncodeKB * 4), 0, s, M, N, K,
                               A, lda, B, ldb, enc_a, enc_b, a.enc_ld, k_blocks, row_groups, col_groups);
        }
        rc = launch_status();
        if (rc != HPCDNN_OK) return rc;
        const FtKernel k = ft_kernel(opt.tile_class, ta, weighted ? kFtWeighted : wave ? (cadence ? kFtWaveCad : kFtWave) : (cadence ? kFtPreCad : kFtPre));
        if (!k.plain) return HPCDNN_ERR_INVALID_VALUE;
        void (*fn)(const GemmArgs) = edge ? k.edge : k.plain;
        rc = enable_lds(fn, k.lds);
        if (rc != HPCDNN_OK) return rc;
        const int tiles = a.tiles_m * a.tiles_n;
        if (tail.ways >= 2) {
            a.tail_k_chunk = tail.k_chunk;
            a.full_tiles = tiles - tail.tiles;
            a.tail_split = tail.ways;
            a.tail_partial = reinterpret_cast<float*>(static_cast<char*>(ws) + enc_bytes);
            a.tail_status = reinterpret_cast<hpcdnn_ft_status*>(a.tail_partial + static_cast<size_t>(tail.tiles) * tail.ways * fc.bm * fc.bn);
            grid = dim3(a.full_tiles + tail.tiles * tail.ways, 1, 1);
        }
        hipLaunchKernelGGL(fn, grid, dim3(k.threads), k.lds, s, a);
        rc = launch_status();
        if (rc != HPCDNN_OK || a.tail_split < 2) return rc;
        tail_reduce_kernel<><<<dim3(tail.tiles, fc.bm / 32), 256, 0, s>>>(M, N, fc.bm, fc.bn, a.tiles_m, a.tiles_n, a.full_tiles,
                                                                         a.tail_split, a.tail_partial, C, ldc, alpha, beta, a.tail_status,
                                                                         status, gm, gn, a.status_rows, a.status_ld);
        return launch_status();
    }
    const FtKernel k = ft_kernel(opt.tile_class, ta, cadence ? kFtFusedCad : kFtFused);
    if (!k.plain) return HPCDNN_ERR_INVALID_VALUE;
    void (*fn)(const GemmArgs) = edge ? k.edge : k.plain;
    rc = enable_lds(fn, k.lds);
    if (rc != HPCDNN_OK) return rc;
    hipLaunchKernelGGL(fn, grid, dim3(k.threads), k.lds, s, a);
    return launch_status();
}

}  // namespace hpcdnn

using namespace hpcdnn;

extern "C" int hpcdnn_ft_tile_info(int tile_class, int* bm, int* bn) {
    if (tile_class < 0 || tile_class >= HPCDNN_FT_NUM_CLASSES) return HPCDNN_ERR_INVALID_VALUE;
    if (bm) *bm = kFtClasses[tile_class].bm;
    if (bn) *bn = kFtClasses[tile_class].bn;
    return HPCDNN_OK;
}

extern "C" int hpcdnn_ft_check_tile_info(int tile_class, int granularity, int* cm, int* cn) {
    if (tile_class < 0 || tile_class >= HPCDNN_FT_NUM_CLASSES) return HPCDNN_ERR_INVALID_VALUE;
    if (granularity != HPCDNN_FT_GRAN_TILE && granularity != HPCDNN_FT_GRAN_WAVE) return HPCDNN_ERR_INVALID_VALUE;
    int m = 0, n = 0;
    check_tile(kFtClasses[tile_class], granularity, &m, &n);
    if (cm) *cm = m;
    if (cn) *cn = n;
    return HPCDNN_OK;
}

extern "C" int hpcdnn_ft_num_check_tiles(int tile_class, int granularity, int M, int N) {
    int cm = 0, cn = 0;
    if (M < 0 || N < 0 || hpcdnn_ft_check_tile_info(tile_class, granularity, &cm, &cn) != HPCDNN_OK) return 0;
    return static_cast<int>(ceil_div(M, cm) * ceil_div(N, cn));
}

extern "C" int hpcdnn_ft_num_tiles_ex(int tile_class, int M, int N) {
    return hpcdnn_ft_num_check_tiles(tile_class, HPCDNN_FT_GRAN_TILE, M, N);
}

extern "C" int hpcdnn_ft_num_tiles(int M, int N) { return hpcdnn_ft_num_tiles_ex(0, M, N); }

// The class with the shortest predicted run of a call that passes a workspace of ws_bytes (0: none).  Matrix-core
// time: rounds of tiles over the CUs times the tile's flops, a partial last round counting for what its K split leaves
// of it plus the second pass over those tiles (when the workspace has room for the split), with the measured
// efficiency of the smaller tiles relative to the 256-row one.  An operand that is read once cannot arrive faster
// than the bytes in flight allow (two K steps of the tile's rows per resident workgroup and trip to memory), which is
// what decides between the classes on tall products with few columns.
extern "C" int hpcdnn_ft_pick_class_ws(int M, int N, int K, size_t ws_bytes) {
    // measured on squares 1024 ... 6144: the 128-row class keeps up with the 256-row one (two of its workgroups share a CU
    // and cover each other's verification), the 64-row class runs 4-5 % behind; the 64-column classes move twice the
    // operand bytes per flop and only pay where the 128-column ones would multiply empty columns
    static const double rel_eff[HPCDNN_FT_NUM_CLASSES] = {1.0, 1.0, 0.955, 0.92, 0.88};
    // without the pre-pass every workgroup forms the checksum vectors of its own tile in the main loop: additions per
    // product grow as 1 / BM + 1 / BN (measured at 4096 and 2048 cubed)
    static const double rel_eff_fused[HPCDNN_FT_NUM_CLASSES] = {1.0, 0.985, 0.91, 0.90, 0.78};
    static const int resident_max[HPCDNN_FT_NUM_CLASSES] = {1, 2, 2, 2, 3};  // workgroups of the class a CU holds
    constexpr double kPeakFlopsPerCu = 157.3e12 / 256.0, kTrip = 0.73e-6;
    const int cus = device_cus();
    int best = 0;
    double best_cost = 1e300;
    for (int c = 0; c < HPCDNN_FT_NUM_CLASSES; ++c) {
        const FtClass& fc = kFtClasses[c];
        const int64_t tiles = hpcdnn_ft_num_tiles_ex(c, M, N);
        const int tiles_m = static_cast<int>(ceil_div(M, fc.bm)), tiles_n = static_cast<int>(ceil_div(N, fc.bn));
        // as run_ft_sgemm decides: a product one tile wide or high splits every tile; one tile wide with a workspace it
        // takes the rows as the screen (a pre-pass over B only, nothing of A summed in the loop), else it forms the
        // vectors in the loop
        const bool one_wide = K > 0 && (tiles_m == 1 || tiles_n == 1) && tiles >= cus / 8;
        const size_t enc_bytes = ft_enc_bytes(fc, HPCDNN_FT_GRAN_TILE, M, N, K);
        const bool rows_screen = one_wide && tiles_n == 1 && ws_bytes >= ft_weighted_enc_bytes(fc, N, K);
        const bool pre = !one_wide && K > 0 && ws_bytes >= enc_bytes;
        FtTail tail{1, 0, 0};
        if (one_wide) {
            tail = ft_split_all_plan(static_cast<int>(tiles), K, kGemmBK);
            if (ws_bytes < ft_tail_bytes(fc, HPCDNN_FT_GRAN_TILE, tail)) tail = FtTail{1, 0, 0};
        } else if (pre) {
            tail = ft_tail_plan(fc, M, N, K);
            if (ws_bytes < enc_bytes + ft_tail_bytes(fc, HPCDNN_FT_GRAN_TILE, tail)) tail = FtTail{1, 0, 0};
        }
        double rounds = static_cast<double>(ceil_div(tiles > 0 ? tiles : 1, cus));
        int64_t groups = tiles;  // workgroups of the launch
        if (tail.ways >= 2) {
            rounds = static_cast<double>((tiles - tail.tiles) / cus) + static_cast<double>(ceil_div(static_cast<int64_t>(tail.tiles) * tail.ways, cus)) / tail.ways + 0.06;
            groups = tiles - tail.tiles + static_cast<int64_t>(tail.tiles) * tail.ways;
        }
        double cost = rounds * 2.0 * fc.bm * fc.bn * (K > 0 ? K : 1) / kPeakFlopsPerCu / (pre || rows_screen ? rel_eff[c] : rel_eff_fused[c]);
        // the pre-pass reads the operands it sums once more (about 5.5 TB/s), which counts on a product with few columns
        constexpr double kPrePassBytesPerSecond = 5.5e12;
        if (pre) cost += 4.0 * static_cast<double>(M) * K / kPrePassBytesPerSecond;  // (the workgroup-tile pre-pass reads A only)
        if (rows_screen) cost += 4.0 * static_cast<double>(K) * N / kPrePassBytesPerSecond;
        const double busy = static_cast<double>(groups < cus ? groups : cus);
        double resident = static_cast<double>(ceil_div(groups > 0 ? groups : 1, cus));
        if (resident > resident_max[c]) resident = resident_max[c];
        const double in_flight = busy * resident * 2.0 * kGemmBK;  // k values of every tile row / column on their way
        const double stream_a = static_cast<double>(M) * K * kTrip / (in_flight * fc.bm);
        const double stream_b = static_cast<double>(N) * K * kTrip / (in_flight * fc.bn);
        const double stream = stream_a > stream_b ? stream_a : stream_b;
        if (stream > cost) cost = stream;
        // (a smaller tile has to promise 2 % to be taken: below that the model cannot tell them apart, and fewer, larger
        // check tiles mean fewer records)
        if (cost < best_cost * 0.98) { best_cost = cost; best = c; }
    }
    return best;
}

// (a workspace of hpcdnn_workspace_bytes(HPCDNN_OP_FT_SGEMM, ...) or more)
extern "C" int hpcdnn_ft_pick_class(int M, int N, int K) { return hpcdnn_ft_pick_class_ws(M, N, K, ~static_cast<size_t>(0)); }

// Fault-free residuals are the FP32 rounding of the accumulators added over a tile line; for operands uniform in
// [-1, 1] their maximum over a whole matrix grows linearly with K (measured 4.0e-7 ... 4.9e-7 per unit of K from
// K = 256 to 65536).  The default leaves a factor of two to that and stays below the 1e-2 faults at K = 4096.
extern "C" float hpcdnn_ft_default_tau(int K) {
    const int k = K > 64 ? K : 64;
    return 1.1e-6f * static_cast<float>(k);
}

extern "C" int hpcdnn_ft_sgemm_opt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                                   float alpha, float beta, float tau, const hpcdnn_ft_options* opt, hpcdnn_ft_status* status,
                                   void* ws, size_t ws_bytes, void* stream) {
    hpcdnn_ft_options none{};
    return run_ft_sgemm(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, tau, opt ? *opt : none, status, ws, ws_bytes,
                        static_cast<hipStream_t>(stream));
}

extern "C" int hpcdnn_ft_sgemm_ex(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                                  float alpha, float beta, float tau, const hpcdnn_fault* inject, hpcdnn_ft_status* status,
                                  void* ws, size_t ws_bytes, int tile_class, void* stream) {
    hpcdnn_ft_options opt{};
    opt.tile_class = tile_class;
    if (inject) {
        opt.n_faults = 1;
        opt.faults[0].tile = inject->tile;
        opt.faults[0].row = inject->row;
        opt.faults[0].col = inject->col;
        opt.faults[0].delta = inject->delta;
        opt.faults[0].check = 0;
    }
    return run_ft_sgemm(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, tau, opt, status, ws, ws_bytes,
                        static_cast<hipStream_t>(stream));
}

extern "C" int hpcdnn_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                               float alpha, float beta, float tau, const hpcdnn_fault* inject, hpcdnn_ft_status* status,
                               void* ws, size_t ws_bytes, void* stream) {
    return hpcdnn_ft_sgemm_ex(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, tau, inject, status, ws, ws_bytes, 0, stream);
}

// ---- ABFT SGEMM on the reference family's own column-major buffers.  Read row by row, column-major
// C = alpha * A * B^T + beta * C is C^T (N x M) = (B^T)^T * A^T with both operands K-major: the row-major problem with
// its left operand, the memory of B seen as K rows of N, given transposed.
namespace hpcdnn {
size_t ft_cm_nt_workspace_bytes(int M, int N, int K) { return ft_workspace_bytes(N, M, K); }
}  // namespace hpcdnn

extern "C" int hpcdnn_ft_sgemm_cm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                                     float alpha, float beta, float tau, const hpcdnn_ft_options* opt, hpcdnn_ft_status* status,
                                     void* ws, size_t ws_bytes, void* stream) {
    hpcdnn_ft_options none{};
    return run_ft_sgemm(N, M, K, B, ldb, A, lda, C, ldc, alpha, beta, tau, opt ? *opt : none, status, ws, ws_bytes,
                        static_cast<hipStream_t>(stream), true);
}

// ---- ABFT SGEMM for callers that can neither allocate nor pass a workspace: the checksum vectors (and, when they
// fit, the K slices of a partial last round) live in a fixed device array of this library.  Every device the
// library runs on holds its own copy of the array at its own address, looked up once per device.
static __device__ __align__(256) unsigned char scratch[HPCDNN_FT_STATIC_SCRATCH_BYTES];

// First call on a device: look the array's address up and let the two kernels the entry point launches (full-tile
// and ragged-tile forms of the 256 x 128 class) use their LDS.  Neither belongs into a stream capture, so a first call
// that finds its stream capturing is refused; any earlier eager call (M = 0 is enough) has done the set-up.
static int static_scratch_address(void** out, hipStream_t stream) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* address[kMaxDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return HPCDNN_ERR_INVALID_VALUE;
    std::lock_guard<std::mutex> lock(mu);
    if (!address[dev]) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        e = hipStreamIsCapturing(stream, &capturing);
        if (e != hipSuccess) return static_cast<int>(e);
        if (capturing != hipStreamCaptureStatusNone) return HPCDNN_ERR_NOT_READY;
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // the address on the current device
        if (e != hipSuccess) return static_cast<int>(e);
        if (!p) return HPCDNN_ERR_WORKSPACE;
        int rc = HPCDNN_OK;
        for (int kind : {kFtPre, kFtFused}) {  // (kFtFused: products one tile wide or high)
            const FtKernel k = ft_kernel(0, false, kind);
            if (rc == HPCDNN_OK) rc = enable_lds(k.plain, k.lds);
            if (rc == HPCDNN_OK) rc = enable_lds(k.edge, k.lds);
        }
        if (rc != HPCDNN_OK) return rc;
        address[dev] = p;
    }
    *out = address[dev];
    return HPCDNN_OK;
}

extern "C" int hpcdnn_ft_sgemm_static(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C,
                                      int ldc, float alpha, float beta, float tau, const hpcdnn_fault* inject,
                                      hpcdnn_ft_status* status, void* stream) {
    int rc = check_gemm_args(M, N, K, A, lda, B, ldb, C, ldc);
    if (rc != HPCDNN_OK) return rc;
    void* ws = nullptr;
    rc = static_scratch_address(&ws, static_cast<hipStream_t>(stream));
    if (rc != HPCDNN_OK) return rc;
    if (M == 0 || N == 0) return HPCDNN_OK;
    // the checksum vectors of the 256 x 128 class must fit; beyond that the call is refused, never silently slower
    if (K > 0 && ft_enc_bytes(kFtClasses[0], HPCDNN_FT_GRAN_TILE, M, N, K) > HPCDNN_FT_STATIC_SCRATCH_BYTES) return HPCDNN_ERR_WORKSPACE;
    // Nothing in the array has to start at zero: the pre-pass rewrites every word of the checksum vectors the GEMM
    // reads (their zero padding included), and the K slices and their records are written before they are read.
    // (a product one tile wide or high runs the kernels that need no pre-pass; their K slices use the array alone)
    return hpcdnn_ft_sgemm_ex(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, tau, inject, status, ws,
                              HPCDNN_FT_STATIC_SCRATCH_BYTES, 0, stream);
}

namespace hpcdnn {
// enough for any tile class at either granularity (the lowest class has the most tile rows)
size_t ft_workspace_bytes(int M, int N, int K) {
    size_t most = 0;
    for (int c = 0; c < HPCDNN_FT_NUM_CLASSES; ++c) {
        const size_t b = ft_class_workspace_bytes(c, M, N, K);
        if (b > most) most = b;
    }
    return most;
}
}  // namespace hpcdnn
