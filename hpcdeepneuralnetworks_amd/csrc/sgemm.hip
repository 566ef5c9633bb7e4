// SGEMM / ABFT-SGEMM entry points: argument checks, tile + split-K choice, launch.
#include "sgemm_kernel.h"
#include "sgemm_small_kernel.h"

#include <mutex>

namespace hpcdnn {

struct TileConfig {
    int bm, bn, bk;
    int threads;
    int blocks_per_cu;  // resident workgroups per CU the kernel is built for (its launch bound)
    size_t lds_bytes;
    void (*plain)(const GemmArgs);
    void (*edge)(const GemmArgs);
    float eff;  // fitted steady-state fraction of the FP32 MFMA peak of one CU
    bool wave_split_k;  // small-problem kernel: the waves of a workgroup split K (other summation order, no tail split)
    int nslot;          // K steps a workgroup keeps on their way from memory (0: not modelled)
};

#define HPCDNN_TILE(BM, BN, WGM, WGN, OCC, EFF)                                                          \
    {                                                                                                    \
        BM, BN, kGemmBK, WGM * WGN * kWave, OCC, gemm_lds_bytes<BM, BN>(),                               \
            sgemm_kernel<BM, BN, WGM, WGN, false, 0, OCC>, sgemm_kernel<BM, BN, WGM, WGN, true, 0, OCC>, EFF, false, 2 \
    }

#define HPCDNN_TILE_DEEP(BM, BN, WGM, WGN, OCC, EFF, NSLOT)                                               \
    {                                                                                                    \
        BM, BN, kGemmBK, WGM * WGN * kWave, OCC, gemm_lds_bytes<BM, BN>(),                               \
            sgemm_kernel<BM, BN, WGM, WGN, false, 0, OCC, NSLOT>, sgemm_kernel<BM, BN, WGM, WGN, true, 0, OCC, NSLOT>, EFF, \
            false, NSLOT                                                                                 \
    }

#define HPCDNN_SMALL_TILE(TMB, OCC, EFF)                                                                  \
    {                                                                                                    \
        32 * TMB, 32, kSmallBK, kSmallThreads, OCC, small_lds_bytes<TMB>(), sgemm_small_kernel<TMB, false, OCC>, \
            sgemm_small_kernel<TMB, true, OCC>, EFF, true, 0                                             \
    }

// The counterpart of the reference's small/medium/large/tall/wide/huge shape table
// (kernel/ft_sgemm/code_gen/main.py:8-16), re-derived for 32x32 MFMA blocks and four or eight 64-lane waves per
// workgroup.  EFF comes from a least-squares fit of plan_cost() below to measured times of every tile over
// squares 256..6144 with K = n, 1024 and 256 and a set of skinny shapes on an MI355X.
static const TileConfig kTiles[] = {
    HPCDNN_TILE(256, 128, 2, 2, 2, 0.978f),  // 0 huge (the ABFT tile)
    HPCDNN_TILE(128, 128, 2, 2, 2, 0.970f),  // 1 large
    HPCDNN_TILE(128, 64, 2, 2, 2, 0.945f),   // 2 tall
    HPCDNN_TILE(64, 128, 2, 2, 2, 0.939f),   // 3 wide
    HPCDNN_TILE(64, 64, 2, 2, 4, 0.900f),    // 4 medium
    HPCDNN_TILE(192, 256, 2, 2, 1, 0.964f),  // 5 6144-friendly: 32 x 24 tiles = 3 full rounds of 256 CUs
    HPCDNN_TILE(256, 192, 2, 2, 1, 0.946f),  // 6
    HPCDNN_TILE(128, 256, 2, 2, 2, 0.987f),  // 7
    HPCDNN_TILE(256, 256, 2, 4, 1, 1.000f),  // 8 giant, eight waves
    HPCDNN_TILE(256, 128, 4, 2, 1, 1.000f),  // 9 huge, eight waves
    HPCDNN_TILE(256, 256, 4, 2, 1, 1.000f),  // 10 giant, eight waves (4 x 2)
    // 11 small: 32 x 32, K split between the four waves.  Every lane fetches its own operands, so the rate is set by
    // the vector memory path, about half the matrix peak: for problems with too few 64 x 64 tiles to go round
    HPCDNN_SMALL_TILE(1, 4, 0.50f),
    // 12 medium with its loads four K steps ahead: a 64-row tile moves 64 bytes per row and K step, and with one
    // workgroup per CU two steps in flight do not cover the trip to HBM when A is long and read once.  Staged data
    // is so old when it is needed that the LDS writes lead the step and are done long before the barrier.
    HPCDNN_TILE_DEEP(64, 64, 2, 2, 4, 0.905f, 4),
    HPCDNN_TILE(192, 192, 2, 2, 1, 0.943f),  // 13 3072-friendly: 16 x 16 tiles = one full round of 256 CUs
};
constexpr int kNumTiles = sizeof(kTiles) / sizeof(kTiles[0]);

// row length of the pre-encoded checksum vectors: K rounded up to the K step, plus two K steps of zeros for the
// fetches that run ahead of the main loop
static int ft_enc_ld(int K) { return (static_cast<int>(ceil_div(K, kGemmBK)) + 2) * kGemmBK; }
size_t ft_workspace_bytes(int M, int N, int K);
// ABFT tile classes (the counterpart of the reference's abft_kernel_{huge,large,wide,...} family,
// kernel/ft_sgemm/sgemm.cu:187-188): class 0 is the 256 x 128 tile of HPCDNN_FT_TILE_M/N; the smaller classes keep
// more CUs busy on smaller problems.  The encode is laid out for 128-column tiles, so the classes differ in height.
//
// Without a workspace (FT = 1) four waves: on this part every VALU instruction takes its issue cycles away from the
// FP32 matrix pipe of the same SIMD, whichever wave it comes from, so more waves do not hide the checksum arithmetic;
// fewer, fatter threads need the fewest VALU instructions per K step.  With the operands' checksum vectors read from
// a workspace (FT = 2) no cross-lane reductions are left in the loop, the thread count no longer changes the VALU
// work per SIMD, and eight waves (two per SIMD) hide each other's barriers and LDS latency: measured 2 % faster.
struct FtClass {
    int bm, bn;
    int threads_fused, threads_pre;
    size_t lds_fused, lds_pre;
    void (*fused_plain)(const GemmArgs);
    void (*fused_edge)(const GemmArgs);
    void (*pre_plain)(const GemmArgs);
    void (*pre_edge)(const GemmArgs);
    void (*encode)(int, int, int, const float*, int, const float*, int, float*, float*, int, int, int);
};

#define HPCDNN_FT_CLASS(BM, FM, FN, PM, PN)                                                                      \
    {                                                                                                            \
        BM, 128, FM * FN * kWave, PM * PN * kWave, gemm_lds_bytes<BM, 128, 1, FM * FN * kWave>(),                \
            gemm_lds_bytes<BM, 128, 2, PM * PN * kWave>(), sgemm_kernel<BM, 128, FM, FN, false, 1, 1>,           \
            sgemm_kernel<BM, 128, FM, FN, true, 1, 1>, sgemm_kernel<BM, 128, PM, PN, false, 2, 1>,               \
            sgemm_kernel<BM, 128, PM, PN, true, 2, 1>, abft_encode_kernel<BM, 128>                               \
    }

static const FtClass kFtClasses[HPCDNN_FT_NUM_CLASSES] = {
    HPCDNN_FT_CLASS(256, 2, 2, 2, 4),  // 0 huge
    HPCDNN_FT_CLASS(128, 2, 2, 2, 2),  // 1 large
    HPCDNN_FT_CLASS(64, 2, 2, 2, 2),   // 2 wide
};

// Kernels that use more than the default 64 KiB of LDS must opt in once per device.
static int enable_lds(void (*fn)(const GemmArgs), size_t bytes) {
    if (bytes <= 64 * 1024) return HPCDNN_OK;
    struct Done {
        const void* fn;
        int device;
    };
    static std::mutex mu;
    static Done done[16 * kNumTiles] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    std::lock_guard<std::mutex> lock(mu);
    const void* key = reinterpret_cast<const void*>(fn);
    for (const Done& d : done)
        if (d.fn == key && d.device == dev) return HPCDNN_OK;
    e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
    if (e != hipSuccess) return static_cast<int>(e);
    for (Done& d : done)
        if (!d.fn) { d = Done{key, dev}; break; }  // a full table only costs a repeated call
    return HPCDNN_OK;
}

struct Plan {
    int tile;
    int split;  // > 1: every tile split this many ways along K; < -1: only the tiles after the last full round of CUs
                // are split (-split ways); 1: no split
};

// Predicted run time in seconds (up to a constant per launch).  Workgroups are dealt evenly to the CUs, so a launch
// takes as long as the CU with the most tiles: n = ceil(tiles / CUs) tile times on its matrix cores (co-resident
// workgroups share them), plus the part of each tile's prologue and epilogue that nothing overlaps: all of it when
// one workgroup owns the CU, a fraction of it (after the first) when co-resident workgroups cover for each other.
// The epilogue grows with the tile's area (C is written at the CU's share of HBM bandwidth).  A four-per-CU tile
// with two staging sets running with fewer co-residents loses efficiency: one wave per SIMD cannot hide its own
// waits (the deep-staging variant writes LDS early enough not to have them).
constexpr double kPeakFlopsPerCu = 157.3e12 / 256.0;
constexpr double kEdgePenalty = 1.03;          // ragged tiles: partly empty tiles are paid in full by tile counting; this is the rest
constexpr double kFixedBase = 2.133e-6;        // prologue + epilogue of a tile: base ...
constexpr double kFixedPer32K = 2.31e-6;       // ... plus this per 32768 elements of tile area
constexpr double kCoveredFraction = 0.209;     // exposed share of the fixed part behind a co-resident workgroup
constexpr double kThinPenalty = 0.12;          // efficiency lost by a small tile when all co-residents are missing
constexpr double kStreamLatency = 0.73e-6;     // trip to HBM under load, fitted on 16384 x 64 x 4096
constexpr double kReduceFixed = 2.5e-6;        // second launch of split-K
constexpr double kReduceBytesPerSec = 8e12;    // partials written once and read once, C written once

static double plan_cost(const TileConfig& t, int M, int N, int K, int split, int cus) {
    const double tiles = static_cast<double>(ceil_div(M, t.bm)) * ceil_div(N, t.bn) * split;
    const double n = ceil(tiles / cus);
    const double k_slice = ceil(static_cast<double>(ceil_div(K, split)) / t.bk) * t.bk;
    const bool edge = (M % t.bm) || (N % t.bn) || (K % t.bk);
    double eff = t.eff;
    const double resident = t.blocks_per_cu < n ? t.blocks_per_cu : n;
    // tiles whose waves own one or two 32x32 blocks (two staging sets): alone on a SIMD a wave cannot hide its waits
    if (t.bm * t.bn <= 128 * 64 && t.nslot == 2) eff *= 1.0 - kThinPenalty * (t.blocks_per_cu - resident) / t.blocks_per_cu;
    // (the ragged-tile variant of a deep-staging kernel runs more masked steps at the end of the slice)
    const double edge_cost = edge ? kEdgePenalty * (t.nslot > 2 ? 1.06 : 1.0) : 1.0;
    const double per_tile = 2.0 * t.bm * t.bn * k_slice / (kPeakFlopsPerCu * eff) * edge_cost;
    const double fixed = kFixedBase + kFixedPer32K * t.bm * t.bn / 32768.0;
    const double exposed = t.blocks_per_cu == 1 ? n : 1.0 + kCoveredFraction * (n - 1.0);
    double cost = n * per_tile + exposed * fixed;
    if (t.nslot > 0) {
        // An operand read once from HBM cannot arrive faster than the bytes in flight allow: per busy CU, resident
        // workgroups x staged K steps x one K step of the tile's rows (A) or columns (B), per trip to memory
        const double busy = tiles < cus ? tiles : cus;
        const double steps_in_flight = busy * resident * t.nslot;
        const double stream_a = static_cast<double>(M) * K * kStreamLatency / (steps_in_flight * t.bm * t.bk);
        const double stream_b = static_cast<double>(N) * K * kStreamLatency / (steps_in_flight * t.bn * t.bk);
        const double stream = (stream_a > stream_b ? stream_a : stream_b) + fixed;
        if (stream > cost) cost = stream;
    }
    if (split > 1) cost += kReduceFixed + (2.0 * split + 1.0) * M * static_cast<double>(N) * 4.0 / kReduceBytesPerSec;
    return cost;
}

// Tail split: with T tiles on `cus` CUs the last T % cus tiles keep only some CUs busy for a whole tile time.
// Splitting just those tiles s ways along K turns that round into ceil(r*s/cus) rounds of 1/s tile time each, at the
// price of writing and re-reading r*s raw tiles.  Returns the cost, and the chosen s through *ways (0 = no gain).
static double tail_plan_cost(const TileConfig& t, int M, int N, int K, int cus, size_t ws_bytes, int* ways) {
    *ways = 0;
    const int64_t tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
    const int64_t r = tiles % cus, full = tiles - r;
    if (full == 0 || r == 0 || 2 * r > cus) return 1e300;
    int64_t s = cus / r;
    const int64_t most = K / (8 * t.bk);  // at least 8 K steps per slice
    if (s > most) s = most;
    if (s > 16) s = 16;
    const size_t tile_bytes = static_cast<size_t>(t.bm) * t.bn * sizeof(float);
    while (s >= 2 && static_cast<size_t>(r * s) * tile_bytes > ws_bytes) --s;
    if (s < 2) return 1e300;
    const bool edge = (M % t.bm) || (N % t.bn) || (K % t.bk);
    const double per_tile = 2.0 * t.bm * t.bn * K / (kPeakFlopsPerCu * t.eff) * (edge ? kEdgePenalty : 1.0);
    const double n_full = static_cast<double>(full / cus);
    const double fixed = kFixedBase + kFixedPer32K * t.bm * t.bn / 32768.0;
    const double n = n_full + 1.0;
    const double exposed = t.blocks_per_cu == 1 ? n : 1.0 + kCoveredFraction * (n - 1.0);
    *ways = static_cast<int>(s);
    return n_full * per_tile + ceil(static_cast<double>(r * s) / cus) * per_tile / s + exposed * fixed + kReduceFixed +
           (2.0 * s + 1.0) * r * static_cast<double>(tile_bytes) / kReduceBytesPerSec;
}

static Plan choose_plan(int M, int N, int K, bool allow_split, size_t ws_bytes, bool allow_tail = true,
                        double* cost_out = nullptr, bool same_bits_only = false) {
    const int cus = device_cus();
    struct Candidate {
        Plan plan;
        double cost;
    };
    Candidate cand[kNumTiles * 8];
    int n_cand = 0;
    double best_cost = 1e300;
    for (int t = 0; t < kNumTiles; ++t) {
        const TileConfig& cfg = kTiles[t];
        if (cfg.eff <= 0.f || (same_bits_only && cfg.wave_split_k)) continue;
        for (int split = 1; split <= 64; split *= 2) {
            if (split > 1) {
                if (!allow_split) break;
                if (ceil_div(K, split) < 8 * cfg.bk) break;
                if (static_cast<size_t>(M) * N * split * sizeof(float) > ws_bytes) break;
            }
            const double c = plan_cost(cfg, M, N, K, split, cus);
            cand[n_cand++] = Candidate{Plan{t, split}, c};
            if (c < best_cost) best_cost = c;
        }
        if (allow_split && allow_tail && !cfg.wave_split_k) {
            int ways = 0;
            const double c = tail_plan_cost(cfg, M, N, K, cus, ws_bytes, &ways);
            if (ways >= 2) {
                cand[n_cand++] = Candidate{Plan{t, -ways}, c};
                if (c < best_cost) best_cost = c;
            }
        }
    }
    // A split has to promise more than the model's error on it (measured: predicted gains below 2-3 % turned out
    // as losses of about 1 %): if some unsplit plan is within 2.5 % of the best, only unsplit plans compete.
    double best_unsplit = 1e300;
    for (int i = 0; i < n_cand; ++i)
        if (cand[i].plan.split == 1 && cand[i].cost < best_unsplit) best_unsplit = cand[i].cost;
    if (best_unsplit <= best_cost * 1.025) {
        best_cost = best_unsplit;
        int kept = 0;
        for (int i = 0; i < n_cand; ++i)
            if (cand[i].plan.split == 1) cand[kept++] = cand[i];
        n_cand = kept;
    }
    // Among plans the model cannot tell apart (within 1 %), take the one that moves the least data: no split
    // before a split, then the larger tile (A and B are re-read once per tile column / tile row).
    Plan best{0, 1};
    bool have = false;
    double best_area = 0.0, best_c = 0.0;
    for (int i = 0; i < n_cand; ++i) {
        if (cand[i].cost > best_cost * 1.01) continue;
        const TileConfig& cfg = kTiles[cand[i].plan.tile];
        const double area = static_cast<double>(cfg.bm) * cfg.bn;
        const bool unsplit = cand[i].plan.split == 1, best_unsplit = best.split == 1;
        const bool better = !have || (unsplit != best_unsplit ? unsplit
                                      : area != best_area     ? area > best_area
                                                              : cand[i].cost < best_c);
        if (better) {
            have = true;
            best = cand[i].plan;
            best_area = area;
            best_c = cand[i].cost;
            if (cost_out) *cost_out = cand[i].cost;
        }
    }
    return best;
}

// Row split, the workspace-free answer to a partial last round: the first rows1 rows of C (whole rounds of big tiles)
// go to one launch, the remaining rows to a second launch with whatever tile suits that thin strip.  Every element
// of C still comes from one workgroup that walks all of K, so the result has the same bits as a single launch.
struct RowSplit {
    int tile1, rows1, tile2;
    double cost;
};
constexpr double kSecondLaunch = 3e-6;

static RowSplit choose_row_split(int M, int N, int K, int cus) {
    RowSplit best{-1, 0, -1, 1e300};
    for (int t = 0; t < kNumTiles; ++t) {
        const TileConfig& cfg = kTiles[t];
        if (cfg.eff <= 0.f || cfg.wave_split_k) continue;
        const int64_t tiles_n = ceil_div(N, cfg.bn), tiles_m = ceil_div(M, cfg.bm);
        const int64_t rounds = tiles_m * tiles_n / cus;
        for (int64_t k = rounds; k >= 1 && k + 1 >= rounds; --k) {
            const int64_t tile_rows = k * cus / tiles_n;
            const int64_t rows1 = tile_rows * cfg.bm;
            if (tile_rows < 1 || rows1 >= M) continue;
            const double c1 = plan_cost(cfg, static_cast<int>(rows1), N, K, 1, cus);
            double c2 = 0.0;
            const Plan rest = choose_plan(M - static_cast<int>(rows1), N, K, false, 0, false, &c2, true);
            const double c = c1 + c2 + kSecondLaunch;
            if (c < best.cost) best = RowSplit{t, static_cast<int>(rows1), rest.tile, c};
        }
    }
    return best;
}

constexpr int kMaxLda = (1 << 21) - 64;   // 256 * lda * 4 < 2^31
constexpr int kMaxLdb = (1 << 25) - 1024;  // 16 * ldb * 4 + row < 2^31

static int check_gemm_args(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc) {
    if (M < 0 || N < 0 || K < 0) return HPCDNN_ERR_INVALID_VALUE;
    if (lda < (K > 1 ? K : 1) || ldb < (N > 1 ? N : 1) || ldc < (N > 1 ? N : 1)) return HPCDNN_ERR_INVALID_VALUE;
    if (M > 0 && N > 0 && !C) return HPCDNN_ERR_INVALID_VALUE;
    if (M > 0 && N > 0 && K > 0 && (!A || !B)) return HPCDNN_ERR_INVALID_VALUE;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C)) & 3u)
        return HPCDNN_ERR_INVALID_VALUE;
    // byte offsets inside one tile are 32-bit: 256 rows of A, 16 rows of B
    if (lda > kMaxLda || ldb > kMaxLdb) return HPCDNN_ERR_INVALID_VALUE;
    return HPCDNN_OK;
}

static GemmArgs make_args(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                          float alpha, float beta, const TileConfig& cfg) {
    GemmArgs a{};
    a.M = M; a.N = N; a.K = K;
    a.A = A; a.lda = lda; a.B = B; a.ldb = ldb; a.C = C; a.ldc = ldc;
    a.alpha = alpha; a.beta = beta;
    a.tiles_m = static_cast<int>(ceil_div(M, cfg.bm));
    a.tiles_n = static_cast<int>(ceil_div(N, cfg.bn));
    a.k_chunk = static_cast<int>(ceil_div(K > 0 ? K : 1, cfg.bk)) * cfg.bk;
    a.partial = nullptr;
    a.fault_tile = -1;
    return a;
}

// The ragged-tile kernel masks the K tail and the columns past N; full tiles with K a multiple of the K step
// (per slice, which k_chunk guarantees for all but the last) skip that work.
static bool needs_edge(const GemmArgs& a, const TileConfig& cfg) {
    return !(a.M % cfg.bm == 0 && a.N % cfg.bn == 0 && a.K % cfg.bk == 0);
}

static int run_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                     float alpha, float beta, void* ws, size_t ws_bytes, int tile, int split, hipStream_t stream) {
    int rc = check_gemm_args(M, N, K, A, lda, B, ldb, C, ldc);
    if (rc != HPCDNN_OK) return rc;
    if (tile >= kNumTiles || split == -1) return HPCDNN_ERR_INVALID_VALUE;
    if (tile >= 0 && kTiles[tile].wave_split_k && split < -1) return HPCDNN_ERR_INVALID_VALUE;
    if (M == 0 || N == 0) return HPCDNN_OK;

    if (tile < 0 || split == 0) {
        // The decision is a function of the shape and of what the workspace allows; callers tend to repeat shapes,
        // so each thread remembers its last one instead of re-evaluating the cost model on every call.
        struct Decision {
            int M, N, K, cus;
            size_t ws_bytes;
            bool ws_aligned, valid;
            Plan plan;
            RowSplit rows;
        };
        static thread_local Decision memo{};
        // the tail split moves 16-byte groups through the workspace
        const bool ws_aligned = (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
        const size_t usable = ws ? ws_bytes : 0;
        const int cus = device_cus();  // of the current device: the plan depends on it
        if (!(memo.valid && memo.M == M && memo.N == N && memo.K == K && memo.cus == cus && memo.ws_bytes == usable &&
              memo.ws_aligned == ws_aligned)) {
            double cost = 0.0;
            memo.plan = choose_plan(M, N, K, ws != nullptr, usable, ws_aligned, &cost);
            memo.rows = RowSplit{-1, 0, -1, 1e300};
            if (K > 0) {
                const RowSplit rs = choose_row_split(M, N, K, cus);
                if (rs.tile1 >= 0 && rs.cost < 0.97 * cost) memo.rows = rs;
            }
            memo.M = M; memo.N = N; memo.K = K; memo.cus = cus;
            memo.ws_bytes = usable;
            memo.ws_aligned = ws_aligned;
            memo.valid = true;
        }
        Plan plan = memo.plan;
        // a forced tail split needs a tile that has one (not the 32 x 32 tile, whose waves split K among themselves)
        if (tile < 0 && split < -1) plan = choose_plan(M, N, K, false, 0, false, nullptr, true);
        const RowSplit rs = memo.rows;  // copied: the nested calls below do not touch the memo, but keep it simple
        if (tile < 0 && split == 0 && rs.tile1 >= 0) {
            rc = run_sgemm(rs.rows1, N, K, A, lda, B, ldb, C, ldc, alpha, beta, nullptr, 0, rs.tile1, 1, stream);
            if (rc != HPCDNN_OK) return rc;
            return run_sgemm(M - rs.rows1, N, K, A + static_cast<int64_t>(rs.rows1) * lda, lda, B, ldb,
                             C + static_cast<int64_t>(rs.rows1) * ldc, ldc, alpha, beta, nullptr, 0, rs.tile2, 1, stream);
        }
        if (tile < 0) {
            tile = plan.tile;
            if (split == 0) split = plan.split;
        } else if (split == 0) {
            split = 1;
        }
    }
    const TileConfig& cfg = kTiles[tile];
    if (cfg.wave_split_k && split < -1) return HPCDNN_ERR_INVALID_VALUE;  // whichever way the tile was chosen
    GemmArgs a = make_args(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, cfg);
    const int tiles = a.tiles_m * a.tiles_n;
    a.full_tiles = tiles;
    a.tail_split = 1;
    int tail_tiles = 0;
    if (split < -1) {
        // tail split: the tiles after the last full round of CUs, -split ways (fewer if K is short)
        const int cus = device_cus();
        tail_tiles = tiles % cus;
        int ways = -split;
        a.tail_k_chunk = static_cast<int>(ceil_div(ceil_div(K, ways), cfg.bk)) * cfg.bk;
        ways = K > 0 ? static_cast<int>(ceil_div(K, a.tail_k_chunk)) : 1;  // drop empty slices
        if (tail_tiles == 0 || tail_tiles == tiles || ways < 2) {
            tail_tiles = 0;  // nothing to gain: plain launch
        } else {
            const size_t need = static_cast<size_t>(tail_tiles) * ways * cfg.bm * cfg.bn * sizeof(float);
            if (!ws || need > ws_bytes) return HPCDNN_ERR_WORKSPACE;
            if (reinterpret_cast<uintptr_t>(ws) & 15u) return HPCDNN_ERR_INVALID_VALUE;
            a.full_tiles = tiles - tail_tiles;
            a.tail_split = ways;
            a.tail_partial = static_cast<float*>(ws);
        }
        split = 1;
    }
    if (split > 1) {
        if (!ws || static_cast<size_t>(M) * N * split * sizeof(float) > ws_bytes) return HPCDNN_ERR_WORKSPACE;
        if (reinterpret_cast<uintptr_t>(ws) & 3u) return HPCDNN_ERR_INVALID_VALUE;
        a.k_chunk = static_cast<int>(ceil_div(ceil_div(K, split), cfg.bk)) * cfg.bk;
        split = static_cast<int>(ceil_div(K, a.k_chunk));  // drop empty slices
        if (split > 1) a.partial = static_cast<float*>(ws);
    }
    const bool edge = needs_edge(a, cfg);
    void (*fn)(const GemmArgs) = edge ? cfg.edge : cfg.plain;
    rc = enable_lds(fn, cfg.lds_bytes);
    if (rc != HPCDNN_OK) return rc;

    dim3 grid(a.full_tiles + tail_tiles * a.tail_split, 1, split);
    hipLaunchKernelGGL(fn, grid, dim3(cfg.threads), cfg.lds_bytes, stream, a);
    rc = launch_status();
    if (rc != HPCDNN_OK) return rc;
    if (tail_tiles > 0) {
        tail_reduce_kernel<<<dim3(tail_tiles, cfg.bm / 32), 256, 0, stream>>>(M, N, cfg.bm, cfg.bn, a.tiles_m, a.tiles_n,
                                                                             a.full_tiles, a.tail_split, a.tail_partial, C,
                                                                             ldc, alpha, beta);
        return launch_status();
    }
    if (split == 1) return rc;

    const int64_t total = static_cast<int64_t>(M) * N;
    int rgrid = static_cast<int>(ceil_div(total, 256));
    const int cap = device_cus() * 8;
    if (rgrid > cap) rgrid = cap;
    splitk_reduce_kernel<<<rgrid, 256, 0, stream>>>(M, N, split, static_cast<const float*>(ws), C, ldc, alpha, beta);
    return launch_status();
}

}  // namespace hpcdnn

using namespace hpcdnn;

extern "C" int hpcdnn_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                            float alpha, float beta, void* ws, size_t ws_bytes, void* stream) {
    return run_sgemm(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, ws, ws_bytes, -1, 0, static_cast<hipStream_t>(stream));
}

extern "C" int hpcdnn_sgemm_ex(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                               float alpha, float beta, void* ws, size_t ws_bytes, int tile, int split_k, void* stream) {
    return run_sgemm(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, ws, ws_bytes, tile, split_k,
                     static_cast<hipStream_t>(stream));
}

extern "C" int hpcdnn_sgemm_num_tiles(void) { return kNumTiles; }

extern "C" int hpcdnn_sgemm_tile_info(int tile, int* bm, int* bn, int* bk) {
    if (tile < 0 || tile >= kNumTiles) return HPCDNN_ERR_INVALID_VALUE;
    if (bm) *bm = kTiles[tile].bm;
    if (bn) *bn = kTiles[tile].bn;
    if (bk) *bk = kTiles[tile].bk;
    return HPCDNN_OK;
}

extern "C" int hpcdnn_sgemm_plan(int M, int N, int K, size_t ws_bytes, int* tile, int* split_k) {
    if (M < 0 || N < 0 || K < 0) return HPCDNN_ERR_INVALID_VALUE;
    const Plan plan = choose_plan(M, N, K, ws_bytes > 0, ws_bytes);
    if (tile) *tile = plan.tile;
    if (split_k) *split_k = plan.split;
    return HPCDNN_OK;
}

extern "C" int hpcdnn_sgemm_row_split(int M, int N, int K, size_t ws_bytes, int* rows_first, int* tile_first,
                                      int* tile_rest) {
    if (M < 0 || N < 0 || K < 0) return HPCDNN_ERR_INVALID_VALUE;
    int rows = 0, t1 = -1, t2 = -1;
    if (M > 0 && N > 0 && K > 0) {
        double cost = 0.0;
        choose_plan(M, N, K, ws_bytes > 0, ws_bytes, true, &cost);
        const RowSplit rs = choose_row_split(M, N, K, device_cus());
        if (rs.tile1 >= 0 && rs.cost < 0.97 * cost) { rows = rs.rows1; t1 = rs.tile1; t2 = rs.tile2; }
    }
    if (rows_first) *rows_first = rows;
    if (tile_first) *tile_first = t1;
    if (tile_rest) *tile_rest = t2;
    return HPCDNN_OK;
}

extern "C" int hpcdnn_ft_tile_info(int tile_class, int* bm, int* bn) {
    if (tile_class < 0 || tile_class >= HPCDNN_FT_NUM_CLASSES) return HPCDNN_ERR_INVALID_VALUE;
    if (bm) *bm = kFtClasses[tile_class].bm;
    if (bn) *bn = kFtClasses[tile_class].bn;
    return HPCDNN_OK;
}

extern "C" int hpcdnn_ft_num_tiles_ex(int tile_class, int M, int N) {
    if (M < 0 || N < 0 || tile_class < 0 || tile_class >= HPCDNN_FT_NUM_CLASSES) return 0;
    return static_cast<int>(ceil_div(M, kFtClasses[tile_class].bm) * ceil_div(N, kFtClasses[tile_class].bn));
}

extern "C" int hpcdnn_ft_num_tiles(int M, int N) { return hpcdnn_ft_num_tiles_ex(0, M, N); }

// ABFT with a workspace splits the tiles of a partial last round of CUs along K, like plain SGEMM's tail split: every
// slice is a workgroup that verifies (and corrects) its own partial product - the checksums are linear in K - and
// writes it raw; tail_reduce_kernel adds the slices, ft_tail_status_kernel merges their records.  With fewer tiles
// than half the CUs every tile is split.  Returns the number of ways (1: no split) and the tiles it applies to.
struct FtTail {
    int ways, tiles;
};
static FtTail ft_tail_plan(const FtClass& fc, int M, int N, int K) {
    const int cus = device_cus();
    const int64_t tiles = ceil_div(M, fc.bm) * ceil_div(N, fc.bn);
    const int64_t r = tiles % cus;
    if (r == 0 || 2 * r > cus) return FtTail{1, 0};
    int64_t s = cus / r;
    const int64_t most = K / (16 * kGemmBK);  // at least 16 K steps per slice: each slice pays a verification
    if (s > most) s = most;
    if (s > 8) s = 8;
    if (s < 2) return FtTail{1, 0};
    return FtTail{static_cast<int>(s), static_cast<int>(r)};
}
static size_t ft_enc_bytes(const FtClass& fc, int M, int N, int K) {
    const size_t b = static_cast<size_t>(ceil_div(M, fc.bm) + ceil_div(N, fc.bn)) * ft_enc_ld(K) * sizeof(float);
    return (b + 15) & ~static_cast<size_t>(15);
}
static size_t ft_tail_bytes(const FtClass& fc, const FtTail& t) {
    return t.ways < 2 ? 0
                      : static_cast<size_t>(t.tiles) * t.ways * (static_cast<size_t>(fc.bm) * fc.bn * sizeof(float) + sizeof(hpcdnn_ft_status));
}

// The class with the shortest predicted run (workspace variant): rounds of tiles over the CUs times the tile height
// (all classes are 128 columns wide), a partial last round counting for what its K split leaves of it plus the
// second pass over those tiles, with the measured efficiency of the smaller tiles relative to the 256-row one.
extern "C" int hpcdnn_ft_pick_class(int M, int N, int K) {
    // measured on squares 1024 ... 6144: the 128-row class keeps up with the 256-row one (two of its workgroups share a CU
    // and cover each other's verification), the 64-row class runs 4-5 % behind
    static const double rel_eff[HPCDNN_FT_NUM_CLASSES] = {1.0, 1.0, 0.955};
    const int cus = device_cus();
    int best = 0;
    double best_cost = 1e300;
    for (int c = 0; c < HPCDNN_FT_NUM_CLASSES; ++c) {
        const int64_t tiles = hpcdnn_ft_num_tiles_ex(c, M, N);
        const FtTail tail = ft_tail_plan(kFtClasses[c], M, N, K);
        double rounds = static_cast<double>(ceil_div(tiles > 0 ? tiles : 1, cus));
        if (tail.ways >= 2)
            rounds = static_cast<double>(tiles / cus) + static_cast<double>(ceil_div(static_cast<int64_t>(tail.tiles) * tail.ways, cus)) / tail.ways + 0.06;
        const double cost = rounds * kFtClasses[c].bm / rel_eff[c];
        if (cost < best_cost) { best_cost = cost; best = c; }
    }
    return best;
}

// Fault-free residuals are the FP32 rounding of the accumulators added over a tile line; for operands uniform in
// [-1, 1] their maximum over a whole matrix grows linearly with K (measured 4.0e-7 ... 4.9e-7 per unit of K from
// K = 256 to 65536).  The default leaves a factor of two to that and stays below the 1e-2 faults at K = 4096.
extern "C" float hpcdnn_ft_default_tau(int K) {
    const int k = K > 64 ? K : 64;
    return 1.1e-6f * static_cast<float>(k);
}

static size_t ft_class_workspace_bytes(int tile_class, int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const FtClass& fc = kFtClasses[tile_class];
    return ft_enc_bytes(fc, M, N, K) + ft_tail_bytes(fc, ft_tail_plan(fc, M, N, K));
}

extern "C" int hpcdnn_ft_sgemm_ex(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                                  float alpha, float beta, float tau, const hpcdnn_fault* inject, hpcdnn_ft_status* status,
                                  void* ws, size_t ws_bytes, int tile_class, void* stream) {
    int rc = check_gemm_args(M, N, K, A, lda, B, ldb, C, ldc);
    if (rc != HPCDNN_OK) return rc;
    if (tile_class < 0 || tile_class >= HPCDNN_FT_NUM_CLASSES) return HPCDNN_ERR_INVALID_VALUE;
    if (M == 0 || N == 0) return HPCDNN_OK;
    const FtClass& fc = kFtClasses[tile_class];
    TileConfig cfg{};
    cfg.bm = fc.bm;
    cfg.bn = fc.bn;
    cfg.bk = kGemmBK;
    GemmArgs a = make_args(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, cfg);
    // tau > 0: absolute; tau == 0: the absolute default for unit-range data; tau < 0: scaled to the data, the
    // threshold of a line of n elements being -tau * 4.3 FP32 rounding units * sqrt(max(K, 64)) * sqrt(n) * the larger
    // of the line's and the tile's mean |accumulator|
    a.tau = (tau > 0.f) ? tau : (tau == 0.f ? hpcdnn_ft_default_tau(K) : 0.f);
    a.tau_rel = (tau < 0.f) ? -tau * 2.56e-7f * sqrtf(static_cast<float>(K > 64 ? K : 64)) : 0.f;
    a.status = status;
    if (inject) {
        if (inject->tile < 0 || inject->tile >= a.tiles_m * a.tiles_n || inject->row < 0 || inject->row >= fc.bm ||
            inject->col < 0 || inject->col >= fc.bn)
            return HPCDNN_ERR_INVALID_VALUE;
        a.fault_tile = inject->tile;
        a.fault_row = inject->row;
        a.fault_col = inject->col;
        a.fault_delta = inject->delta;
    }
    const bool edge = needs_edge(a, cfg);
    hipStream_t s = static_cast<hipStream_t>(stream);
    dim3 grid(a.tiles_m * a.tiles_n, 1, 1);
    // With a workspace the checksum vectors of A and B are formed once per tile row / tile column by a small
    // bandwidth-bound kernel and the main loop only reads them; without one every workgroup forms them itself.
    if (ws && K > 0) {
        const size_t enc_bytes = ft_enc_bytes(fc, M, N, K);
        if (ws_bytes < enc_bytes || (reinterpret_cast<uintptr_t>(ws) & 15u)) return HPCDNN_ERR_WORKSPACE;
        // the K split of a partial last round is taken when the workspace has room for it
        FtTail tail = ft_tail_plan(fc, M, N, K);
        if (ws_bytes < enc_bytes + ft_tail_bytes(fc, tail)) tail = FtTail{1, 0};
        a.enc_ld = ft_enc_ld(K);
        float* enc_a = static_cast<float*>(ws);
        float* enc_b = enc_a + static_cast<size_t>(a.tiles_m) * a.enc_ld;
        a.enc_a = enc_a;
        a.enc_b = enc_b;
        const int k_blocks = static_cast<int>(ceil_div(a.enc_ld, 256));
        hipLaunchKernelGGL(fc.encode, dim3(k_blocks * (a.tiles_m + a.tiles_n)), dim3(1024), 0, s, M, N, K, A, lda, B, ldb,
                           enc_a, enc_b, a.enc_ld, k_blocks, a.tiles_m);
        rc = launch_status();
        if (rc != HPCDNN_OK) return rc;
        void (*fn)(const GemmArgs) = edge ? fc.pre_edge : fc.pre_plain;
        rc = enable_lds(fn, fc.lds_pre);
        if (rc != HPCDNN_OK) return rc;
        const int tiles = a.tiles_m * a.tiles_n;
        a.full_tiles = tiles;
        a.tail_split = 1;
        if (tail.ways >= 2) {
            a.tail_k_chunk = static_cast<int>(ceil_div(ceil_div(K, tail.ways), kGemmBK)) * kGemmBK;
            tail.ways = static_cast<int>(ceil_div(K, a.tail_k_chunk));  // drop empty slices
        }
        if (tail.ways >= 2) {
            a.full_tiles = tiles - tail.tiles;
            a.tail_split = tail.ways;
            a.tail_partial = reinterpret_cast<float*>(static_cast<char*>(ws) + enc_bytes);
            a.tail_status = reinterpret_cast<hpcdnn_ft_status*>(a.tail_partial + static_cast<size_t>(tail.tiles) * tail.ways * fc.bm * fc.bn);
            grid = dim3(a.full_tiles + tail.tiles * tail.ways, 1, 1);
        }
        hipLaunchKernelGGL(fn, grid, dim3(fc.threads_pre), fc.lds_pre, s, a);
        rc = launch_status();
        if (rc != HPCDNN_OK || a.tail_split < 2) return rc;
        tail_reduce_kernel<<<dim3(tail.tiles, fc.bm / 32), 256, 0, s>>>(M, N, fc.bm, fc.bn, a.tiles_m, a.tiles_n, a.full_tiles,
                                                                       a.tail_split, a.tail_partial, C, ldc, alpha, beta);
        rc = launch_status();
        if (rc != HPCDNN_OK || !status) return rc;
        ft_tail_status_kernel<<<static_cast<int>(ceil_div(tail.tiles, 64)), 64, 0, s>>>(tail.tiles, a.tail_split, a.tiles_m, a.tiles_n,
                                                                                      a.full_tiles, a.tail_status, status);
        return launch_status();
    }
    void (*fn)(const GemmArgs) = edge ? fc.fused_edge : fc.fused_plain;
    rc = enable_lds(fn, fc.lds_fused);
    if (rc != HPCDNN_OK) return rc;
    hipLaunchKernelGGL(fn, grid, dim3(fc.threads_fused), fc.lds_fused, s, a);
    return launch_status();
}

extern "C" int hpcdnn_ft_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                               float alpha, float beta, float tau, const hpcdnn_fault* inject, hpcdnn_ft_status* status,
                               void* ws, size_t ws_bytes, void* stream) {
    return hpcdnn_ft_sgemm_ex(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, tau, inject, status, ws, ws_bytes, 0, stream);
}

// ---- ABFT SGEMM for callers that can neither allocate nor pass a workspace: the checksum vectors (and, when they
// fit, the K slices of a partial last round) live in a fixed device array of this library.  Every device the
// library runs on holds its own copy of the array at its own address, looked up once per device.
static __device__ __align__(256) unsigned char scratch[HPCDNN_FT_STATIC_SCRATCH_BYTES];

static int static_scratch_address(void** out) {
    constexpr int kMaxDevices = 64;
    static std::mutex mu;
    static void* address[kMaxDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    if (dev < 0 || dev >= kMaxDevices) return HPCDNN_ERR_INVALID_VALUE;
    std::lock_guard<std::mutex> lock(mu);
    if (!address[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));  // the address on the current device
        if (e != hipSuccess) return static_cast<int>(e);
        if (!p) return HPCDNN_ERR_WORKSPACE;
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
    if (M == 0 || N == 0) return HPCDNN_OK;
    // the checksum vectors of the 256 x 128 class must fit; beyond that the call is refused, never silently slower
    if (K > 0 && ft_enc_bytes(kFtClasses[0], M, N, K) > HPCDNN_FT_STATIC_SCRATCH_BYTES) return HPCDNN_ERR_WORKSPACE;
    void* ws = nullptr;
    rc = static_scratch_address(&ws);
    if (rc != HPCDNN_OK) return rc;
    // Nothing in the array has to start at zero: the pre-pass rewrites every word of the checksum vectors the GEMM
    // reads (their zero padding included), and the K slices and their records are written before they are read.
    return hpcdnn_ft_sgemm_ex(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, tau, inject, status, ws,
                              HPCDNN_FT_STATIC_SCRATCH_BYTES, 0, stream);
}

namespace hpcdnn {
// enough for any tile class (the lowest class has the most tile rows)
size_t ft_workspace_bytes(int M, int N, int K) {
    size_t most = 0;
    for (int c = 0; c < HPCDNN_FT_NUM_CLASSES; ++c) {
        const size_t b = ft_class_workspace_bytes(c, M, N, K);
        if (b > most) most = b;
    }
    return most;
}
size_t sgemm_workspace_bytes(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    const Plan plan = choose_plan(M, N, K, true, static_cast<size_t>(-1));
    if (plan.split > 1) return static_cast<size_t>(M) * N * plan.split * sizeof(float);
    if (plan.split < -1) {
        const TileConfig& cfg = kTiles[plan.tile];
        const int64_t tail = (ceil_div(M, cfg.bm) * ceil_div(N, cfg.bn)) % device_cus();
        return static_cast<size_t>(tail) * (-plan.split) * cfg.bm * cfg.bn * sizeof(float);
    }
    return 0;
}
}  // namespace hpcdnn
