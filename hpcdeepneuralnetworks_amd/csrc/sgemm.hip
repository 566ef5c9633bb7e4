// SGEMM / ABFT-SGEMM entry points: argument checks, tile + split-K choice, launch.
#include "gemm_host.h"
#include "sgemm_small_kernel.h"
#include "sgemm_persistent_kernel.h"
#include "sgemm_tiles.h"

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
    // persistent variants for several rounds of whole tiles (beta == 0, beta != 0), or nullptr
    void (*persistent)(const GemmArgs);
    void (*persistent_beta)(const GemmArgs);
    int persistent_per_cu;  // workgroups of the persistent kernel per CU
};

#define HPCDNN_TILE_(BM, BN, WGM, WGN, OCC, EFF, PERSISTENT, PERSISTENT_BETA, PER_CU)                                                        \
    {                                                                                                    \
        BM, BN, kGemmBK, WGM * WGN * kWave, OCC, gemm_lds_bytes<BM, BN>(),                               \
            sgemm_kernel<BM, BN, WGM, WGN, false, 0, OCC>, sgemm_kernel<BM, BN, WGM, WGN, true, 0, OCC>, EFF, false, 2, \
            PERSISTENT, PERSISTENT_BETA, PER_CU                                                                        \
    }

#define HPCDNN_TILE(BM, BN, WGM, WGN, OCC, EFF) HPCDNN_TILE_(BM, BN, WGM, WGN, OCC, EFF, nullptr, nullptr, 1)
#define HPCDNN_TILE_PERSISTENT(BM, BN, WGM, WGN, OCC, EFF) \
    HPCDNN_TILE_(BM, BN, WGM, WGN, OCC, EFF, (sgemm_persistent_kernel<BM, BN, WGM, WGN, false>),       \
                 (sgemm_persistent_kernel<BM, BN, WGM, WGN, true>), 1)
// (the 128 x 128 tile: 64 accumulators per lane, two persistent workgroups per CU)
#define HPCDNN_TILE_PERSISTENT_TWO(BM, BN, WGM, WGN, OCC, EFF) \
    HPCDNN_TILE_(BM, BN, WGM, WGN, OCC, EFF, (sgemm_persistent_kernel<BM, BN, WGM, WGN, false, 0, 2>),  \
                 (sgemm_persistent_kernel<BM, BN, WGM, WGN, true, 0, 2>), 2)

// (192 accumulators per lane: 64 of a finished tile's stores go out at the tile boundary, no beta != 0 variant)
#define HPCDNN_TILE_PERSISTENT_BIG(BM, BN, WGM, WGN, OCC, EFF) \
    HPCDNN_TILE_(BM, BN, WGM, WGN, OCC, EFF, (sgemm_persistent_kernel<BM, BN, WGM, WGN, false, 64>), nullptr, 1)

#define HPCDNN_TILE_DEEP(BM, BN, WGM, WGN, OCC, EFF, NSLOT)                                               \
    {                                                                                                    \
        BM, BN, kGemmBK, WGM * WGN * kWave, OCC, gemm_lds_bytes<BM, BN>(),                               \
            sgemm_kernel<BM, BN, WGM, WGN, false, 0, OCC, NSLOT>, sgemm_kernel<BM, BN, WGM, WGN, true, 0, OCC, NSLOT>, EFF, \
            false, NSLOT, nullptr, nullptr, 1                                                             \
    }

#define HPCDNN_SMALL_TILE(TMB, OCC, EFF)                                                                  \
    {                                                                                                    \
        32 * TMB, 32, kSmallBK, kSmallThreads, OCC, small_lds_bytes<TMB>(), sgemm_small_kernel<TMB, false, OCC>, \
            sgemm_small_kernel<TMB, true, OCC>, EFF, true, 0, nullptr, nullptr, 1                         \
    }

static const TileConfig kTiles[] = {HPCDNN_SGEMM_TILE_LIST};
constexpr int kNumTiles = sizeof(kTiles) / sizeof(kTiles[0]);

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

// Persistent kernel against the tile-per-workgroup kernel of the same tile.  What it saves is a fixed time per tile,
// so the gain shrinks with K (measured 5 % at K = 256, 3 % at 512, 1-2.5 % at 1024, 0.5-1 % at 4096): that is the
// estimate a split plan has to beat.  Among unsplit plans a flat 2.5 % ranks better (it also stands for the
// eight-wave tiles' efficiency being fitted a little high): 4096 x 4096 x 1024 runs 2 % faster on the persistent
// 128 x 256 tile than on the 256 x 256 tile that the K-dependent figure would pick.
constexpr double kPersistGainK = 12.8, kPersistGainMax = 0.05, kPersistRankGain = 0.025;

// The persistent kernel takes unsplit problems of more than one round of whole tiles with an even number of K steps,
// enough of them to spread a tile's stores over.
static int persistent_grid(const TileConfig& t, int M, int N, int K, int cus) {
    const int grid = cus / kXcds * kXcds * t.persistent_per_cu;
    if (!t.persistent || (M % t.bm) || (N % t.bn) || (K % (2 * t.bk)) || K / t.bk < kPersistDripSteps + 2) return 0;
    return static_cast<int64_t>(M / t.bm) * (N / t.bn) > grid ? grid : 0;
}

static double plan_cost(const TileConfig& t, int M, int N, int K, int split, int cus, bool count_persistent = true) {
    const double tiles = static_cast<double>(ceil_div(M, t.bm)) * ceil_div(N, t.bn) * split;
    const double k_slice = ceil(static_cast<double>(ceil_div(K, split)) / t.bk) * t.bk;
    const bool edge = (M % t.bm) || (N % t.bn) || (K % t.bk);
    const double n = ceil(tiles / cus);
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
    if (count_persistent && split == 1 && persistent_grid(t, M, N, K, cus) > 0) cost *= 1.0 - kPersistRankGain;
    return cost;
}

// Tail split: with T tiles on `cus` CUs the last T % cus tiles keep only some CUs busy for a whole tile time.
// Splitting just those tiles s ways along K turns that round into ceil(r*s/cus) rounds of 1/s tile time each, at the
// price of writing and re-reading r*s raw tiles.  Returns the cost of the best s in 2..16 (slices of at least 8 K
// steps, partials that fit the workspace), and that s through *ways (0 = nothing to split or nothing fits).
static double tail_plan_cost(const TileConfig& t, int M, int N, int K, int cus, size_t ws_bytes, int* ways) {
    *ways = 0;
    const int64_t tiles = ceil_div(M, t.bm) * ceil_div(N, t.bn);
    const int64_t r = tiles % cus, full = tiles - r;
    if (full == 0 || r == 0) return 1e300;
    // (more left-over tiles than half the CUs: only the tiles of 128 x 128 and up have slices long enough to pay;
    // measured at 1280^3, where the model promised the 64 x 64 tile 9 % and the split ran 3 % slower)
    if (2 * r > cus && t.bm * t.bn < 128 * 128) return 1e300;
    const bool edge = (M % t.bm) || (N % t.bn) || (K % t.bk);
    const double per_tile = 2.0 * t.bm * t.bn * K / (kPeakFlopsPerCu * t.eff) * (edge ? kEdgePenalty : 1.0);
    const double n_full = static_cast<double>(full / cus);
    const double fixed = kFixedBase + kFixedPer32K * t.bm * t.bn / 32768.0;
    const double n = n_full + 1.0;
    const double exposed = t.blocks_per_cu == 1 ? n : 1.0 + kCoveredFraction * (n - 1.0);
    const size_t tile_bytes = static_cast<size_t>(t.bm) * t.bn * sizeof(float);
    const int64_t most = K / (8 * t.bk);
    double best = 1e300;
    for (int64_t s = 2; s <= 16 && s <= most; ++s) {
        if (static_cast<size_t>(r * s) * tile_bytes > ws_bytes) break;
        const double c = n_full * per_tile + ceil(static_cast<double>(r * s) / cus) * per_tile / s + exposed * fixed + kReduceFixed +
                         (2.0 * s + 1.0) * r * static_cast<double>(tile_bytes) / kReduceBytesPerSec;
        if (c < best) {
            best = c;
            *ways = static_cast<int>(s);
        }
    }
    return best;
}

static Plan choose_plan(int M, int N, int K, bool allow_split, size_t ws_bytes, bool allow_tail = true,
                        double* cost_out = nullptr, bool same_bits_only = false) {
    const int cus = device_cus();
    struct Candidate {
        Plan plan;
        double cost;
    };
    Candidate cand[kNumTiles * 10];
    int n_cand = 0;
    double best_cost = 1e300;
    for (int t = 0; t < kNumTiles; ++t) {
        const TileConfig& cfg = kTiles[t];
        if (cfg.eff <= 0.f || (same_bits_only && cfg.wave_split_k)) continue;
        // (more than 64 slices only for the tiles of at most 64 x 64: they are for products too small to fill the CUs
        // otherwise; measured on 96..256-square products with K up to 262144, the larger tiles lost with them)
        const int max_split = cfg.bm * cfg.bn <= 64 * 64 ? 256 : 64;
        for (int split = 1; split <= max_split; split *= 2) {
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
    int best_unsplit_tile = -1;
    for (int i = 0; i < n_cand; ++i)
        if (cand[i].plan.split == 1 && cand[i].cost < best_unsplit) {
            best_unsplit = cand[i].cost;
            best_unsplit_tile = cand[i].plan.tile;
        }
    double unsplit_to_beat = best_unsplit;
    if (best_unsplit_tile >= 0 && persistent_grid(kTiles[best_unsplit_tile], M, N, K, cus) > 0) {
        const double gain = kPersistGainK / K;
        unsplit_to_beat *= (1.0 - (gain < kPersistGainMax ? gain : kPersistGainMax)) / (1.0 - kPersistRankGain);
    }
    if (unsplit_to_beat <= best_cost * 1.025 || best_unsplit <= best_cost) {
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
            // (without the persistent kernel's gain: a second launch has to pay for itself on round counting alone)
            const double c1 = plan_cost(cfg, static_cast<int>(rows1), N, K, 1, cus, false);
            double c2 = 0.0;
            const Plan rest = choose_plan(M - static_cast<int>(rows1), N, K, false, 0, false, &c2, true);
            const double c = c1 + c2 + kSecondLaunch;
            if (c < best.cost) best = RowSplit{t, static_cast<int>(rows1), rest.tile, c};
        }
    }
    return best;
}

// ta: A is given transposed (K x M row-major): the kernels of sgemm_ta.hip; everything else (plans, splits,
// reductions) is shared.
static int run_sgemm(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                     float alpha, float beta, void* ws, size_t ws_bytes, int tile, int split, hipStream_t stream,
                     bool ta = false) {
    int rc = check_gemm_args(M, N, K, A, lda, B, ldb, C, ldc, ta);
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
            bool ws_aligned, valid, ta;
            Plan plan;
            RowSplit rows;
        };
        static thread_local Decision memo{};
        // the tail split moves 16-byte groups through the workspace
        const bool ws_aligned = (reinterpret_cast<uintptr_t>(ws) & 15u) == 0;
        const size_t usable = ws ? ws_bytes : 0;
        const int cus = device_cus();  // of the current device: the plan depends on it
        if (!(memo.valid && memo.M == M && memo.N == N && memo.K == K && memo.cus == cus && memo.ws_bytes == usable &&
              memo.ws_aligned == ws_aligned && memo.ta == ta)) {
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
            memo.ta = ta;
            memo.valid = true;
        }
        Plan plan = memo.plan;
        // a forced tail split needs a tile that has one (not the 32 x 32 tile, whose waves split K among themselves)
        if (tile < 0 && split < -1) plan = choose_plan(M, N, K, false, 0, false, nullptr, true);
        const RowSplit rs = memo.rows;  // copied: the nested calls below do not touch the memo, but keep it simple
        if (tile < 0 && split == 0 && rs.tile1 >= 0) {
            rc = run_sgemm(rs.rows1, N, K, A, lda, B, ldb, C, ldc, alpha, beta, nullptr, 0, rs.tile1, 1, stream, ta);
            if (rc != HPCDNN_OK) return rc;
            return run_sgemm(M - rs.rows1, N, K, A + (ta ? rs.rows1 : static_cast<int64_t>(rs.rows1) * lda), lda, B, ldb,
                             C + static_cast<int64_t>(rs.rows1) * ldc, ldc, alpha, beta, nullptr, 0, rs.tile2, 1, stream, ta);
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
    GemmArgs a = make_args(M, N, K, A, lda, B, ldb, C, ldc, alpha, beta, cfg.bm, cfg.bn);
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
    const bool edge = needs_edge(a, cfg.bm, cfg.bn, cfg.bk);
    void (*fn)(const GemmArgs) = ta ? sgemm_ta_kernel(tile, cfg.bm, cfg.bn, edge) : edge ? cfg.edge : cfg.plain;
    if (!fn) return HPCDNN_ERR_INVALID_VALUE;
    dim3 grid(a.full_tiles + tail_tiles * a.tail_split, 1, split);
    // Several rounds of whole tiles written straight to C: one persistent workgroup per CU walks its tiles as one
    // stream of K steps (same bits; see sgemm_persistent_kernel.h for what it saves)
    const int persistent = (split == 1 && tail_tiles == 0 && ldc <= kMaxLdc) ? persistent_grid(cfg, M, N, K, device_cus()) : 0;
    void (*const pfn)(const GemmArgs) = ta ? sgemm_ta_persistent_kernel(tile, cfg.bm, cfg.bn, beta != 0.f)
                                           : beta == 0.f ? cfg.persistent : cfg.persistent_beta;
    if (persistent > 0 && pfn) {
        fn = pfn;
        grid = dim3(persistent, 1, 1);
    }
    rc = enable_lds(fn, cfg.lds_bytes);
    if (rc != HPCDNN_OK) return rc;

    hipLaunchKernelGGL(fn, grid, dim3(cfg.threads), cfg.lds_bytes, stream, a);
    rc = launch_status();
    if (rc != HPCDNN_OK) return rc;
    if (tail_tiles > 0) {
        tail_reduce_kernel<><<<dim3(tail_tiles, cfg.bm / 32), 256, 0, stream>>>(M, N, cfg.bm, cfg.bn, a.tiles_m, a.tiles_n,
                                                                             a.full_tiles, a.tail_split, a.tail_partial, C,
                                                                             ldc, alpha, beta, nullptr, nullptr, 1, 1, 0, 0);
        return launch_status();
    }
    if (split == 1) return rc;

    const int64_t total = static_cast<int64_t>(M) * N;
    if (split > 8 && N % 4 == 0 && (reinterpret_cast<uintptr_t>(ws) & 15u) == 0) {
        // many slices: four lanes per group of elements, so that all of a lane's slices are in flight at once
        launch_splitk_reduce_wide(M, N, split, static_cast<const float*>(ws), C, ldc, alpha, beta, device_cus(), stream);
        return launch_status();
    }
    int rgrid = static_cast<int>(ceil_div(total, 256));
    const int cap = device_cus() * 8;
    if (rgrid > cap) rgrid = cap;
    splitk_reduce_kernel<><<<rgrid, 256, 0, stream>>>(M, N, split, static_cast<const float*>(ws), C, ldc, alpha, beta);
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

extern "C" int hpcdnn_sgemm_tn(int M, int N, int K, const float* At, int ldat, const float* B, int ldb, float* C, int ldc,
                               float alpha, float beta, void* ws, size_t ws_bytes, void* stream) {
    return run_sgemm(M, N, K, At, ldat, B, ldb, C, ldc, alpha, beta, ws, ws_bytes, -1, 0, static_cast<hipStream_t>(stream), true);
}

extern "C" int hpcdnn_sgemm_tn_ex(int M, int N, int K, const float* At, int ldat, const float* B, int ldb, float* C, int ldc,
                                  float alpha, float beta, void* ws, size_t ws_bytes, int tile, int split_k, void* stream) {
    return run_sgemm(M, N, K, At, ldat, B, ldb, C, ldc, alpha, beta, ws, ws_bytes, tile, split_k,
                     static_cast<hipStream_t>(stream), true);
}

// Column-major C (M x N) = alpha * A (M x K) * B (N x K)^T + beta * C is, read row by row, the N x M matrix
// C^T = alpha * (B^T)^T * A^T + beta * C^T with B^T = the memory of B as K rows of N and A^T = the memory of A as K
// rows of M: the transposed-left-operand product with the operands swapped.
extern "C" int hpcdnn_sgemm_cm_nt(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                                  float alpha, float beta, void* ws, size_t ws_bytes, void* stream) {
    return run_sgemm(N, M, K, B, ldb, A, lda, C, ldc, alpha, beta, ws, ws_bytes, -1, 0, static_cast<hipStream_t>(stream), true);
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

namespace hpcdnn {
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
