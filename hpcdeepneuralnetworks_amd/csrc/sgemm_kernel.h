// Row-major FP32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32).
//
// One workgroup of WGM x WGN waves (4 or 8) owns a BM x BN tile of C; wave w owns
// a (BM/WGM) x (BN/WGN) sub-tile made of 32x32 MFMA blocks whose accumulators
// stay in registers for the whole K loop.  K advances in steps of 16.
//
// Data path per K step: HBM/L2 -> VGPR with buffer_load_dwordx4 (the hardware
// range check of the buffer descriptor returns 0 for rows past the end of the
// matrix, so ragged tiles need no branches) -> LDS (ds_write_b128) -> operand
// fragments (ds_read) -> MFMA.  Global loads run two K steps ahead of the
// MFMAs that consume them, LDS is double buffered, fragments are double
// buffered in registers.
//
// LDS layout (floats):
//   A stage: [BM][20]       k contiguous, as in memory.  Lane (row r, half h)
//            reads 16 bytes = k {8g+4h .. 8g+4h+3}: one ds_read_b128 feeds four
//            MFMA k-steps.  Row stride 20 spreads 8 consecutive rows over all
//            banks for that read.
//   B stage: [16][BN + 8]   n contiguous, as in memory; lane (col c, half h)
//            reads B[8g+4h+q][c] with ds_read_b32.  Stride BN+8 puts the two
//            half-waves (rows 4 apart) on disjoint banks.  128- and 192-column
//            tiles use stride 264 (same banks): with rows less than 256 words
//            apart the compiler pairs the reads into ds_read2_b32, whose 8-bit
//            offsets cannot hold the stage and block offsets, and adds those to
//            the address with vector-ALU instructions inside the K loop.
// The MFMA k index is a permutation of the memory k index (lane half h of
// k-step q in group g carries k = 8g+4h+q); A and B use the same permutation,
// so the contraction is unchanged.
//
// Accumulator layout of one 32x32 block (16 VGPRs): register v of lane l holds
// element (row 8*(v/4) + 4*(l/32) + v%4, col l%32).
//
// Instruction order in the main loop is fixed by hand: the MFMA pipe takes 64
// cycles per instruction, and "side" instructions (fragment reads, global
// loads, LDS writes, a few checksum VALU ops) are placed one group behind each
// MFMA so that they issue while the matrix core is busy.  sched_barrier fences
// keep the compiler from regrouping them.
//
// With FT != 0 the kernel is the online-ABFT variant: see "ABFT encode" in the
// main loop and "ABFT verification" after it.  GRAN = 1 keeps one checksum pair
// per wave tile instead of one per workgroup tile; CADENCE verifies every
// check_interval values of k inside the K loop as well as after it.
#pragma once

#include <type_traits>

#include "common.h"

namespace hpcdnn {

constexpr int kMaxFaults = HPCDNN_FT_MAX_FAULTS;

struct GemmArgs {
    int M, N, K;
    const float* A;
    int lda;
    const float* B;
    int ldb;
    float* C;
    int ldc;
    float alpha, beta;
    int tiles_m, tiles_n;
    int k_chunk;     // K range of one grid.z slice, a multiple of 16 (>= K when not split)
    float* partial;  // split-K: [gridDim.z][M][N] raw accumulators; nullptr = write C directly
    // tail split: workgroups 0 .. full_tiles-1 compute whole tiles; the tiles after them are each split tail_split
    // ways along K (tail_k_chunk per slice) and write raw accumulators to tail_partial[tile - full_tiles][slice][BM*BN]
    int full_tiles, tail_split, tail_k_chunk;
    float* tail_partial;
    hpcdnn_ft_status* tail_status;  // ABFT with a tail split: [tile - full_tiles][slice][check tile of the workgroup tile]
    // ABFT
    float tau;      // absolute residual threshold; 0 = relative mode
    float tau_rel;  // relative mode: threshold of a line = tau_rel * sum |accumulators of the line| / sqrt(elements in it)
    int n_faults;   // test faults: delta is added to accumulator (row, col) of workgroup tile `tile` before verification `check`
    struct {
        int tile, row, col;
        float delta;
        int check;
    } faults[kMaxFaults];
    int check_interval;          // CADENCE kernels: values of k between two verifications, a multiple of the K step
    int locate_rc;               // FT == 3 kernels: 0 = the column from the weighted checksum; 1 = row x column, the rows as the screen
    int status_rows, status_ld;  // records are laid out as a status_rows x status_ld grid of check tiles
    hpcdnn_ft_status* status;
    const float* enc_a;  // FT == 2: [row groups][enc_ld] column sums of A over the rows of each check tile
                         // FT == 3: [column groups][enc_ld] weighted row sums of B (weights 1, 2, ... over the tile's columns)
    const float* enc_b;  // FT >= 2: [column groups][enc_ld] row sums of B over the columns of each check tile
    int enc_ld;          // row length: K rounded up to the K step, plus two K steps of zeros
};

constexpr int kGemmBK = 16;
constexpr int kXcds = 8;
constexpr int kGroupM = 4;  // tile rows swept together so that co-resident tiles share A and B panels

// Row stride (floats) of the staged B tile (see the LDS layout above).  The 64-column tiles take the wide stride in
// the ABFT kernels only: four plain 64 x 64 workgroups per CU would not fit in LDS with it, and their loops have the
// registers to keep the paired reads' addresses.
template <int BN, int FT = 0>
constexpr int b_stage_stride() {
    return (BN == 128 || BN == 192 || (BN == 64 && FT != 0)) ? 264 : BN + 8;
}

// LDS the ABFT verification needs (it reuses the staging buffers once the K loop has drained): FP64 partials of the
// reference checksums, observed line sums and their absolute counterparts per wave row / wave column, one residual
// per line, one record per check tile, per-wave sums of |acc| per check tile.  GM x GN check tiles per workgroup tile.
// (the kernels whose screen is the row checksum - the weighted locator, and row x column on products one tile wide -
// keep, behind the BM row residuals, either the weighted residual of the flagged row or the BN column residuals)
template <int BM, int BN, int WGM, int WGN, int GM, int GN, bool WEIGHTED = false>
constexpr size_t ft_verify_lds_bytes() {
    constexpr size_t threads = static_cast<size_t>(WGM) * WGN * 64;
    constexpr size_t ccp = threads / (BN / 4), crp = kGemmBK / 4;
    constexpr size_t lines = WEIGHTED ? static_cast<size_t>(BM) + (BM > BN ? BM : BN) : static_cast<size_t>(GN) * BM + static_cast<size_t>(GM) * BN;
    return sizeof(double) * (GM * ccp * BN + GN * crp * BM) + sizeof(float) * (2 * (WGM * BN + WGN * BM) + lines) +
           32 * GM * GN + sizeof(float) * GM * GN * (threads / 64) + 2 * sizeof(float) * GM * GN;
}

template <int BM, int BN, int FT = 0, int THREADS = 256, int WGM = 2, int WGN = 2, int GRAN = 0>
constexpr size_t gemm_lds_bytes() {
    // two stages of the A and B tiles; the ABFT kernel adds two stages of checksum partials (16 k x one column
    // sum per wave, 16 row sums) and a dump area for the branch-free predicated writes of the lanes that
    // publish nothing (one word per thread plus the reach of the strided writes)
    constexpr size_t staging = sizeof(float) * 2 * (static_cast<size_t>(BM) * (kGemmBK + 4) + static_cast<size_t>(kGemmBK) * b_stage_stride<BN, FT>()) +
           (FT == 1 ? sizeof(float) * (2 * (kGemmBK * (THREADS / 64) + kGemmBK) + THREADS + 2 * kGemmBK * (THREADS / 64)) : 0);
    constexpr size_t verify = FT ? ft_verify_lds_bytes<BM, BN, WGM, WGN, GRAN ? WGM : 1, GRAN ? WGN : 1, FT == 3>() : 0;
    return staging > verify ? staging : verify;
}

template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// Pins a value at this point of the instruction stream: the compiler may neither sink the computation that
// produces it below this point nor hoist its uses above it (it would otherwise gather the checksum arithmetic,
// which has no side effects, into one block and stall the matrix core behind it).
#define HPCDNN_PIN(x) asm volatile("" : "+v"(x))

// Workgroup id -> tile.  The hardware deals consecutive workgroup ids round-
// robin to the 8 XCDs (each with a private L2), so id -> (xcd = id % 8,
// slot = id / 8) and XCD x is handed the contiguous tile range it alone will
// touch; inside the range tiles go down kGroupM rows before moving one column
// right, so the tiles resident at one time form a compact block of C.
__device__ __forceinline__ void tile_of_block(int id, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int nt = tiles_m * tiles_n;
    const int per = nt / kXcds, rem = nt % kXcds;
    const int xcd = id % kXcds, slot = id / kXcds;
    const int logical = xcd * per + (xcd < rem ? xcd : rem) + slot;
    const int width = kGroupM * tiles_n;
    const int group = logical / width;
    const int first_m = group * kGroupM;
    const int gsz = (tiles_m - first_m < kGroupM) ? tiles_m - first_m : kGroupM;
    const int in_group = logical - group * width;
    tm = first_m + in_group % gsz;
    tn = in_group / gsz;
}

// One element of A * B computed again, for the ABFT correction: the sum over k in [k0, k1) of
// a[k * a_stride] * b[k * b_stride] as one chain of fused multiply-adds in the order the matrix core adds them (per K
// step of 16 and half step g, the pairs k = 8g + q, 8g + 4 + q for q = 0..3: a 32x32x2 FP32 MFMA is two chained FMAs,
// lanes 0-31's k first; zeros pad the last K step), so the element gets exactly the bits a fault-free run gives it.
// All `threads` threads of the workgroup call it together: they stage the operand row and column through LDS
// (`stage`: 2 * chunk floats, chunk a multiple of 16), thread 0 walks them, and only thread 0's return value means
// anything.  Kept out of line on purpose: inlined into the GEMM kernels, the address arithmetic of this (cold) code
// changed the register assignment of their main loops, which cost the 256x128 kernel 1 % of a 4096^3 product.
static __device__ __attribute__((noinline)) float recompute_element(const float* a, int64_t a_stride, const float* b, int64_t b_stride,
                                                           int k0, int k1, float* stage, int chunk, int tid, int threads) {
    float* const s_fa = stage;
    float* const s_fb = stage + chunk;
    float val = 0.f;
#pragma unroll 1
    for (int kc = k0; kc < k1; kc += chunk) {
        const int len = (k1 - kc < chunk) ? k1 - kc : chunk;
        const int padded = (len + kGemmBK - 1) / kGemmBK * kGemmBK;
#pragma unroll 1
        for (int i = tid; i < padded; i += threads) {
            const int k = kc + i;
            s_fa[i] = i < len ? a[static_cast<int64_t>(k) * a_stride] : 0.f;
            s_fb[i] = i < len ? b[static_cast<int64_t>(k) * b_stride] : 0.f;
        }
        __syncthreads();
        if (tid == 0) {
#pragma unroll 1
            for (int i = 0; i < padded; i += kGemmBK) {
                float av[kGemmBK], bv[kGemmBK];
#pragma unroll
                for (int e = 0; e < kGemmBK; e += 4) {
                    *reinterpret_cast<v4f*>(av + e) = *reinterpret_cast<const v4f*>(s_fa + i + e);
                    *reinterpret_cast<v4f*>(bv + e) = *reinterpret_cast<const v4f*>(s_fb + i + e);
                }
#pragma unroll
                for (int g = 0; g < 2; ++g)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        val = __builtin_fmaf(av[8 * g + q], bv[8 * g + q], val);
                        val = __builtin_fmaf(av[8 * g + 4 + q], bv[8 * g + 4 + q], val);
                    }
            }
        }
        __syncthreads();
    }
    return val;
}

// FT: 0 = plain SGEMM; 1 = ABFT, checksum vectors e^T A and B e formed inside the main loop; 2 = ABFT, checksum
// vectors read from a workspace filled by abft_encode_kernel (fewer VALU instructions in the main loop); 3 = ABFT with
// the weighted-checksum locator (the reference's "kernel 2", kernel/ft_sgemm/README.md:16-26: two row sums of B,
// e1 = [1, 1, ...] and e2 = [1, 2, ...], and nothing from A): references A (B e1) and A (B e2) against the plain and
// the weighted row sums of the accumulators; a faulty row is found by the first pair, the column inside it as the
// ratio of the two residuals; both vectors of B come from the workspace (abft_encode_weighted_kernel).  The main loop
// accumulates the first reference only: the second pair is needed for one row, and only once that row is flagged, so
// it is formed then (the row of A times the weighted vector, the weighted sum of the row's accumulators).
//
// NSLOT: staging register sets.  K step t + 1 waits in one of them while steps up to t + NSLOT are on their way from
// memory.  Two are enough while a K step takes longer than a trip to memory (big tiles) or the operands come from
// L2; a small tile that streams an operand from HBM with one workgroup per CU needs its loads further ahead.
//
// GRAN (ABFT only): 0 = one checksum pair, one verification and one status record per workgroup tile; 1 = per wave
// tile (BM / WGM) x (BN / WGN): every wave tile is verified, located and corrected on its own, so one fault per wave
// tile is correctable.  Needs the pre-encoded checksum vectors (FT == 2), one per wave row / wave column.
// CADENCE (ABFT only): the K loop runs in intervals of p.check_interval; after each interval the pipeline drains,
// the accumulators are verified against the references of the k range done so far, and the references are
// re-synchronised, as the reference kernel does every 256 k (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:143,263-271).
//
// TA: the left operand is given transposed, p.A = A^T as a K x M row-major matrix with row length
// p.lda >= M, which is how the operands of a column-major C = A * B^T lie in memory
// (kernel/ft_sgemm/include/sgemm_huge.cuh:14, cublasSgemm(N, T, ...) in kernel/ft_sgemm/sgemm.cu:111).  A K step of
// the tile is then 16 rows of BM floats, like B's; a lane fetches four consecutive m of one k and writes them as four
// words into the same [m][k] staging layout, so everything from the fragment reads on is the code of the untransposed
// case and every element of C sums its products in the same order.  The ABFT loop, whose row checksums work on a
// lane's four k of one row, reads those back from the LDS stage that the transposed writes have just filled.
template <int BM, int BN, int WGM, int WGN, bool EDGE, int FT, int MIN_BLOCKS, int NSLOT = 2, int GRAN = 0, bool CADENCE = false,
          bool TA = false>
__global__ __launch_bounds__(WGM * WGN * kWave, MIN_BLOCKS) void sgemm_kernel(const GemmArgs p) {
    constexpr int BK = kGemmBK;
    static_assert(NSLOT >= 2 && NSLOT % 2 == 0, "an even number of staging sets: LDS stages alternate with the K steps");
    static_assert(NSLOT == 2 || FT == 0, "the ABFT kernels are instantiated and tested with two staging sets");
    static_assert(FT != 0 || (GRAN == 0 && !CADENCE), "granularity and cadence belong to the ABFT kernels");
    static_assert(GRAN == 0 || FT == 2, "wave-tile checksums come from the pre-encoded vectors");
    static_assert(FT != 3 || (GRAN == 0 && !CADENCE), "the weighted locator checks a workgroup tile once, after the K loop");
    constexpr bool kWeighted = FT == 3;
    constexpr int GM = GRAN ? WGM : 1, GN = GRAN ? WGN : 1;  // check tiles per workgroup tile
    constexpr int CM = BM / GM, CN = BN / GN;                // check tile
    static_assert(CM % 32 == 0 && CN % 32 == 0, "check tiles are made of 32x32 blocks");
    constexpr int kGemmThreads = WGM * WGN * kWave;
    static_assert(WGM * WGN == 4 || WGM * WGN == 8, "four or eight waves per workgroup");
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(TM >= 1 && TN >= 1 && WM % 32 == 0 && WN % 32 == 0, "wave tile is made of 32x32 blocks");
    constexpr int AS = BK + 4, BS = b_stage_stride<BN, FT>();
    constexpr int A_STAGE = BM * AS, B_STAGE = BK * BS;
    constexpr int A_V4_PER_ROW = BK / 4, B_V4_PER_ROW = BN / 4;
    constexpr int A_SLOTS = BM * BK / 4 / kGemmThreads, B_SLOTS = BK * BN / 4 / kGemmThreads;
    static_assert(A_SLOTS >= 1 && B_SLOTS >= 1, "every thread stages at least one 16-byte group of A and of B");
    static_assert((BM * BK) % (4 * kGemmThreads) == 0 && (BN * BK) % (4 * kGemmThreads) == 0,
                  "tiles split evenly over the threads");
    constexpr int NGL = A_SLOTS + B_SLOTS;  // global loads (and LDS writes) per thread per K step
    constexpr int NRD = TM + TN;            // fragment read groups per half K step
    constexpr int NMG = 4 * TM * TN;        // MFMAs per half K step (8 k values)
    constexpr bool kShortStep = FT == 0 && NMG <= 8;  // one or two 32x32 blocks per wave: little to hide latencies behind
    constexpr bool kNoBounds = kShortStep && !EDGE;
    constexpr bool kEarlyStore = kShortStep && NSLOT > 2;
    // Plain SGEMM on ragged tiles: the loads of every K step but the slice's last touch nothing outside the
    // matrices once rows m >= M are folded onto row M - 1 (what they read only reaches accumulators that are never
    // stored), so those steps run with unbounded descriptors and plain pointer steps; the byte counts that the range
    // checks need are formed only for the steps at the end of the slice.
    constexpr bool kLazyBounds = EDGE && FT == 0;
    // ABFT with checksum vectors from the workspace, ragged tiles: the staged columns n >= N of B (TA: m >= M of A^T)
    // hold the next row or padding.  The vectors cover the matrix only, so that data reaches nothing but the
    // accumulators and reference sums of lines outside the matrix, which the verification sets to zero first; the K
    // steps then need no masks but the last two of a slice.  The kernels without a workspace sum the staged rows of A
    // themselves - nothing of B, see kLazyRows -, so they run the same way unless A is given transposed (its staged
    // columns m >= M would enter the column sums).
    constexpr bool kLazyOutside = EDGE && (FT >= 2 || !TA);
    // Row x column locator: the column checksums screen every verification, the row checksums are looked at only when
    // a column is flagged - so the main loop carries the column references alone (a_c from the workspace or summed
    // from the staged rows of A), and the row references of the tile (its rows of A times the row sums of B, from the
    // workspace or summed from B then) are formed when they are needed, by the whole workgroup, in the verification.
    // The weighted locator, whose screen is the plain row checksum, carries that one.
    constexpr bool kLazyRows = FT == 1 || FT == 2;
    // ... and the row sums of B they need are formed then as well, unless there is one per wave column (wave-tile
    // checksums: those come from the workspace): the pre-pass of the workgroup-tile kernels reads A only.
    constexpr bool kRowSumsAtDetection = FT == 1 || (FT == 2 && GRAN == 0);

    extern __shared__ __align__(16) float smem[];
    float* const As = smem;
    float* const Bs = smem + 2 * A_STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave / WGN, wn = wave % WGN;

    int tile_m, tile_n;
    int tile_id = blockIdx.x, k_slice = blockIdx.z, k_chunk = p.k_chunk;
    float* tail_out = nullptr;
    int tail_slot = 0;  // index of this slice among all tail slices
    if (p.tail_split > 1 && tile_id >= p.full_tiles) {
        const int r = tile_id - p.full_tiles;
        tail_slot = r;
        tile_id = p.full_tiles + r / p.tail_split;
        k_slice = r % p.tail_split;
        k_chunk = p.tail_k_chunk;
        tail_out = p.tail_partial + static_cast<size_t>(r) * (BM * BN);
    }
    if (FT == 0 && gridDim.z > 1 && gridDim.z % kXcds == 0) {
        // Split K with a multiple of eight slices: every XCD takes whole K slices with all their tiles (workgroups are
        // dealt to the XCDs round-robin in the order x, then z), so a K slice of A and of B crosses from memory into
        // one L2 once, whichever tiles share its rows and columns.  Dealt tile by tile, the few tiles of a deep
        // product land on different XCDs and each fetches its operands for itself (128 x 128 x 65536: 131 MB from
        // memory for 67 MB of operands, which made the slices wait for memory).
        const int linear = blockIdx.x + gridDim.x * blockIdx.z;
        const int slot = linear / kXcds;
        k_slice = (slot / gridDim.x) * kXcds + linear % kXcds;
        tile_id = slot % gridDim.x;
        tile_m = tile_id % p.tiles_m;
        tile_n = tile_id / p.tiles_m;
    } else {
        tile_of_block(tile_id, p.tiles_m, p.tiles_n, tile_m, tile_n);
    }
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    // (a tile that hangs over the last column reads B past the ends of its rows: into the next row, which must exist
    // and be long enough for that to stay inside the matrix)
    const bool lazy_ok = (n0 + BN <= p.N || p.ldb >= BN) && (!TA || m0 + BM <= p.M || p.lda >= BM);
    // the K range of one pass of the pipeline: the slice, or one verification interval of it
    int kbeg = k_slice * k_chunk;
    int kend = (p.K - kbeg < k_chunk) ? p.K : kbeg + k_chunk;
    int nkt = (kend - kbeg + BK - 1) / BK;

    // ---- global -> register staging: which 16-byte groups of the A and B tiles this thread moves.
    // Descriptors start at the tile's first element of the current K step and end with the matrix, so that
    // rows m >= M of A and rows k >= K of B read as 0; the base moves forward by one K step per load.
    // (TA: A^T is walked like B, rows k >= K read as 0, and columns m >= M, the next row or padding, only reach
    // accumulators of rows m >= M, which are never stored)
    auto a_origin = [&](int k) { return TA ? p.A + static_cast<int64_t>(k) * p.lda + m0 : p.A + static_cast<int64_t>(m0) * p.lda + k; };
    auto a_bytes_left = [&](int k) {  // bytes from a_origin(k) to the end of A
        return TA ? (static_cast<int64_t>(p.K - 1 - k) * p.lda + (p.M - m0)) * 4 : (static_cast<int64_t>(p.M - 1 - m0) * p.lda + (p.K - k)) * 4;
    };
    const float* a_base = a_origin(kbeg);
    const float* b_base = p.B + static_cast<int64_t>(kbeg) * p.ldb + n0;
    int64_t a_left = a_bytes_left(kbeg);
    int64_t b_left = (static_cast<int64_t>(p.K - 1 - kbeg) * p.ldb + (p.N - n0)) * 4;
    const int64_t a_step = static_cast<int64_t>(BK) * p.lda;  // TA only (the untransposed A moves on by BK floats)
    const int64_t b_step = static_cast<int64_t>(BK) * p.ldb;

    int a_voff[A_SLOTS], a_lds[A_SLOTS], a_kc[A_SLOTS];
    int a_nvalid[A_SLOTS];  // TA: columns of the slot's group of four m inside the matrix (may be <= 0 or >= 4)
    int a_lds_rows[A_SLOTS];  // TA ABFT: where the untransposed staging keeps this thread's row and k group
    int b_voff[B_SLOTS], b_lds[B_SLOTS], b_row[B_SLOTS], b_nvalid[B_SLOTS];
#pragma unroll
    for (int s = 0; s < A_SLOTS; ++s) {
        const int idx = tid + s * kGemmThreads;
        if constexpr (TA) {
            // four neighbouring lanes take 64 contiguous bytes of one row of A^T (one request to the vector cache,
            // as in the untransposed case), the sixteen quads of a wave the sixteen k; a wave's word writes of one
            // of a lane's four m land in 64 different LDS banks (80 q + k for q = 0..3, k = 0..15)
            const int k = (idx / 4) % BK, m = ((idx / (4 * BK)) * 4 + idx % 4) * 4;
            a_kc[s] = k;
            a_voff[s] = (k * p.lda + m) * 4;
            a_lds[s] = m * AS + k;
            a_nvalid[s] = p.M - (m0 + m);
            a_lds_rows[s] = (idx / A_V4_PER_ROW) * AS + (idx % A_V4_PER_ROW) * 4;
        } else {
            int row = idx / A_V4_PER_ROW;
            a_kc[s] = (idx % A_V4_PER_ROW) * 4;
            if constexpr (kLazyBounds) row = row < p.M - m0 ? row : p.M - 1 - m0;
            a_voff[s] = (row * p.lda + a_kc[s]) * 4;
            a_lds[s] = row * AS + a_kc[s];
        }
    }
#pragma unroll
    for (int s = 0; s < B_SLOTS; ++s) {
        const int idx = tid + s * kGemmThreads;
        b_row[s] = idx / B_V4_PER_ROW;
        const int nc = (idx % B_V4_PER_ROW) * 4;
        b_voff[s] = (b_row[s] * p.ldb + nc) * 4;
        b_lds[s] = b_row[s] * BS + nc;
        b_nvalid[s] = p.N - (n0 + nc);  // columns of this group inside the matrix (may be <= 0 or >= 4)
    }

    v4f ra[NSLOT][A_SLOTS], rb[NSLOT][B_SLOTS];  // staging sets: K steps t+1 .. t+NSLOT are in flight while t is multiplied
    int k_loaded = kbeg;                 // absolute k of the K step the next load call fetches

    // One staging load (part P of the K step at a_base/b_base) into slot S.  Nothing here touches the loaded
    // value, so the load stays in flight until the slot is consumed a K step later.
    int k_mask = kbeg;  // ragged tiles: absolute k of the K step whose staged data goes to LDS next (the one the masks see)
    // FT == 2: the K step's slice of the pre-encoded checksum vectors travels with it (same run-ahead, same
    // slots).  The rows of enc_a / enc_b end with two K steps of zeros, so the fetches that run ahead past the
    // end need no bounds: one descriptor per row, a per-thread offset, and a scalar offset that moves on by one
    // K step per fetch.
    // (with wave-tile checksums the tile's GM / GN rows of the vectors follow each other: one descriptor over all
    // of them, the row chosen by the scalar offset)
    const __amdgpu_buffer_rsrc_t enc_a_rsrc =
        make_rsrc(FT == 2 ? p.enc_a + static_cast<int64_t>(tile_m) * GM * p.enc_ld : nullptr, static_cast<int64_t>(p.enc_ld) * GM * 4);
    const __amdgpu_buffer_rsrc_t enc_b_rsrc =
        make_rsrc(FT >= 2 ? p.enc_b + static_cast<int64_t>(tile_n) * GN * p.enc_ld : nullptr, static_cast<int64_t>(p.enc_ld) * GN * 4);
    const int enc_row_bytes = p.enc_ld * 4;
    // a_c of the k rows of B this thread stages: k = tid / (BN / 4) (and k + 8 when it stages two), which the
    // pre-encode kernel stores side by side (order 0, 8, 1, 9, ... inside each K step)
    const int enc_a_voff = B_SLOTS == 2 ? (tid / B_V4_PER_ROW) * 8 : ((((tid / B_V4_PER_ROW) & 7) * 2 + (tid / B_V4_PER_ROW) / 8) * 4);
    const int enc_b_voff = (tid & 3) * 16;  // b_r of the four k values of A this thread stages
    int enc_off = kbeg * 4;
    float g_ac[NSLOT][GM][B_SLOTS];
    v4f g_br[NSLOT][GN];
    auto gload1 = [&](auto slot, auto part, auto bulk) __attribute__((always_inline)) {  // bulk: this K step is not the slice's last (kLazyBounds)
        constexpr int S = decltype(slot)::value, P = decltype(part)::value;
        if constexpr (kNoBounds || (kLazyBounds && decltype(bulk)::value)) {
            if constexpr (P < A_SLOTS) ra[S][P] = buffer_load_v4f(make_rsrc_unbounded(a_base), a_voff[P]);
            else rb[S][P - A_SLOTS] = buffer_load_v4f(make_rsrc_unbounded(b_base), b_voff[P - A_SLOTS]);
        } else {
            if constexpr (P < A_SLOTS) ra[S][P] = buffer_load_v4f(make_rsrc(a_base, a_left), a_voff[P]);
            else rb[S][P - A_SLOTS] = buffer_load_v4f(make_rsrc(b_base, b_left), b_voff[P - A_SLOTS]);
        }
        if constexpr (FT == 3 && P == NGL - 1) {
            g_br[S][0] = __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(enc_b_rsrc, enc_b_voff, enc_off, 0));
        }
        if constexpr (FT == 2 && P == NGL - 1) {
            static_assert(FT != 2 || B_SLOTS <= 2, "a thread stages one or two k rows of B");
#pragma unroll
            for (int gm = 0; gm < GM; ++gm) {
                const int soff = enc_off + gm * enc_row_bytes;
                if constexpr (B_SLOTS == 2) {
                    typedef float v2f __attribute__((ext_vector_type(2)));
                    const v2f t = __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(enc_a_rsrc, enc_a_voff, soff, 0));
                    g_ac[S][gm][0] = t[0];
                    g_ac[S][gm][B_SLOTS - 1] = t[1];
                } else {
                    g_ac[S][gm][0] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(enc_a_rsrc, enc_a_voff, soff, 0));
                }
            }
        }
    };
    // Ragged tiles only, applied when the slot is consumed: columns k >= kend of A hold padding, the next K
    // slice or the next row: force them to 0 (rows m >= M of A and k >= K of B already read as 0 through the
    // descriptor).  Columns n >= N of B hold the next row or padding too, but they only ever reach accumulators of
    // columns n >= N, which are never stored: plain SGEMM leaves them alone, the ABFT kernels (whose row sums of B
    // run over the whole tile width) force them to 0 as well.
    auto gmask1 = [&](auto slot, auto part) __attribute__((always_inline)) {
        constexpr int S = decltype(slot)::value, P = decltype(part)::value;
        if constexpr (P < A_SLOTS && TA) {
            // rows k >= K of A^T read as 0, and a K slice ends on a K step unless it ends with K; columns m >= M
            // (the next row or padding) matter to the ABFT kernels only, whose column sums run over the whole tile
            if constexpr (FT != 0) {
                const int nv = a_nvalid[P];
                v4f v = ra[S][P];
                v.x = nv > 0 ? v.x : 0.f;
                v.y = nv > 1 ? v.y : 0.f;
                v.z = nv > 2 ? v.z : 0.f;
                v.w = nv > 3 ? v.w : 0.f;
                ra[S][P] = v;
            }
        } else if constexpr (P < A_SLOTS) {
            const int left = kend - (k_mask + a_kc[P]);
            v4f v = ra[S][P];
            v.x = left > 0 ? v.x : 0.f;
            v.y = left > 1 ? v.y : 0.f;
            v.z = left > 2 ? v.z : 0.f;
            v.w = left > 3 ? v.w : 0.f;
            ra[S][P] = v;
        } else if constexpr (FT != 0) {
            constexpr int Q = P - A_SLOTS;
            const int nv = (k_mask + b_row[Q] < kend) ? b_nvalid[Q] : 0;
            v4f v = rb[S][Q];
            v.x = nv > 0 ? v.x : 0.f;
            v.y = nv > 1 ? v.y : 0.f;
            v.z = nv > 2 ? v.z : 0.f;
            v.w = nv > 3 ? v.w : 0.f;
            rb[S][Q] = v;
        }
    };
    // After the last part of a K step: move to the next one, unless that would leave the slice; then the
    // descriptors are emptied, so the fetches that run ahead past the end all return 0 (never multiplied, and
    // neutral for the checksums).
    auto gload_advance_bulk = [&]() __attribute__((always_inline)) {  // kLazyBounds, a step that is not the slice's last: no end to look out for
        if constexpr (TA) a_base += a_step;
        else a_base += BK;
        b_base += b_step;
        k_loaded += BK;
    };
    // kLazyBounds, at the end of the bulk steps: the byte counts from the current bases to the ends of A and B
    auto bounds_from_position = [&]() __attribute__((always_inline)) {
        a_left = a_bytes_left(k_loaded);
        b_left = (static_cast<int64_t>(p.K - 1 - k_loaded) * p.ldb + (p.N - n0)) * 4;
    };
    auto gload_advance = [&]() __attribute__((always_inline)) {
        const bool more = k_loaded + BK < kend;
        if constexpr (TA) {
            // the bases move on regardless (an emptied descriptor returns 0 wherever it starts): with both steps
            // held in registers the compiler would otherwise branch around the updates, and the branch would cut
            // the K step's instruction schedule in two
            a_base += a_step;
            b_base += b_step;
            a_left = more ? a_left - a_step * 4 : 0;
            b_left = more ? b_left - b_step * 4 : 0;
        } else {
            // (statement for statement what the untransposed kernels were tuned with: whether the compiler keeps
            // these as scalar selects or branches around them hangs on their exact form)
            a_base += more ? BK : 0;
            a_left = more ? a_left - BK * 4 : 0;
            b_base += more ? b_step : 0;
            b_left = more ? b_left - b_step * 4 : 0;
        }
        k_loaded += more ? BK : 0;
        if constexpr (FT >= 2) enc_off += BK * 4;
    };
    // The same in two parts, so that the short-step schedule can place them apart.  Its full tiles keep no bounds at
    // all: nothing they fetch lies outside the matrix, and past the end of the slice they fetch its last K step
    // again instead of zeros.
    auto gload_advance_a_bulk = [&]() __attribute__((always_inline)) {
        if constexpr (TA) a_base += a_step;
        else a_base += BK;
    };
    auto gload_advance_b_bulk = [&]() __attribute__((always_inline)) {
        b_base += b_step;
        k_loaded += BK;
    };
    auto gload_advance_a = [&]() __attribute__((always_inline)) {
        const bool more = k_loaded + BK < kend;
        if constexpr (TA) {
            a_base += more ? a_step : 0;
            if constexpr (!kNoBounds) a_left = more ? a_left - a_step * 4 : 0;
        } else {
            a_base += more ? BK : 0;
            if constexpr (!kNoBounds) a_left = more ? a_left - BK * 4 : 0;
        }
    };
    auto gload_advance_b = [&]() __attribute__((always_inline)) {
        const bool more = k_loaded + BK < kend;
        b_base += more ? b_step : 0;
        if constexpr (!kNoBounds) b_left = more ? b_left - b_step * 4 : 0;
        k_loaded += more ? BK : 0;
    };
    auto lstore1 = [&](auto slot, auto part, int stage) __attribute__((always_inline)) {
        constexpr int S = decltype(slot)::value, P = decltype(part)::value;
        if constexpr (P < A_SLOTS && TA) {
            float* const dst = As + stage * A_STAGE + a_lds[P];
            dst[0] = ra[S][P].x;
            dst[AS] = ra[S][P].y;
            dst[2 * AS] = ra[S][P].z;
            dst[3 * AS] = ra[S][P].w;
        } else if constexpr (P < A_SLOTS)
            *reinterpret_cast<v4f*>(As + stage * A_STAGE + a_lds[P]) = ra[S][P];
        else
            *reinterpret_cast<v4f*>(Bs + stage * B_STAGE + b_lds[P - A_SLOTS]) = rb[S][P - A_SLOTS];
    };

    // CADENCE: point the staging state at the start of the next verification interval [kbeg, kend)
    auto k_range_reset = [&]() __attribute__((always_inline)) {
        a_base = a_origin(kbeg);
        b_base = p.B + static_cast<int64_t>(kbeg) * p.ldb + n0;
        a_left = a_bytes_left(kbeg);
        b_left = (static_cast<int64_t>(p.K - 1 - kbeg) * p.ldb + (p.N - n0)) * 4;
        k_loaded = kbeg;
        k_mask = kbeg;
        enc_off = kbeg * 4;
    };

    // ---- LDS -> fragment registers -> MFMA
    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    v4f fa[2][TM];  // fragment buffer b holds the operands of half K step g = b
    float fb[2][TN][4];
    const int a_frag_off = (wm * WM + lr) * AS + lh * 4;
    const int b_frag_off = (lh * 4) * BS + wn * WN + lr;

    auto fread1 = [&](auto buf, auto part, int stage, int g) __attribute__((always_inline)) {  // part < TM: A block `part`; else B block `part - TM`
        constexpr int Bf = decltype(buf)::value, P = decltype(part)::value;
        if constexpr (P < TM) {
            fa[Bf][P] = *reinterpret_cast<const v4f*>(As + stage * A_STAGE + a_frag_off + g * 8 + P * 32 * AS);
        } else {
            constexpr int j = P - TM;
            const float* bs = Bs + stage * B_STAGE + b_frag_off + g * 8 * BS + j * 32;
#pragma unroll
            for (int q = 0; q < 4; ++q) fb[Bf][j][q] = bs[q * BS];
        }
    };
    auto mfma1 = [&](auto buf, auto idx) __attribute__((always_inline)) {
        constexpr int Bf = decltype(buf)::value, I = decltype(idx)::value;
        constexpr int q = I / (TM * TN), i = (I / TN) % TM, j = I % TN;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[Bf][i][q], fb[Bf][j][q], acc[i][j], 0, 0, 0);
    };

    // ---- ABFT encode (dead code when FT == 0).
    // Like the reference, which forms e^T A and B e on its global->shared staging registers with warp shuffles
    // and adds the rank-1 products into spare shared memory (kernel/ft_sgemm/include/ft_sgemm_huge.cuh:442-474),
    // the checksums are encoded from the staging registers of K step t+1 while step t is being multiplied:
    //   before the barrier ("produce", FT == 1 only): this thread holds 4 k values of A_SLOTS rows and 4 columns
    //     of B_SLOTS k rows.  Column sums of A over the tile's rows: in-thread over the slots, then over the 16
    //     lanes of the wave that hold the same k group (row_ror 4, 8; swap with lane^16; swap with lane^32) ->
    //     one partial per wave in LDS.  Row sums of B over the tile's columns: in-thread over the 4 columns, then
    //     over the 32 lanes of the half wave (which holds whole k rows) -> b_r[k] in LDS.
    //   after the barrier ("consume"): a_c[k] = sum of the per-wave partials for the thread's own k rows (FT == 2:
    //     fetched from the pre-encoded vectors with the staged tile), cc[n] += a_c[k] * B[k, n] on its B
    //     registers; b_r[k] for its own 4 k values, cr[m] += A[m, k] * b_r[k] on its A registers.  Partial sums
    //     are FP32 over 16 K steps, then added to FP64 running sums, so the reference checksums carry no drift
    //     of their own over a long K.
    // Per thread the running sums cover columns nc..nc+3 over the k rows it stages (8 threads share a column)
    // and rows row(s) over the k group it stages (4 threads share a row); the verification step adds them up.
    constexpr int kHalfWaves = kGemmThreads / B_V4_PER_ROW;  // threads that share a column of the B tile = k rows staged per slot
    constexpr int kParts = kGemmThreads / kWave;          // column-sum partials per k: one per wave
    constexpr int kPartV4 = kParts / 4;                   // 16-byte groups of them
    static_assert(!FT || (A_V4_PER_ROW == 4 && (B_V4_PER_ROW == 32 || B_V4_PER_ROW == 16)), "ABFT encode is laid out for 128- and 64-column tiles");
    static_assert(!FT || kHalfWaves * B_SLOTS == BK, "the threads of a column group stage the 16 k rows between them");
    float* const s_apart = smem + 2 * (A_STAGE + B_STAGE);          // [2][16 k][waves]
    float* const s_br = s_apart + 2 * BK * kParts;                  // [2][16 k]
    float* const s_dump = s_br + 2 * BK + tid;                      // where the lanes that publish nothing write
    // destinations of this lane's publishes (parity 0); strides and the parity distance are the same for the
    // publishing lanes and the dump, so every write is base + immediate offset
    // (after the transposing reduction lane l < 16 of a wave holds the wave's column sum of k = 4 * (l % 4) + l / 4)
    // (TA: a lane stages four m of k = lane / 4, so the first lane of each quad ends up with the wave's sum of that k)
    float* const pub_a = TA ? ((lane & 3) == 0 ? s_apart + (lane >> 2) * kParts + wave : s_dump)
                            : (lane < 16) ? s_apart + (4 * (tid & 3) + (lane >> 2)) * kParts + wave : s_dump;
    float* const pub_b = (tid % B_V4_PER_ROW < B_SLOTS) ? s_br + tid / B_V4_PER_ROW + kHalfWaves * (tid % B_V4_PER_ROW) : s_dump;
    const int x32_addr = (lane ^ 32) * 4;  // ds_bpermute address of the partner lane in the other half wave
    // With wave-tile checksums a thread keeps one column sum per wave row gm (its columns lie in one wave column)
    // and one row sum per wave column gn (its rows lie in one wave row).
    double cc_ref[GM][4], cr_ref[GN][A_SLOTS];
    float cc_lo[GM][B_SLOTS][4], cr_lo[GN][A_SLOTS][4];  // FP32 partials of the running sums, one per staged element
#pragma unroll
    for (int gm = 0; gm < GM; ++gm)
#pragma unroll
        for (int e = 0; e < 4; ++e) cc_ref[gm][e] = 0.0;
#pragma unroll
    for (int gn = 0; gn < GN; ++gn)
#pragma unroll
        for (int sl = 0; sl < A_SLOTS; ++sl) cr_ref[gn][sl] = 0.0;
#pragma unroll
    for (int gm = 0; gm < GM; ++gm)
#pragma unroll
        for (int sl = 0; sl < B_SLOTS; ++sl)
#pragma unroll
            for (int e = 0; e < 4; ++e) cc_lo[gm][sl][e] = 0.f;
#pragma unroll
    for (int gn = 0; gn < GN; ++gn)
#pragma unroll
        for (int sl = 0; sl < A_SLOTS; ++sl)
#pragma unroll
            for (int e = 0; e < 4; ++e) cr_lo[gn][sl][e] = 0.f;
    float e_pa[4], e_sw[4];
    v4f e_t[kPartV4 * B_SLOTS], e_brv[GN];
    v4f e_a[TA ? A_SLOTS : 1];  // TA: this thread's rows of the staged K step (four k each), read back from LDS
    float e_pb0, e_pb1, e_pk, e_swb, e_ac[GM][B_SLOTS];
    const int e_hw = tid / B_V4_PER_ROW;  // first k row this thread stages of B (a half wave per row of a 128-column tile)
    const int e_class = tid & 3;         // k group (4 k values) this thread stages of A
    constexpr int NPROD = (FT == 1) ? 11 : 0;  // pieces before the barrier
    // pieces after the barrier: fetch, combine (FT == 1), column checksums (one piece per wave row), row checksums
    // (one piece per wave column; two halves of the staged rows with one checksum pair per tile), flush
    constexpr int NCR = GRAN ? GN : 2;
    constexpr int NCONS = FT ? 2 + GM + NCR + 1 : 0;
    constexpr int kDppRor4 = 0x124, kDppRor8 = 0x128;  // rotate right inside each row of 16 lanes

    auto produce1 = [&](auto slot, auto piece, int par) __attribute__((always_inline)) {
        constexpr int S = decltype(slot)::value, E = decltype(piece)::value;
        if constexpr (TA && E <= 3) {
            // column sums of A^T's staged K step: a lane holds four m of one k per slot, the four lanes of a quad
            // the wave's sixteen m-groups of that k between them
            if constexpr (E == 0) {
                v4f t = ra[S][0];
#pragma unroll
                for (int sl = 1; sl < A_SLOTS; ++sl) t += ra[S][sl];
                e_pa[0] = (t.x + t.y) + (t.z + t.w);
                HPCDNN_PIN(e_pa[0]);
            } else if constexpr (E == 1) {
                e_pa[0] += dpp_mov<kDppXor1>(e_pa[0]);
                HPCDNN_PIN(e_pa[0]);
            } else if constexpr (E == 2) {
                e_pa[0] += dpp_mov<kDppXor2>(e_pa[0]);
                HPCDNN_PIN(e_pa[0]);
            }
        } else if constexpr (E == 0) {
            v4f t = ra[S][0];
#pragma unroll
            for (int sl = 1; sl < A_SLOTS; ++sl) t += ra[S][sl];
            e_pa[0] = t.x; e_pa[1] = t.y; e_pa[2] = t.z; e_pa[3] = t.w;
#pragma unroll
            for (int e = 0; e < 4; ++e) HPCDNN_PIN(e_pa[e]);
        } else if constexpr (E == 1) {
            // The four k values of a lane are summed over the 16 lanes of the wave that hold the same k group (lane
            // bits 2 .. 5) by a transposing reduction: lane bit 2 decides which value of a pair stays and which
            // travels to lane ^ 4, bit 3 likewise for the two that are left, then plain exchanges with lane ^ 16 and
            // lane ^ 32.  One value per lane is left after two stages, so the whole costs 5 additions and 6 selects
            // where four separate reductions cost 16 additions.
            const bool up = lane & 4;
            const float s0 = up ? e_pa[0] : e_pa[1], s1 = up ? e_pa[2] : e_pa[3];
            e_pa[0] = up ? e_pa[1] : e_pa[0];
            e_pa[1] = up ? e_pa[3] : e_pa[2];
            e_sw[0] = lane_xor<4>(s0);
            e_sw[1] = lane_xor<4>(s1);
        } else if constexpr (E == 2) {
            e_pa[0] += e_sw[0];
            e_pa[1] += e_sw[1];
            const bool up = lane & 8;
            const float s0 = up ? e_pa[0] : e_pa[1];
            e_pa[0] = up ? e_pa[1] : e_pa[0];
            e_sw[0] = lane_xor<8>(s0);
        } else if constexpr (E == 3) {
            e_pa[0] += e_sw[0];
            e_sw[0] = lane_xor<16>(e_pa[0]);
        } else if constexpr (kLazyRows && E >= 4 && E <= 7) {
            // (the row sums of B are formed in the verification, when a column is flagged)
        } else if constexpr (E == 4) {
            // row sums of B: in-thread over the 4 columns, first butterfly step for each staged k row ...
            e_pb0 = (rb[S][0].x + rb[S][0].y) + (rb[S][0].z + rb[S][0].w);
            e_pb0 += dpp_mov<kDppXor1>(e_pb0);
            HPCDNN_PIN(e_pb0);
            if constexpr (B_SLOTS == 2) {
                e_pb1 = (rb[S][B_SLOTS - 1].x + rb[S][B_SLOTS - 1].y) + (rb[S][B_SLOTS - 1].z + rb[S][B_SLOTS - 1].w);
                e_pb1 += dpp_mov<kDppXor1>(e_pb1);
                HPCDNN_PIN(e_pb1);
            }
        } else if constexpr (E == 5) {
            // ... then the two k rows share one register (even lanes carry row 0, odd lanes row 1) and the
            // remaining steps, which keep lane parity, reduce both at once
            static_assert(B_SLOTS <= 2, "two staged k rows are packed by lane parity");
            e_pk = e_pb0;
            if constexpr (B_SLOTS == 2) e_pk = (lane & 1) ? e_pb1 : e_pb0;
            e_pk += dpp_mov<kDppXor2>(e_pk);
            HPCDNN_PIN(e_pk);
        } else if constexpr (E == 6) {
            e_pk += dpp_mov<kDppRor4>(e_pk);
            e_pk += dpp_mov<kDppRor8>(e_pk);
            HPCDNN_PIN(e_pk);
        } else if constexpr (E == 7) {
            // a k row of a 64-column tile lies in one row of 16 lanes and is complete here
            if constexpr (B_V4_PER_ROW == 32) e_swb = __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, e_pk), 0x401F));
        } else if constexpr (E == 8) {
            if constexpr (!TA) {
                e_pa[0] += e_sw[0];
                e_sw[0] = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(x32_addr, __builtin_bit_cast(int, e_pa[0])));
            }
            if constexpr (!kLazyRows) {
                if constexpr (B_V4_PER_ROW == 32) e_pk += e_swb;
                HPCDNN_PIN(e_pk);
            }
        } else if constexpr (E == 9) {
            if constexpr (!TA) e_pa[0] += e_sw[0];  // sum over the whole wave
            HPCDNN_PIN(e_pa[0]);
        } else {
            // lanes 0..15 of each wave publish the 16 column sums, the first lane (or two) of each k row of B its row sum;
            // the other lanes write to their dump word, which keeps the loop free of branches
            *(pub_a + par * (BK * kParts)) = e_pa[0];
            if constexpr (!kLazyRows) *(pub_b + par * BK) = e_pk;
        }
    };
    bool flush_now = true;  // uniform; set by the main loop before each K step that may flush
    auto consume1 = [&](auto slot, auto piece, int par, auto flush) __attribute__((always_inline)) {
        constexpr int S = decltype(slot)::value, E = decltype(piece)::value;
        constexpr bool kFlush = decltype(flush)::value;
        const float* ap = s_apart + par * BK * kParts;
        const float* br = s_br + par * BK;
        if constexpr (FT >= 2 && E <= 1) {
            if constexpr (E == 0) {
                if constexpr (FT == 2) {
#pragma unroll
                    for (int gm = 0; gm < GM; ++gm)
#pragma unroll
                        for (int sl = 0; sl < B_SLOTS; ++sl) e_ac[gm][sl] = g_ac[S][gm][sl];
                }
                if constexpr (!kLazyRows) {
#pragma unroll
                    for (int gn = 0; gn < GN; ++gn) e_brv[gn] = g_br[S][gn];
                    // (the barrier before the second half has made stage `par`, which holds this K step, complete)
                    if constexpr (TA) {
#pragma unroll
                        for (int sl = 0; sl < A_SLOTS; ++sl) e_a[sl] = *reinterpret_cast<const v4f*>(As + par * A_STAGE + a_lds_rows[sl]);
                    }
                }
            }
        } else if constexpr (E == 0) {
#pragma unroll
            for (int sl = 0; sl < B_SLOTS; ++sl) {
                const float* row = ap + (e_hw + kHalfWaves * sl) * kParts;
#pragma unroll
                for (int v = 0; v < kPartV4; ++v) e_t[kPartV4 * sl + v] = *reinterpret_cast<const v4f*>(row + 4 * v);
            }
            if constexpr (!kLazyRows) {
                e_brv[0] = *reinterpret_cast<const v4f*>(br + 4 * e_class);
                if constexpr (TA) {
#pragma unroll
                    for (int sl = 0; sl < A_SLOTS; ++sl) e_a[sl] = *reinterpret_cast<const v4f*>(As + par * A_STAGE + a_lds_rows[sl]);
                }
            }
        } else if constexpr (E == 1) {
#pragma unroll
            for (int sl = 0; sl < B_SLOTS; ++sl) {
                v4f u = e_t[kPartV4 * sl];
#pragma unroll
                for (int v = 1; v < kPartV4; ++v) u += e_t[kPartV4 * sl + v];
                e_ac[0][sl] = (u.x + u.y) + (u.z + u.w);
                HPCDNN_PIN(e_ac[0][sl]);
            }
        } else if constexpr (kWeighted && E < 2 + GM) {
            // (no column checksums, and the weighted row checksum of a row is formed only once the row is flagged)
        } else if constexpr (E < 2 + GM) {
            // independent accumulators: a wave alone on its SIMD cannot hide the latency of dependent VALU
            // instructions behind other waves
            constexpr int gm = E - 2;
#pragma unroll
            for (int sl = 0; sl < B_SLOTS; ++sl) {
                cc_lo[gm][sl][0] = __builtin_fmaf(e_ac[gm][sl], rb[S][sl].x, cc_lo[gm][sl][0]);
                cc_lo[gm][sl][1] = __builtin_fmaf(e_ac[gm][sl], rb[S][sl].y, cc_lo[gm][sl][1]);
                cc_lo[gm][sl][2] = __builtin_fmaf(e_ac[gm][sl], rb[S][sl].z, cc_lo[gm][sl][2]);
                cc_lo[gm][sl][3] = __builtin_fmaf(e_ac[gm][sl], rb[S][sl].w, cc_lo[gm][sl][3]);
            }
#pragma unroll
            for (int sl = 0; sl < B_SLOTS; ++sl)
#pragma unroll
                for (int e = 0; e < 4; ++e) HPCDNN_PIN(cc_lo[gm][sl][e]);
        } else if constexpr (kLazyRows && E < 2 + GM + NCR) {
            // (the row references are formed in the verification, when a column is flagged)
        } else if constexpr (E < 2 + GM + NCR) {
            constexpr int piece = E - 2 - GM;
            constexpr int gn = GRAN ? piece : 0;
            constexpr int lo = GRAN ? 0 : (piece == 0 ? 0 : A_SLOTS / 2), hi = GRAN ? A_SLOTS : (piece == 0 ? A_SLOTS / 2 : A_SLOTS);
#pragma unroll
            for (int sl = lo; sl < hi; ++sl) {
                const v4f av = TA ? e_a[TA ? sl : 0] : ra[S][sl];
                cr_lo[gn][sl][0] = __builtin_fmaf(av.x, e_brv[gn].x, cr_lo[gn][sl][0]);
                cr_lo[gn][sl][1] = __builtin_fmaf(av.y, e_brv[gn].y, cr_lo[gn][sl][1]);
                cr_lo[gn][sl][2] = __builtin_fmaf(av.z, e_brv[gn].z, cr_lo[gn][sl][2]);
                cr_lo[gn][sl][3] = __builtin_fmaf(av.w, e_brv[gn].w, cr_lo[gn][sl][3]);
            }
#pragma unroll
            for (int sl = lo; sl < hi; ++sl)
#pragma unroll
                for (int e = 0; e < 4; ++e) HPCDNN_PIN(cr_lo[gn][sl][e]);
        } else if constexpr (kFlush) {
            // every 16th K step (and after the last one): FP32 partials -> FP64 running sums.  FP64 VALU
            // instructions are twice as expensive as FP32 ones, so this is kept rare.
            if (flush_now) {
#pragma unroll
                for (int gm = 0; gm < (kWeighted ? 0 : GM); ++gm)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float t = cc_lo[gm][0][e];
#pragma unroll
                        for (int sl = 1; sl < B_SLOTS; ++sl) t += cc_lo[gm][sl][e];
                        cc_ref[gm][e] += static_cast<double>(t);
#pragma unroll
                        for (int sl = 0; sl < B_SLOTS; ++sl) cc_lo[gm][sl][e] = 0.f;
                    }
#pragma unroll
                for (int gn = 0; gn < (kLazyRows ? 0 : GN); ++gn)
#pragma unroll
                    for (int sl = 0; sl < A_SLOTS; ++sl) {
                        cr_ref[gn][sl] += static_cast<double>((cr_lo[gn][sl][0] + cr_lo[gn][sl][1]) + (cr_lo[gn][sl][2] + cr_lo[gn][sl][3]));
#pragma unroll
                        for (int e = 0; e < 4; ++e) cr_lo[gn][sl][e] = 0.f;
                    }
            }
        }
    };

    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;

    // One K step.  On entry: LDS stage kt&1 holds step kt, fragment buffer 0 holds its first half, staging slot
    // `sl_next` holds step kt+1 (possibly still in flight), slot `sl_free` is free.
    //   first half : MFMAs on buffer 0 | read second-half fragments into buffer 1, fetch step kt+2 into sl_free,
    //                write step kt+1 from sl_next into the other LDS stage (+ produce its checksum partials)
    //   barrier    : the other stage is complete; nobody reads this stage's fragments any more
    //   second half: MFMAs on buffer 1 | read the first-half fragments of step kt+1 into buffer 0
    //                (+ consume the checksum partials of step kt+1)
    // Work past the end of the slice (kt+1, kt+2 >= nkt) moves duplicate data that is never multiplied, which
    // keeps the loop free of branches (and lets the loads stay two steps ahead).
    auto step_in = [&](auto sl_next, auto sl_free, auto stage, auto flush, auto masked, auto bulk) __attribute__((always_inline)) {
        constexpr int st = decltype(stage)::value;
        constexpr bool kBulk = kLazyBounds && decltype(bulk)::value;
        constexpr int NMASK = (EDGE && decltype(masked)::value) ? (FT ? NGL : A_SLOTS) : 0;
        constexpr int NS0 = NRD + NMASK + NPROD + 2 * NGL;
        constexpr int NS1 = NRD + NCONS;
        // A wave with few MFMAs per half step (one or two 32x32 blocks) has little to hide latencies behind: its
        // second half reads the next step's fragments right behind the first MFMA (the next step starts with them),
        // and the scalar arithmetic that moves the descriptors on goes behind the second one instead of joining
        // the loads and LDS writes of the first half (a wave alone on its SIMD pays for clumps of scalar work).
        static_for<NMG>([&](auto m) {
            constexpr int Mi = decltype(m)::value;
            mfma1(S0{}, m);
            // side ops k_lo .. k_hi-1 of NS0 go behind MFMA Mi: fragment reads first (needed soonest), then
            // loads, LDS writes, and last the checksum pieces (they need the same staged data as the LDS writes)
            constexpr int k_lo = (Mi * NS0 + NMG - 1) / NMG, k_hi = ((Mi + 1) * NS0 + NMG - 1) / NMG;
            static_for<k_hi - k_lo>([&](auto d) {
                constexpr int o = k_lo + decltype(d)::value;
                // order: fragment reads (needed soonest); ragged-tile masks and checksum pieces of step kt+1 (its
                // staged data arrived a step ago; the cross-lane chain must be finished well before the barrier);
                // global loads of step kt+2; LDS writes of step kt+1
                if constexpr (kEarlyStore) {
                    // deep staging: the data of step kt+1 arrived steps ago, so its LDS writes go first and are
                    // complete long before the barrier; the loads of the step furthest ahead follow
                    if constexpr (o < NRD) fread1(S1{}, std::integral_constant<int, o>{}, st, 1);
                    else if constexpr (o < NRD + NMASK) gmask1(sl_next, std::integral_constant<int, o - NRD>{});
                    else if constexpr (o < NRD + NMASK + NGL) lstore1(sl_next, std::integral_constant<int, o - NRD - NMASK>{}, st ^ 1);
                    else gload1(sl_free, std::integral_constant<int, o - NRD - NMASK - NGL>{}, bulk);
                } else if constexpr (o < NRD) {
                    fread1(S1{}, std::integral_constant<int, o>{}, st, 1);
                } else if constexpr (o < NRD + NMASK) {
                    gmask1(sl_next, std::integral_constant<int, o - NRD>{});
                } else if constexpr (o < NRD + NMASK + NPROD) {
                    produce1(sl_next, std::integral_constant<int, o - NRD - NMASK>{}, st ^ 1);
                } else if constexpr (o < NRD + NMASK + NPROD + NGL) {
                    gload1(sl_free, std::integral_constant<int, o - NRD - NMASK - NPROD>{}, bulk);
                    if constexpr (o == NRD + NMASK + NPROD + NGL - 1 && !kShortStep) {
                        if constexpr (kBulk) gload_advance_bulk();
                        else gload_advance();
                    }
                } else {
                    lstore1(sl_next, std::integral_constant<int, o - NRD - NMASK - NPROD - NGL>{}, st ^ 1);
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
        if constexpr (EDGE) k_mask += BK;  // the next step's masks belong to the K step after this one's successor
        __builtin_amdgcn_sched_barrier(0);
        static_for<NMG>([&](auto m) {
            constexpr int Mi = decltype(m)::value;
            mfma1(S1{}, m);
            if constexpr (kShortStep) {
                if constexpr (Mi == 0) static_for<NRD>([&](auto o) { fread1(S0{}, o, st ^ 1, 0); });
                if constexpr (Mi == 1) {
                    if constexpr (kBulk) gload_advance_a_bulk();
                    else gload_advance_a();
                }
                if constexpr (Mi == 2) {
                    if constexpr (kBulk) gload_advance_b_bulk();
                    else gload_advance_b();
                }
            } else {
                constexpr int k_lo = (Mi * NS1 + NMG - 1) / NMG, k_hi = ((Mi + 1) * NS1 + NMG - 1) / NMG;
                static_for<k_hi - k_lo>([&](auto d) {
                    constexpr int o = k_lo + decltype(d)::value;
                    // fragment reads first (the next step's first MFMAs wait for them), then the checksum pieces
                    if constexpr (o < NRD) fread1(S0{}, std::integral_constant<int, o>{}, st ^ 1, 0);
                    else consume1(sl_next, std::integral_constant<int, o - NRD>{}, st ^ 1, flush);
                });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // with two staging sets steps alternate between (next = slot 1, LDS stage 0) and (next = slot 0, LDS stage 1)
    auto step = [&](auto sl_next, auto sl_free, auto flush, auto masked, auto bulk) __attribute__((always_inline)) {
        step_in(sl_next, sl_free, std::integral_constant<int, (decltype(sl_next)::value == 1) ? 0 : 1>{}, flush, masked, bulk);
    };
    // step number kt with kt % NSLOT == phase: its successor waits in slot (phase + 1) % NSLOT, slot phase is free
    auto step_at = [&](auto phase, auto masked, auto bulk, auto flush) __attribute__((always_inline)) {
        constexpr int Ph = decltype(phase)::value;
        step_in(std::integral_constant<int, (Ph + 1) % NSLOT>{}, std::integral_constant<int, Ph % NSLOT>{},
                std::integral_constant<int, Ph % 2>{}, flush, masked, bulk);
    };

    // One pass of the software pipeline over [kbeg, kend).
    auto run_k_range = [&]() {
    if (nkt > 0) {
        // prologue: step 0 -> LDS stage 0, step 1 -> staging slot 1, first-half fragments of step 0 -> buffer 0
        static_for<NGL>([&](auto s) { gload1(S0{}, s, std::false_type{}); });
        gload_advance();
        if constexpr (EDGE) static_for<NGL>([&](auto s) { gmask1(S0{}, s); });
        if constexpr (EDGE) k_mask += BK;
        static_for<NGL>([&](auto s) { lstore1(S0{}, s, 0); });
        static_for<NPROD>([&](auto e) { produce1(S0{}, e, 0); });
        static_for<NGL>([&](auto s) { gload1(S1{}, s, std::false_type{}); });
        gload_advance();
        static_for<NSLOT - 2>([&](auto extra) {  // steps 2 .. NSLOT-1 -> their slots
            static_for<NGL>([&](auto s) { gload1(std::integral_constant<int, decltype(extra)::value + 2>{}, s, std::false_type{}); });
            gload_advance();
        });
        __syncthreads();
        static_for<NCONS>([&](auto e) { consume1(S0{}, e, 0, std::true_type{}); });
        static_for<NRD>([&](auto s) { fread1(S0{}, s, 0, 0); });
        int kt = 0;
        if constexpr (NSLOT > 2) {
            // whole groups of NSLOT steps; on a ragged tile only the slice's last K step can be partial, and it is
            // step nkt - 2 that moves it to LDS, so the steps before that one run without the masks
            const int bulk_end = EDGE ? nkt - 2 : nkt;
            if constexpr (kLazyBounds) {
                // groups whose loads (NSLOT steps ahead) all stay before the slice's last K step
                for (; lazy_ok && kt + 2 * NSLOT + 1 <= nkt; kt += NSLOT)
                    static_for<NSLOT>([&](auto ph) { step_at(ph, std::false_type{}, std::true_type{}, std::false_type{}); });
                if (kt > 0) bounds_from_position();
            }
            // (ABFT: the checksums of a ragged problem want zeros in the columns n >= N of every step, so its groups
            // run with the masks; the FP32 partial sums are flushed with the last step of every fourth group of four)
            for (; kt + NSLOT <= bulk_end; kt += NSLOT) {
                if constexpr (FT != 0) flush_now = (kt & 12) == 12;
                static_for<NSLOT>([&](auto ph) {
                    step_at(ph, std::integral_constant<bool, EDGE && FT != 0>{}, std::false_type{},
                            std::integral_constant<bool, FT != 0 && decltype(ph)::value == NSLOT - 1>{});
                });
            }
            // what is left (fewer than a group, plus the two last steps of a ragged tile), one step at a time
            flush_now = true;
            static_for<NSLOT + (EDGE ? 1 : -1)>([&](auto i) {
                if (kt + decltype(i)::value < nkt)
                    step_at(std::integral_constant<int, decltype(i)::value % NSLOT>{}, std::true_type{}, std::false_type{},
                            std::integral_constant<bool, FT != 0>{});
            });
        } else {
            if constexpr (EDGE && FT == 0) {
                // plain SGEMM on a ragged tile: only the last K step can be partial, and step kt consumes the staged
                // data of step kt+1, so every step before kt = nkt-2 runs without the masks
                // pairs whose loads (two steps ahead) both stay before the slice's last K step
                for (; lazy_ok && kt + 4 < nkt; kt += 2) {
                    step(S1{}, S0{}, std::false_type{}, std::false_type{}, std::true_type{});
                    step(S0{}, S1{}, std::false_type{}, std::false_type{}, std::true_type{});
                }
                if (kt > 0) bounds_from_position();
                for (; kt + 3 < nkt; kt += 2) {
                    step(S1{}, S0{}, std::false_type{}, std::false_type{}, std::false_type{});
                    step(S0{}, S1{}, std::false_type{}, std::false_type{}, std::false_type{});
                }
            }
            if constexpr (EDGE && FT != 0) {
                // ABFT on a ragged problem: a tile that does not hang over the last column needs the masks only where
                // plain SGEMM does, in the slice's last two K steps (its checksums want zeros in columns k >= kend of
                // A and rows k >= kend of B; the columns n >= N that the other steps would have to clear do not exist).
                // With pre-encoded vectors a tile that does hang over runs the same way: what its columns n >= N (TA:
                // rows m >= M) pick up reaches only their own accumulators and reference sums, and the verification
                // clears those before it looks at anything (kLazyOutside).
                if (kLazyOutside || (n0 + BN <= p.N && (!TA || m0 + BM <= p.M))) {
                    for (; kt + 3 < nkt; kt += 2) {
                        step(S1{}, S0{}, std::false_type{}, std::false_type{}, std::false_type{});
                        flush_now = (kt & 14) == 14;
                        step(S0{}, S1{}, std::true_type{}, std::false_type{}, std::false_type{});
                    }
                }
            }
            for (; kt + 1 < nkt; kt += 2) {
                step(S1{}, S0{}, std::false_type{}, std::true_type{}, std::false_type{});
                flush_now = ((kt & 14) == 14) || (kt + 2 >= nkt);
                step(S0{}, S1{}, std::true_type{}, std::true_type{}, std::false_type{});
            }
            flush_now = true;
            if (kt < nkt) step(S1{}, S0{}, std::true_type{}, std::true_type{}, std::false_type{});
        }
        __syncthreads();  // every wave is done with the staging buffers (the verification below reuses them)
    }
    };

    if constexpr (FT == 0) {
        run_k_range();
    } else {
    // the tile's epilogue as a function: these kernels call it before or after their last verification (early_store)
    auto store_c = [&]() __attribute__((always_inline)) {
        const int row_base = m0 + wm * WM + lh * 4;  // + i*32 + 8*(v/4) + v%4
        const int col_base = n0 + wn * WN + lr;      // + j*32
        // C = alpha*acc + beta*C.  With beta != 0 the 16 old values of a 32x32 block are fetched together before the
        // first store, so that their latencies overlap instead of queueing behind each other.
        // Tiles of at most 128x128 store C with the streaming hint: many small workgroups finish close together, and
        // keeping their output out of the L2 leaves it to the operand panels (1 to 2 % on 1024^3, 2048^3, 4096x4096x256;
        // the 256x128 tiles measured 0.2 % slower with it and keep the plain store).
        constexpr bool kStreamC = BM * BN <= 128 * 128;
        const float alpha = p.alpha, beta = p.beta;
        if constexpr (EDGE) {
            // Ragged tiles: a buffer descriptor from the tile's corner to the last element of C inside the tile, so the
            // hardware drops stores to rows >= M (and returns 0 for loads there); the row offset has to be part of the
            // vector offset for that (a scalar offset is not range-checked).  Columns >= N would land in the next row:
            // they are switched off once per block column.  A compare, a branch and a 64-bit multiply per store, which
            // is what the pointer form compiles to, cost a 64x64 tile 3200 cycles here.
            const int64_t c_bytes = (static_cast<int64_t>(p.M - 1 - m0) * p.ldc + (p.N - n0)) * 4;
            const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc(p.C + static_cast<int64_t>(m0) * p.ldc + n0, c_bytes);
            const int ldc_bytes = p.ldc * 4;  // BM * ldc * 4 < 2^31 (host check)
            const int lane_off = (wm * WM + lh * 4) * ldc_bytes + (wn * WN + lr) * 4;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (col_base + j * 32 >= p.N) continue;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    float old[16];
                    if (beta != 0.f) {
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            old[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                         c_rsrc, lane_off + j * 128 + (i * 32 + 8 * (v / 4) + (v % 4)) * ldc_bytes, 0, 0));
                    }
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const float t = alpha * acc[i][j][v];
                        const float out = (beta == 0.f) ? t : __builtin_fmaf(beta, old[v], t);
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, out), c_rsrc,
                                                              lane_off + j * 128 + (i * 32 + 8 * (v / 4) + (v % 4)) * ldc_bytes, 0,
                                                              kStreamC ? 2 : 0);
                    }
                }
            }
        } else {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = col_base + j * 32;
                float* cbase = p.C + static_cast<size_t>(row_base + i * 32) * p.ldc + col;
                float old[16];
                if (beta != 0.f) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int r = 8 * (v / 4) + (v % 4);
                        old[v] = cbase[static_cast<size_t>(r) * p.ldc];
                    }
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = 8 * (v / 4) + (v % 4);
                    const float t = alpha * acc[i][j][v];
                    const float out = (beta == 0.f) ? t : __builtin_fmaf(beta, old[v], t);
                    if constexpr (kStreamC) __builtin_nontemporal_store(out, &cbase[static_cast<size_t>(r) * p.ldc]);
                    else cbase[static_cast<size_t>(r) * p.ldc] = out;
                }
            }
        }
    };

    // ---- ABFT verification: inject (testing aid), observe, compare, locate, correct, re-synchronise
    constexpr int CCP = kHalfWaves, CRP = A_V4_PER_ROW;   // partials per column / per row checksum
    constexpr int NCT = GM * GN;                          // check tiles per workgroup tile
    constexpr int kRowLines = GN * BM;                    // row lines (gn, m) come first, column lines (gm, n) after them
    // (row-screen kernels: the BM row lines, then the weighted residual of a flagged row or the BN column lines)
    constexpr int kLines = kWeighted ? BM + (BM > BN ? BM : BN) : kRowLines + GM * BN;
    // lines per thread in the pass over the column lines and in the pass over the row lines
    constexpr int kColPass = kWeighted ? 0 : GM * BN, kRowPass = kRowLines;
    constexpr int LPT_C = (kColPass + kGemmThreads - 1) / kGemmThreads > 0 ? (kColPass + kGemmThreads - 1) / kGemmThreads : 1;
    constexpr int LPT_R = (kRowPass + kGemmThreads - 1) / kGemmThreads;
    static_assert(NCT <= kGemmThreads, "one thread per check tile keeps its record");
    double off_col[LPT_C], off_row[LPT_R];  // CADENCE: what re-synchronisation has taken out of each of this thread's lines
#pragma unroll
    for (int it = 0; it < LPT_C; ++it) off_col[it] = 0.0;
#pragma unroll
    for (int it = 0; it < LPT_R; ++it) off_row[it] = 0.0;
    const int k_first = kbeg;      // first k of this workgroup's K range (kbeg moves on from interval to interval)
    // With beta == 0 the tile goes to C before its (last) verification instead of after it, so that the stores are on
    // their way while the checksums are compared; a located element is then written a second time, by its owner, with
    // the value computed again.  (With beta != 0 the old value of C that the corrected element needs is gone once the
    // tile is stored: the order stays verify, then store.  The K slices of a split tile write raw accumulators.  The
    // cadence kernels, whose verification sits in a loop, spill 100-200 registers with the stores inside it.)
    const bool early_store = !CADENCE && p.beta == 0.f && tail_out == nullptr;
    hpcdnn_ft_status rec;          // thread ct < NCT: the record of check tile ct, merged over the verifications
    rec.flag = 0; rec.row = -1; rec.col = -1; rec.n_bad_rows = 0; rec.n_bad_cols = 0;
    rec.row_residual = 0.f; rec.col_residual = 0.f; rec.max_clean_residual = 0.f;

    auto verify = [&](int check, bool last) {
        double* const s_ccref = reinterpret_cast<double*>(smem);        // [GM][CCP][BN] reference column checksum partials
        double* const s_crref = s_ccref + GM * CCP * BN;                // [GN][CRP][BM] reference row checksum partials
        float* const s_ccobs = reinterpret_cast<float*>(s_crref + GN * CRP * BM);  // [WGM][BN] observed column sums
        float* const s_crobs = s_ccobs + WGM * BN;                      // [WGN][BM] observed row sums
        float* const s_ccabs = s_crobs + WGN * BM;                      // [WGM][BN] column sums of |accumulators|
        float* const s_crabs = s_ccabs + WGM * BN;                      // [WGN][BM] row sums of |accumulators|
        float* const s_dr = s_crabs + WGN * BM;                         // [kLines] residuals
        int* const s_meta = reinterpret_cast<int*>(s_dr + kLines);      // [NCT][8] nbr, nbc, bad row, bad col, max clean (float bits)
        float* const s_tsum = reinterpret_cast<float*>(s_meta + 8 * NCT);  // [NCT][waves] partial sums of |acc| over a check tile
        float* const s_fix = s_tsum + NCT * (kGemmThreads / kWave);        // [NCT][2] recomputed element, and what it changed
        static_assert(gemm_lds_bytes<BM, BN, FT, kGemmThreads, WGM, WGN, GRAN>() >= ft_verify_lds_bytes<BM, BN, WGM, WGN, GM, GN, kWeighted>(),
                      "verification scratch fits in the kernel's LDS");
        const int tile_linear = tile_m * p.tiles_n + tile_n;

        // acc element (r, c) of the tile lives in wave (r/WM, c/WN), block (i, j), lane (c%32, (r%32/4)%2), register v
        auto add_at = [&](int r, int c, float val) {
            const int rr = r % 32;
            const int fi = (r % WM) / 32, fj = (c % WN) / 32, fv = 4 * (rr / 8) + rr % 4;
            if (wm == r / WM && wn == c / WN && lr == c % 32 && lh == (rr / 4) % 2) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (i == fi && j == fj && v == fv) acc[i][j][v] += val;
            }
        };

        // the same element set to val by its owner, who also leaves (val - old value) in *change
        auto set_at = [&](int r, int c, float val, float* change) -> float {
            const int rr = r % 32;
            const int fi = (r % WM) / 32, fj = (c % WN) / 32, fv = 4 * (rr / 8) + rr % 4;
            float old = 0.f;
            if (wm == r / WM && wn == c / WN && lr == c % 32 && lh == (rr / 4) % 2) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
#pragma unroll
                        for (int v = 0; v < 16; ++v)
                            if (i == fi && j == fj && v == fv) { old = acc[i][j][v]; acc[i][j][v] = val; }
                *change = val - old;
            }
            return old;
        };

        // the element again, into C (tile already stored): the owner waits until its stores of the tile are written
        auto rewrite_c = [&](int r, int c, float val) {
            const int rr = r % 32;
            if (wm == r / WM && wn == c / WN && lr == c % 32 && lh == (rr / 4) % 2) {
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
                p.C[static_cast<int64_t>(m0 + r) * p.ldc + (n0 + c)] = p.alpha * val;
            }
        };

        // Soft-error injection: one accumulator per fault, after the K loop (or interval), before the checks
        // (run-time form of `t[2].x += error_inject`, ft_sgemm_huge.cuh:40,145).  A fault aimed at a row or column
        // of an edge tile that lies outside the matrix is ignored.  A kernel that verifies once injects every fault
        // before that verification.
        // (a tile split along K verifies every slice on its own - the checksums are linear in K; a kernel that
        // verifies once per slice takes the test faults into the tile's first slice, a cadence kernel, whose slices
        // start on a multiple of the interval, into the slice and interval that verification number `check` of the
        // whole K range falls into)
        if constexpr (kLazyOutside) {
            if (n0 + BN > p.N) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    const bool inside = n0 + wn * WN + j * 32 + lr < p.N;
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int v = 0; v < 16; ++v) acc[i][j][v] = inside ? acc[i][j][v] : 0.f;
                }
#pragma unroll
                for (int gm = 0; gm < GM; ++gm)
#pragma unroll
                    for (int e = 0; e < 4; ++e) cc_ref[gm][e] = e < b_nvalid[0] ? cc_ref[gm][e] : 0.0;
            }
            if (TA && m0 + BM > p.M) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const bool inside = m0 + wm * WM + i * 32 + 8 * (v >> 2) + 4 * lh + (v & 3) < p.M;
#pragma unroll
                        for (int j = 0; j < TN; ++j) acc[i][j][v] = inside ? acc[i][j][v] : 0.f;
                    }
#pragma unroll
                for (int sl = 0; sl < A_SLOTS; ++sl) {
                    const bool inside = m0 + (tid >> 2) + (kGemmThreads / A_V4_PER_ROW) * sl < p.M;
#pragma unroll
                    for (int gn = 0; gn < GN; ++gn) cr_ref[gn][sl] = inside ? cr_ref[gn][sl] : 0.0;
                }
            }
        }
        const int check_global = CADENCE ? k_first / p.check_interval + check : 0;
#pragma unroll 1
        for (int f = 0; f < p.n_faults; ++f)
            if (tile_linear == p.faults[f].tile && (CADENCE ? p.faults[f].check == check_global : k_slice == 0) &&
                m0 + p.faults[f].row < p.M && n0 + p.faults[f].col < p.N)
                add_at(p.faults[f].row, p.faults[f].col, p.faults[f].delta);
        if (last && early_store) store_c();

        if (tid < NCT) { s_meta[8 * tid] = 0; s_meta[8 * tid + 1] = 0; s_meta[8 * tid + 2] = -1; s_meta[8 * tid + 3] = -1; s_meta[8 * tid + 4] = 0; s_fix[2 * tid + 1] = 0.f; }

        // Two stages (the reference acts on a tile only when a column checksum AND a row checksum disagree,
        // ft_sgemm_huge.cuh:263-296 `if (error > err_bound1 && error1 > err_bound1)`): the column checksums screen -
        // observed column sums are in-lane additions, the cheap half of the work -, and the row checksums of the
        // workgroup tile are formed and compared only when some column was flagged.  A check tile none of whose
        // columns is flagged is clean; its rows are not looked at (nor counted, nor re-synchronised).  The weighted
        // locator has no column lines: there the plain row checksums are the screen, evaluated every time.
        // Reference checksums: every thread publishes its partial sums (columns nc..nc+3 over its k rows, its rows
        // over its k group); the residual passes below add the partials in a fixed order.
        auto publish_col_refs = [&]() {
#pragma unroll
            for (int gm = 0; gm < GM; ++gm)
#pragma unroll
                for (int e = 0; e < 4; ++e) s_ccref[(gm * CCP + e_hw) * BN + (tid % B_V4_PER_ROW) * 4 + e] = cc_ref[gm][e];
        };
        auto publish_row_refs = [&]() {
            if constexpr (kLazyRows) {
                // Row references formed now: ref[gn][m] = sum over the k range done so far of A[m][k] * b_r[gn][k], FP64,
                // b_r summed here from B, 1024 values of k at a time (with wave-tile checksums: read from the workspace), into the LDS the
                // column partials no longer need.  Only run when a column is flagged, so its cost (a pass over the tile's
                // rows of A, and of B without a workspace, by one workgroup) is that of a detection, not of a product.
                constexpr int kWaves = kGemmThreads / kWave;
                constexpr bool kFromB = kRowSumsAtDetection;
                constexpr int kChunk = 1024;
                static_assert(sizeof(double) * GM * CCP * BN >= sizeof(float) * kChunk, "a chunk of row sums fits in the column partials' place");
                float* const s_b = reinterpret_cast<float*>(s_ccref);
                for (int i = tid; i < GN * CRP * BM; i += kGemmThreads) s_crref[i] = 0.0;
                __syncthreads();
#pragma unroll 1
                for (int kc = k_first, ke = k_first; kc < kend; kc = ke) {
                    ke = (kFromB && kend - kc > kChunk) ? kc + kChunk : kend;  // (b_r from the workspace: one pass)
                    if constexpr (kFromB) {
                        // b_r[k] over the tile's columns inside the matrix: a half wave per k row, eight rows in flight
                        constexpr int kHalfs = kGemmThreads / 32;
                        const int hw = tid >> 5, l32 = tid & 31;
                        int cols_in = p.N - n0;
                        cols_in = cols_in < BN ? cols_in : BN;
                        const int ke_pad = kc + ((ke - kc + 3) & ~3);  // the sums are read four at a time
#pragma unroll 1
                        for (int kb = kc + hw * 8; kb < ke_pad; kb += kHalfs * 8) {
                            float t[8];
#pragma unroll
                            for (int i = 0; i < 8; ++i) {
                                const int k = kb + i;
                                const float* const brow = p.B + static_cast<int64_t>(k < ke ? k : kc) * p.ldb + n0 + l32 * 4;
                                // (a lane whose four columns all lie inside loads them at once; the one lane of a row
                                // that straddles the last column loads word by word; both predicated, nothing waits)
                                const bool whole = k < ke && l32 * 4 + 3 < cols_in;
                                v4f b4 = {0.f, 0.f, 0.f, 0.f};
                                if (whole) b4 = load_v4f_words(brow);
                                float x[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    if (!whole && k < ke && l32 * 4 + e < cols_in) x[e] = brow[e];
                                t[i] = (x[0] + x[1]) + (x[2] + x[3]);
                            }
#pragma unroll
                            for (int i = 0; i < 8; ++i) {
#pragma unroll
                                for (int off = 16; off > 0; off >>= 1) t[i] += __shfl_xor(t[i], off, kWave);
                                if (l32 == 0 && kb + i < ke_pad) s_b[kb + i - kc] = t[i];
                            }
                        }
                        __syncthreads();
                    }
                    if constexpr (!TA) {
                        // a wave per two rows, its lanes 4 values of k of each per pass (1 KiB of a row, one 16-byte load per
                        // lane: four word loads move the same bytes in four times the instructions, and the vector memory
                        // pipe of the one CU at work here is what limits this pass); the lanes' sums are added by a
                        // butterfly, the same tree every time
#pragma unroll 1
                        for (int r0 = 2 * wave; r0 < BM; r0 += 2 * kWaves) {
                            if (m0 + r0 >= p.M) break;
                            const float* const a_row0 = p.A + static_cast<int64_t>(m0 + r0) * p.lda;
                            const bool two = m0 + r0 + 1 < p.M;  // (else the second row reads the first again and is not kept)
                            const float* const a_row1 = two ? a_row0 + p.lda : a_row0;
                            double sum[2][GN];
#pragma unroll
                            for (int gn = 0; gn < GN; ++gn) sum[0][gn] = sum[1][gn] = 0.0;
#pragma unroll 1
                            for (int k = kc + lane * 4; k < ke; k += kWave * 4) {
                                float av[2][4];
                                if (k + 3 < ke) {
                                    const v4f a0 = load_v4f_words(a_row0 + k);
                                    const v4f a1 = load_v4f_words(a_row1 + k);
                                    av[0][0] = a0.x; av[0][1] = a0.y; av[0][2] = a0.z; av[0][3] = a0.w;
                                    av[1][0] = a1.x; av[1][1] = a1.y; av[1][2] = a1.z; av[1][3] = a1.w;
                                } else {
#pragma unroll
                                    for (int e = 0; e < 4; ++e) {
                                        av[0][e] = (k + e < ke) ? a_row0[k + e] : 0.f;
                                        av[1][e] = (k + e < ke) ? a_row1[k + e] : 0.f;
                                    }
                                }
#pragma unroll
                                for (int gn = 0; gn < GN; ++gn) {
                                    const v4f b = kFromB ? *reinterpret_cast<const v4f*>(s_b + (k - kc))
                                                          : *reinterpret_cast<const v4f*>(p.enc_b + (static_cast<int64_t>(tile_n) * GN + gn) * p.enc_ld + k);
                                    const double bx = static_cast<double>(b.x), by = static_cast<double>(b.y), bz = static_cast<double>(b.z), bw = static_cast<double>(b.w);
#pragma unroll
                                    for (int j = 0; j < 2; ++j)
                                        sum[j][gn] += static_cast<double>(av[j][0]) * bx + static_cast<double>(av[j][1]) * by +
                                                      static_cast<double>(av[j][2]) * bz + static_cast<double>(av[j][3]) * bw;
                                }
                            }
#pragma unroll
                            for (int j = 0; j < 2; ++j)
#pragma unroll
                                for (int gn = 0; gn < GN; ++gn) {
                                    double t = sum[j][gn];
#pragma unroll
                                    for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, kWave);
                                    if (lane == 0 && (j == 0 || two)) s_crref[(gn * CRP) * BM + r0 + j] += t;
                                }
                        }
                    } else {
                        // A^T: a lane per row (64 neighbouring rows per wave, contiguous in memory for each k), the waves
                        // that share a group of 64 rows take a part of the k range each: one partial per part
                        constexpr int kGroups = BM / kWave, kKParts = kWaves / kGroups;
                        static_assert(kWaves % kGroups == 0 && kKParts >= 1 && kKParts <= CRP, "the k parts of a row fit the partial slots");
                        const int r = (wave % kGroups) * kWave + lane, part = wave / kGroups;
                        const int per = (ke - kc + kKParts - 1) / kKParts;
                        const int ka = kc + part * per, kb = ka + per < ke ? ka + per : ke;
                        if (m0 + r < p.M) {
                            double sum[GN];
#pragma unroll
                            for (int gn = 0; gn < GN; ++gn) sum[gn] = 0.0;
                            const float* a_col = p.A + static_cast<int64_t>(ka) * p.lda + (m0 + r);
                            // (eight k rows' loads go out together)
#pragma unroll 1
                            for (int k0 = ka; k0 < kb; k0 += 8, a_col += 8 * static_cast<int64_t>(p.lda)) {
                                float av[8];
#pragma unroll
                                for (int u = 0; u < 8; ++u) av[u] = k0 + u < kb ? a_col[u * static_cast<int64_t>(p.lda)] : 0.f;
#pragma unroll
                                for (int u = 0; u < 8; ++u) {
                                    const int k = k0 + u < kb ? k0 + u : kb - 1;  // (past the part: a zero times a value that exists)
#pragma unroll
                                    for (int gn = 0; gn < GN; ++gn) {
                                        const float b = kFromB ? s_b[k - kc] : p.enc_b[(static_cast<int64_t>(tile_n) * GN + gn) * p.enc_ld + k];
                                        sum[gn] += static_cast<double>(av[u]) * static_cast<double>(b);
                                    }
                                }
                            }
#pragma unroll
                            for (int gn = 0; gn < GN; ++gn) s_crref[(gn * CRP + part) * BM + r] += sum[gn];
                        }
                    }
                    if constexpr (kFromB) __syncthreads();  // the next chunk's sums go where these were
                }
                return;
            }
#pragma unroll
            for (int gn = 0; gn < GN; ++gn)
#pragma unroll
                for (int sl = 0; sl < A_SLOTS; ++sl)
                    s_crref[(gn * CRP + e_class) * BM + (tid >> 2) + (kGemmThreads / A_V4_PER_ROW) * sl] = cr_ref[gn][sl];
        };
        // observed column sums of the accumulators (ft_sgemm_huge.cuh:147-154): lane = column.  In relative mode the
        // sums of absolute values go with them: they scale the threshold to the data.
        const bool relative = p.tau <= 0.f;
        auto observe_cols = [&]() {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                float s = 0.f, sa = 0.f;
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    float si = 0.f;
#pragma unroll
                    for (int v = 0; v < 16; ++v) si += acc[i][j][v];
                    s += si;
                }
                s += __shfl_xor(s, 32, kWave);
                if (relative) {
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int v = 0; v < 16; ++v) sa += __builtin_fabsf(acc[i][j][v]);
                    sa += __shfl_xor(sa, 32, kWave);
                }
                if (lh == 0) {
                    s_ccobs[wm * BN + wn * WN + j * 32 + lr] = s;
                    s_ccabs[wm * BN + wn * WN + j * 32 + lr] = sa;
                }
            }
        };
        // observed row sums (ft_sgemm_huge.cuh:156-171): register = row, summed over the 32 column lanes.  The
        // TM * 16 sums of a lane are reduced together, 32 (or 16) at a time: afterwards lane lr of each half holds
        // the sum of row number lr of the group, and every lane stores one
        auto observe_rows = [&]() {
            constexpr int RG = TM >= 2 ? 32 : 16;      // rows reduced together
            constexpr int NRG = TM * 16 / RG;          // groups per wave tile
#pragma unroll
            for (int g = 0; g < NRG; ++g) {
                float rs[RG], ra_[RG];
#pragma unroll
                for (int e = 0; e < RG; ++e) {
                    const int i = (g * RG + e) / 16, v = (g * RG + e) % 16;
                    float s = acc[i][0][v];
#pragma unroll
                    for (int j = 1; j < TN; ++j) s += acc[i][j][v];
                    rs[e] = s;
                }
                half32_transpose_sum<RG>(rs, lane);
                if (relative) {
#pragma unroll
                    for (int e = 0; e < RG; ++e) {
                        const int i = (g * RG + e) / 16, v = (g * RG + e) % 16;
                        float sa = 0.f;
#pragma unroll
                        for (int j = 0; j < TN; ++j) sa += __builtin_fabsf(acc[i][j][v]);
                        ra_[e] = sa;
                    }
                    half32_transpose_sum<RG>(ra_, lane);
                } else {
                    ra_[0] = 0.f;
                }
                // this lane's row: number e = lr % RG of the group -> block i, register v
                const int e = g * RG + (lr & (RG - 1)), v = e & 15;
                const int row = wm * WM + (e >> 4) * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                if (RG == 32 || lr < RG) {
                    s_crobs[wn * BM + row] = rs[0];
                    s_crabs[wn * BM + row] = ra_[0];
                }
            }
        };
        // Relative mode: tau of a line of n elements inside the matrix = tau_rel * sqrt(n) * max(mean |acc| of the line,
        // mean |acc| of the check tile): the rounding noise of a sum of n accumulators grows like sqrt(n) times their
        // magnitude, and the tile mean stands in for a short or cancelling line whose own accumulators say little about
        // the size of its terms.  The tile sum is formed in a fixed order (per wave, then wave by wave) from the sums
        // of the screening lines: columns, or rows with the weighted locator.
        constexpr int WPGM = WGM / GM, WPGN = WGN / GN;  // wave rows / wave columns per check tile
        auto tile_abs_sums = [&]() {
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) {
                const int gm = ct / GN, gn = ct % GN;
                float part = 0.f;
                if constexpr (kWeighted) {
                    for (int r = tid; r < CM; r += kGemmThreads)
#pragma unroll
                        for (int w = 0; w < WPGN; ++w) part += s_crabs[(gn * WPGN + w) * BM + gm * CM + r];
                } else {
                    for (int c = tid; c < CN; c += kGemmThreads)
#pragma unroll
                        for (int w = 0; w < WPGM; ++w) part += s_ccabs[(gm * WPGM + w) * BN + gn * CN + c];
                }
                part = wave_sum_lane63(part);
                if (lane == kWave - 1) s_tsum[ct * (kGemmThreads / kWave) + wave] = part;
            }
        };
        // One pass over the lines [first, first + count): residual = reference - observed; |d| > tau marks the line
        // (ft_sgemm_huge.cuh:200-271).  gated: a row line counts only if its check tile has a flagged column.
        auto residual_pass = [&](auto first_c, auto count_c, auto gated_c, double* d_out, const double* off) {
            constexpr int kFirst = decltype(first_c)::value, kCount = decltype(count_c)::value;
            constexpr bool kGated = decltype(gated_c)::value;
            constexpr int kPer = (kCount + kGemmThreads - 1) / kGemmThreads;
#pragma unroll
            for (int it = 0; it < kPer; ++it) {
                const int line = kFirst + tid + it * kGemmThreads;
                d_out[it] = 0.0;
                float clean = 0.f;
                int line_ct = -1;  // check tile of this line, if it has one inside the matrix (and is looked at)
                if (line < kFirst + kCount) {
                    const bool is_row = line < kRowLines;
                    // row line (gn, idx): row idx of the tile against wave column gn; column line (gm, idx) likewise
                    const int grp = kWeighted ? 0 : is_row ? line / BM : (line - kRowLines) / BN;
                    const int idx = kWeighted ? (is_row ? line : line - BM) : is_row ? line - grp * BM : (line - kRowLines) - grp * BN;
                    const int gm = kWeighted ? 0 : is_row ? idx / CM : grp, gn = kWeighted ? 0 : is_row ? grp : idx / CN;
                    const int ct = gm * GN + gn;
                    int rows_in = p.M - (m0 + gm * CM), cols_in = p.N - (n0 + gn * CN);
                    rows_in = rows_in < CM ? rows_in : CM;
                    cols_in = cols_in < CN ? cols_in : CN;
                    double ref = 0.0, obs = 0.0;
                    float mag = 0.f;
                    if (is_row) {
#pragma unroll
                        for (int w = 0; w < CRP; ++w) ref += s_crref[(grp * CRP + w) * BM + idx];
#pragma unroll
                        for (int w = 0; w < WPGN; ++w) obs += static_cast<double>(s_crobs[(grp * WPGN + w) * BM + idx]);
#pragma unroll
                        for (int w = 0; w < WPGN; ++w) mag += s_crabs[(grp * WPGN + w) * BM + idx];
                    } else {
#pragma unroll
                        for (int w = 0; w < CCP; ++w) ref += s_ccref[(grp * CCP + w) * BN + idx];
#pragma unroll
                        for (int w = 0; w < WPGM; ++w) obs += static_cast<double>(s_ccobs[(grp * WPGM + w) * BN + idx]);
#pragma unroll
                        for (int w = 0; w < WPGM; ++w) mag += s_ccabs[(grp * WPGM + w) * BN + idx];
                    }
                    const double d = (CADENCE ? ref - off[it] : ref) - obs;
                    d_out[it] = d;
                    const bool looked_at = !kGated || s_meta[8 * ct + 1] > 0;
                    if (rows_in > 0 && cols_in > 0 && looked_at) {  // check tiles of an edge tile that lie outside the matrix have no lines
                        double tau = static_cast<double>(p.tau);
                        if (relative) {
                            float total = 0.f;
#pragma unroll
                            for (int w = 0; w < kGemmThreads / kWave; ++w) total += s_tsum[ct * (kGemmThreads / kWave) + w];
                            const float mean = total / (static_cast<float>(rows_in) * static_cast<float>(cols_in));
                            const float n_line = static_cast<float>(is_row ? cols_in : rows_in);
                            const float own = mag * (p.tau_rel / __builtin_sqrtf(n_line));
                            const float floor = p.tau_rel * __builtin_sqrtf(n_line) * mean;
                            tau = static_cast<double>(own > floor ? own : floor);
                        }
                        if (fabs(d) > tau) {
                            atomicAdd(&s_meta[8 * ct + (is_row ? 0 : 1)], 1);
                            atomicMax(&s_meta[8 * ct + (is_row ? 2 : 3)], idx);
                            if constexpr (kWeighted) s_meta[8 * ct + 5] = __float_as_int(static_cast<float>(tau));  // (used when it is the only one)
                        } else {
                            clean = static_cast<float>(fabs(d));
                        }
                        line_ct = ct;
                    }
                    s_dr[line] = static_cast<float>(d);
                }
                // largest residual among the clean lines: the 32 lines of a half wave belong to one check tile (check
                // tiles are multiples of 32 rows and columns), so one lane per half records their maximum
                const float half_max = half32_allmax(clean);
                if (lr == 0 && line_ct >= 0) atomicMax(&s_meta[8 * line_ct + 4], __float_as_int(half_max));
            }
        };
        double d_col[LPT_C], d_row[LPT_R];  // this verification's residuals of this thread's lines
        bool rows_done = kWeighted;
        if constexpr (kWeighted) {
            publish_row_refs();
            observe_rows();
            __syncthreads();
            if (relative) {
                tile_abs_sums();
                __syncthreads();
            }
            residual_pass(std::integral_constant<int, 0>{}, std::integral_constant<int, kRowPass>{}, std::false_type{}, d_row, off_row);
            __syncthreads();
        } else {
            publish_col_refs();
            observe_cols();
            __syncthreads();
            if (relative) {
                tile_abs_sums();
                __syncthreads();
            }
            residual_pass(std::integral_constant<int, kRowLines>{}, std::integral_constant<int, kColPass>{}, std::false_type{}, d_col, off_col);
            __syncthreads();
            int flagged_cols = 0;
#pragma unroll
            for (int ct = 0; ct < NCT; ++ct) flagged_cols |= s_meta[8 * ct + 1];
            rows_done = __builtin_amdgcn_readfirstlane(flagged_cols) > 0;  // the same in every thread of the workgroup
            if (rows_done) {
                publish_row_refs();
                observe_rows();
                __syncthreads();
                residual_pass(std::integral_constant<int, 0>{}, std::integral_constant<int, kRowPass>{}, std::true_type{}, d_row, off_row);
                __syncthreads();
            }
        }
        // locate: one faulty row x one faulty column of a check tile (ft_sgemm_huge.cuh:273-296).  Correct: the
        // reference subtracts round(|residual|) (:352-371), which only fits its +1.0 test fault, and the signed row
        // residual would leave the fault-free rounding noise of a whole row in one element; the located accumulator
        // is computed again from A and B instead (recompute_element: one chain of fused multiply-adds over the k range
        // done so far, in the matrix core's order, so the element gets exactly the bits a fault-free run gives it).  The
        // operand row and column are staged through the LDS the reference partials no longer need, a chunk of kFixChunk
        // values of k at a time, by all threads (the condition is uniform over the workgroup).
        // Weighted locator (kernel/ft_sgemm/README.md:16-26): one faulty row; with a fault delta in column n its two
        // residuals are -delta and -(n + 1) delta, so their ratio names the column.  The element found that way is
        // computed again like any located element; the location counts as confirmed when that changed the element by
        // what the row's residual says (computing a healthy element again changes nothing, so a wrong guess does no
        // harm: the tile is then reported as detected, not corrected).
        float w_d1 = 0.f;
        bool w_located = false;
        if constexpr (kWeighted) {
            if (p.locate_rc && s_meta[0] > 0) {
                // Row x column with the rows as the screen (products one tile wide, whose operand A is read once and
                // has no checksum vector): a row is flagged, so the column references are formed now, cc[n] = sum over
                // the k range of a_c[k] * B[k][n] with a_c[k] the column sums of the tile's rows of A, a chunk of k at
                // a time through the LDS the row partials have left; then the columns are observed and thresholded
                // like the rows were.
                constexpr int kWavesV = kGemmThreads / kWave;
                constexpr int kChunkA = 8 * BM > 1024 ? 1024 : 8 * BM;  // floats in the place of GN * CRP * BM doubles
                static_assert(sizeof(double) * GN * CRP * BM >= sizeof(float) * kChunkA, "a chunk of column sums of A fits in the row partials' place");
                constexpr int kColGroups = BN / kWave, kKPartsV = kWavesV / kColGroups;
                static_assert(BN % kWave == 0 && kWavesV % kColGroups == 0 && kKPartsV >= 1 && kKPartsV <= CCP, "the k parts of a column fit the partial slots");
                float* const s_a = reinterpret_cast<float*>(s_crref);
                int rows_in = p.M - m0, cols_in = p.N - n0;
                rows_in = rows_in < BM ? rows_in : BM;
                cols_in = cols_in < BN ? cols_in : BN;
                __syncthreads();  // the row partials are no longer read
                for (int i = tid; i < GM * CCP * BN; i += kGemmThreads) s_ccref[i] = 0.0;
#pragma unroll 1
                for (int kc = k_first, ke = k_first; kc < kend; kc = ke) {
                    ke = kend - kc > kChunkA ? kc + kChunkA : kend;
                    if constexpr (!TA) {
                        // a thread per four values of k, four rows' loads in flight
#pragma unroll 1
                        for (int q = tid; q * 4 < ke - kc; q += kGemmThreads) {
                            const int k = kc + q * 4;
                            float t[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
                            for (int m = 0; m < rows_in; m += 4) {
                                float v[4][4];
#pragma unroll
                                for (int j = 0; j < 4; ++j) {
                                    const float* const src = p.A + static_cast<int64_t>(m0 + (m + j < rows_in ? m + j : m)) * p.lda + k;
                                    if (k + 3 < ke) {
                                        const v4f a4 = load_v4f_words(src);
                                        v[j][0] = a4.x; v[j][1] = a4.y; v[j][2] = a4.z; v[j][3] = a4.w;
                                    } else {
#pragma unroll
                                        for (int e = 0; e < 4; ++e) v[j][e] = k + e < ke ? src[e] : 0.f;
                                    }
                                }
#pragma unroll
                                for (int j = 0; j < 4; ++j)
#pragma unroll
                                    for (int e = 0; e < 4; ++e) t[e] += m + j < rows_in ? v[j][e] : 0.f;
                            }
#pragma unroll
                            for (int e = 0; e < 4; ++e) s_a[q * 4 + e] = t[e];
                        }
                    } else {
                        // A^T: row k holds the tile's rows side by side; a half wave per k
                        const int hw = tid >> 5, l32 = tid & 31;
#pragma unroll 1
                        for (int k = kc + hw; k < ke; k += kGemmThreads / 32) {
                            const float* const src = p.A + static_cast<int64_t>(k) * p.lda + m0;
                            float t = 0.f;
                            for (int m = l32; m < rows_in; m += 32) t += src[m];
#pragma unroll
                            for (int off = 16; off > 0; off >>= 1) t += __shfl_xor(t, off, kWave);
                            if (l32 == 0) s_a[k - kc] = t;
                        }
                    }
                    __syncthreads();
                    {
                        // a lane per column, the waves that share 64 columns a part of the chunk each
                        const int n = (wave % kColGroups) * kWave + lane, part = wave / kColGroups;
                        const int per = (ke - kc + kKPartsV - 1) / kKPartsV;
                        const int ka = kc + part * per, kb = ka + per < ke ? ka + per : ke;
                        if (n < cols_in) {
                            double sum = 0.0;
                            const float* bp = p.B + static_cast<int64_t>(ka) * p.ldb + n0 + n;
#pragma unroll 1
                            for (int k0 = ka; k0 < kb; k0 += 8, bp += 8 * static_cast<int64_t>(p.ldb)) {
                                float bv[8];
#pragma unroll
                                for (int u = 0; u < 8; ++u) bv[u] = k0 + u < kb ? bp[u * static_cast<int64_t>(p.ldb)] : 0.f;
#pragma unroll
                                for (int u = 0; u < 8; ++u) {
                                    const int k = k0 + u < kb ? k0 + u : kb - 1;
                                    sum += static_cast<double>(bv[u]) * static_cast<double>(s_a[k - kc]);
                                }
                            }
                            s_ccref[part * BN + n] += sum;
                        }
                    }
                    __syncthreads();
                }
                observe_cols();
                __syncthreads();
                residual_pass(std::integral_constant<int, kRowLines>{}, std::integral_constant<int, BN>{}, std::false_type{}, d_col, off_col);
                __syncthreads();
            }
            w_located = !p.locate_rc && s_meta[0] == 1;
            if (w_located) {
                const int bad_r = s_meta[2];
                w_d1 = s_dr[bad_r];
                // The weighted residual of that one row, formed now: the weighted sum of its accumulators (column n of
                // the tile weighted by n + 1) against the product of its row of A with the weighted row sums of B from
                // the workspace.  Every thread takes a share of the k range and of the accumulators, thread 0 adds the
                // shares in thread order.
                __syncthreads();  // the reference partials at the start of the LDS are no longer read
                double* const s_share = reinterpret_cast<double*>(smem);
                static_assert(sizeof(double) * (GM * CCP * BN + GN * CRP * BM) >= sizeof(double) * kGemmThreads, "one share per thread fits");
                float obs_share = 0.f;
                {
                    const int rr = bad_r % 32;
                    const int fi = (bad_r % WM) / 32, fv = 4 * (rr / 8) + rr % 4;
                    if (wm == bad_r / WM && lh == (rr / 4) % 2) {
#pragma unroll
                        for (int i = 0; i < TM; ++i)
#pragma unroll
                            for (int j = 0; j < TN; ++j)
#pragma unroll
                                for (int v = 0; v < 16; ++v)
                                    if (i == fi && v == fv)
                                        obs_share = __builtin_fmaf(acc[i][j][v], static_cast<float>(wn * WN + j * 32 + lr + 1), obs_share);
                    }
                }
                const float* const a_row = TA ? p.A + (m0 + bad_r) : p.A + static_cast<int64_t>(m0 + bad_r) * p.lda;
                const int64_t a_stride = TA ? p.lda : 1;
                const float* const bw = p.enc_a + static_cast<int64_t>(tile_n) * p.enc_ld;
                double ref_share = 0.0;
                for (int k = k_first + tid; k < kend; k += kGemmThreads)
                    ref_share += static_cast<double>(a_row[k * a_stride]) * static_cast<double>(bw[k]);
                s_share[tid] = ref_share - static_cast<double>(obs_share);
                __syncthreads();
                if (tid == 0) {
                    double d2 = 0.0;
                    for (int t = 0; t < kGemmThreads; ++t) d2 += s_share[t];
                    s_dr[BM + bad_r] = static_cast<float>(d2);
                }
                __syncthreads();
                int cols_in = p.N - n0;
                cols_in = cols_in < BN ? cols_in : BN;
                int col = static_cast<int>(__builtin_rintf(s_dr[BM + bad_r] / w_d1)) - 1;
                col = col < 0 ? 0 : (col >= cols_in ? cols_in - 1 : col);
                __syncthreads();  // everybody has read the line counts
                if (tid == 0) { s_meta[1] = 1; s_meta[3] = col; }
                __syncthreads();
            }
        }
        bool any_fixed = false;
#pragma unroll 1
        for (int ct = 0; ct < NCT; ++ct) {
            if (s_meta[8 * ct] == 1 && s_meta[8 * ct + 1] == 1) {
                const int bad_r = s_meta[8 * ct + 2], bad_c = s_meta[8 * ct + 3];
                if (m0 + bad_r >= p.M || n0 + bad_c >= p.N) continue;  // (lines outside the matrix are all zeros: not reached)
                constexpr int kFixChunk = static_cast<int>(sizeof(double) * (GM * CCP * BN + GN * CRP * BM) / (2 * sizeof(float))) / BK * BK;
                const float* const a_src = TA ? p.A + (m0 + bad_r) : p.A + static_cast<int64_t>(m0 + bad_r) * p.lda;
                const float* const b_src = p.B + (n0 + bad_c);
                const float fixed_val = recompute_element(a_src, TA ? p.lda : 1, b_src, p.ldb, k_first, kend, smem, kFixChunk, tid, kGemmThreads);
                // thread 0 hands the value to the accumulator's owner, who reports what the correction changed
                // (the re-synchronisation takes exactly that out of the two lines' residuals)
                if (tid == 0) s_fix[2 * ct] = fixed_val;
                __syncthreads();
                const float old_val = set_at(bad_r, bad_c, s_fix[2 * ct], &s_fix[2 * ct + 1]);
                (void)old_val;
                if (last && early_store) rewrite_c(bad_r, bad_c, s_fix[2 * ct]);
                any_fixed = true;
            }
        }
        if (CADENCE && any_fixed) __syncthreads();  // s_fix[2 ct + 1] = corrected - faulty value, for the resync below
        if constexpr (kWeighted) {
            if (w_located) {
                __syncthreads();  // s_fix[1] = what computing the element again changed
                // (the row's threshold plus sixteen rounding units of the residual: the observed sums of a row that holds
                // a fault of thousands of thresholds are themselves only good to a few units of its size)
                const bool confirmed = __builtin_fabsf(s_fix[1] - w_d1) <= __int_as_float(s_meta[5]) + 0x1p-20f * __builtin_fabsf(w_d1);
                if (!confirmed && tid == 0) s_meta[1] = 0;  // (read again by this same thread below)
            }
        }
        if constexpr (CADENCE) {
            // re-synchronise (ft_sgemm_huge.cuh:268-271): every line that was looked at starts the next interval with
            // what is left of its residual after the correction taken out of its reference
            constexpr int kColPer = (kColPass + kGemmThreads - 1) / kGemmThreads, kRowPer = (kRowLines + kGemmThreads - 1) / kGemmThreads;
#pragma unroll
            for (int it = 0; it < kColPer; ++it) {
                const int cl = tid + it * kGemmThreads;
                if (cl < kColPass) {
                    const int gm = cl / BN, idx = cl - gm * BN;
                    const int ct = gm * GN + idx / CN;
                    double fixed = 0.0;
                    if (s_meta[8 * ct] == 1 && s_meta[8 * ct + 1] == 1 && idx == s_meta[8 * ct + 3]) fixed = static_cast<double>(s_fix[2 * ct + 1]);
                    off_col[it] += d_col[it] - fixed;
                }
            }
            if (rows_done) {
#pragma unroll
                for (int it = 0; it < kRowPer; ++it) {
                    const int line = tid + it * kGemmThreads;
                    if (line < kRowLines) {
                        const int gn = line / BM, idx = line - gn * BM;
                        const int ct = (idx / CM) * GN + gn;
                        if (s_meta[8 * ct + 1] > 0) {
                            double fixed = 0.0;
                            if (s_meta[8 * ct] == 1 && s_meta[8 * ct + 1] == 1 && idx == s_meta[8 * ct + 2]) fixed = static_cast<double>(s_fix[2 * ct + 1]);
                            off_row[it] += d_row[it] - fixed;
                        }
                    }
                }
            }
        }
        if (tid < NCT) {
            const int ct = tid, gm = ct / GN, gn = ct % GN;
            const int nbr = s_meta[8 * ct], nbc = s_meta[8 * ct + 1], bad_r = s_meta[8 * ct + 2], bad_c = s_meta[8 * ct + 3];
            const int flag = (nbr == 1 && nbc == 1) ? 1 : ((nbr != 0 || nbc != 0) ? 2 : 0);
            rec.n_bad_rows += nbr;
            rec.n_bad_cols += nbc;
            const float clean = __int_as_float(s_meta[8 * ct + 4]);
            rec.max_clean_residual = clean > rec.max_clean_residual ? clean : rec.max_clean_residual;
            if (flag == 2) {
                rec.flag = 2;
            } else if (flag == 1 && rec.flag == 0) {
                rec.flag = 1;
                rec.row = bad_r - gm * CM;
                rec.col = bad_c - gn * CN;
                rec.row_residual = s_dr[gn * BM + bad_r];
                rec.col_residual = kWeighted ? s_dr[BM + (p.locate_rc ? bad_c : bad_r)] : s_dr[kRowLines + gm * BN + bad_c];
            }
            if (last && p.status) {
                hpcdnn_ft_status st = rec;
                if (st.flag == 2) { st.row = -1; st.col = -1; st.row_residual = 0.f; st.col_residual = 0.f; }
                const int srow = tile_m * GM + gm, scol = tile_n * GN + gn;
                if (tail_out) p.tail_status[tail_slot * NCT + ct] = st;
                else if (srow < p.status_rows && scol < p.status_ld) p.status[srow * p.status_ld + scol] = st;
            }
        }
        if constexpr (CADENCE) __syncthreads();  // the next interval's prologue writes the staging buffers again
    };

    if constexpr (CADENCE) {
        const int slice_end = kend;
        for (int check = 0;; ++check) {
            kend = (slice_end - kbeg > p.check_interval) ? kbeg + p.check_interval : slice_end;
            nkt = (kend - kbeg + BK - 1) / BK;
            const bool last = kend >= slice_end;
            if (check > 0) k_range_reset();
            run_k_range();
            verify(check, last);
            if (last) break;
            kbeg = kend;
        }
    } else {
        run_k_range();
        verify(0, true);
    }
    if (early_store) return;
    if (!tail_out) {
        store_c();
        return;
    }
    }  // FT != 0

    // ---- epilogue
    const int row_base = m0 + wm * WM + lh * 4;  // + i*32 + 8*(v/4) + v%4
    const int col_base = n0 + wn * WN + lr;      // + j*32

    if (tail_out) {
        // whole tile, no bounds: the reduction that reads these images skips rows and columns past the matrix
        float* out = tail_out + (wm * WM + lh * 4) * BN + wn * WN + lr;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) out[(i * 32 + 8 * (v / 4) + (v % 4)) * BN + j * 32] = acc[i][j][v];
        return;
    }
    if (p.partial) {
        float* out = p.partial + static_cast<size_t>(k_slice) * p.M * p.N;
        if constexpr (EDGE) {
            // (ragged tiles: through a descriptor that ends with the slice's last element of this tile, as for C below)
            const __amdgpu_buffer_rsrc_t o_rsrc = make_rsrc(out + static_cast<int64_t>(m0) * p.N + n0,
                                                            (static_cast<int64_t>(p.M - 1 - m0) * p.N + (p.N - n0)) * 4);
            const int ld_bytes = p.N * 4;
            const int lane_off = (wm * WM + lh * 4) * ld_bytes + (wn * WN + lr) * 4;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if (col_base + j * 32 >= p.N) continue;
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const float value = acc[i][j][v];
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), o_rsrc,
                                                              lane_off + j * 128 + (i * 32 + 8 * (v / 4) + (v % 4)) * ld_bytes, 0, 0);
                    }
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = row_base + i * 32 + 8 * (v / 4) + (v % 4);
                    const int col = col_base + j * 32;
                    out[static_cast<size_t>(row) * p.N + col] = acc[i][j][v];
                }
        return;
    }

    // C = alpha*acc + beta*C.  With beta != 0 the 16 old values of a 32x32 block are fetched together before the
    // first store, so that their latencies overlap instead of queueing behind each other.
    // Tiles of at most 128x128 store C with the streaming hint: many small workgroups finish close together, and
    // keeping their output out of the L2 leaves it to the operand panels (1 to 2 % on 1024^3, 2048^3, 4096x4096x256;
    // the 256x128 tiles measured 0.2 % slower with it and keep the plain store).
    constexpr bool kStreamC = BM * BN <= 128 * 128;
    const float alpha = p.alpha, beta = p.beta;
    if constexpr (EDGE) {
        // Ragged tiles: a buffer descriptor from the tile's corner to the last element of C inside the tile, so the
        // hardware drops stores to rows >= M (and returns 0 for loads there); the row offset has to be part of the
        // vector offset for that (a scalar offset is not range-checked).  Columns >= N would land in the next row:
        // they are switched off once per block column.  A compare, a branch and a 64-bit multiply per store, which
        // is what the pointer form compiles to, cost a 64x64 tile 3200 cycles here.
        const int64_t c_bytes = (static_cast<int64_t>(p.M - 1 - m0) * p.ldc + (p.N - n0)) * 4;
        const __amdgpu_buffer_rsrc_t c_rsrc = make_rsrc(p.C + static_cast<int64_t>(m0) * p.ldc + n0, c_bytes);
        const int ldc_bytes = p.ldc * 4;  // BM * ldc * 4 < 2^31 (host check)
        const int lane_off = (wm * WM + lh * 4) * ldc_bytes + (wn * WN + lr) * 4;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if (col_base + j * 32 >= p.N) continue;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                float old[16];
                if (beta != 0.f) {
#pragma unroll
                    for (int v = 0; v < 16; ++v)
                        old[v] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                     c_rsrc, lane_off + j * 128 + (i * 32 + 8 * (v / 4) + (v % 4)) * ldc_bytes, 0, 0));
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const float t = alpha * acc[i][j][v];
                    const float out = (beta == 0.f) ? t : __builtin_fmaf(beta, old[v], t);
                    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, out), c_rsrc,
                                                          lane_off + j * 128 + (i * 32 + 8 * (v / 4) + (v % 4)) * ldc_bytes, 0,
                                                          kStreamC ? 2 : 0);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int col = col_base + j * 32;
            float* cbase = p.C + static_cast<size_t>(row_base + i * 32) * p.ldc + col;
            float old[16];
            if (beta != 0.f) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r = 8 * (v / 4) + (v % 4);
                    old[v] = cbase[static_cast<size_t>(r) * p.ldc];
                }
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r = 8 * (v / 4) + (v % 4);
                const float t = alpha * acc[i][j][v];
                const float out = (beta == 0.f) ? t : __builtin_fmaf(beta, old[v], t);
                if constexpr (kStreamC) __builtin_nontemporal_store(out, &cbase[static_cast<size_t>(r) * p.ldc]);
                else cbase[static_cast<size_t>(r) * p.ldc] = out;
            }
        }
}

// Fixed-order second phase of split-K: C = alpha * (ws[0] + ws[1] + ...) + beta*C.
template <int kUnused = 0>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(int M, int N, int splits, const float* __restrict__ ws,
                                                            float* __restrict__ C, int ldc, float alpha, float beta) {
    const int64_t total = static_cast<int64_t>(M) * N;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < total; e += stride) {
        // eight slices are fetched before any is added, so their latencies overlap; the additions keep slice order
        float s = ws[e];
        int z = 1;
        for (; z + 8 <= splits; z += 8) {
            float t[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) t[u] = ws[static_cast<size_t>(z + u) * total + e];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += t[u];
        }
        for (; z < splits; ++z) s += ws[static_cast<size_t>(z) * total + e];
        const int64_t r = e / N, c = e - r * N;
        float* dst = C + r * ldc + c;
        const float t = alpha * s;
        *dst = (beta == 0.f) ? t : __builtin_fmaf(beta, *dst, t);
    }
}

// (splitk_reduce_wide_kernel, the variant for many slices, lives in common.h: the transposed SGEMV shares it)

// Fixed-order second phase of the tail split: for the tiles after the first full_tiles, C = alpha * (slice 0 +
// slice 1 + ...) + beta*C.  grid = (tail tiles, bm / 32): one block adds 32 rows of one tile, 4 columns per thread.
//
// ABFT (slices != nullptr): the first block of every tile also turns the records of the tile's K slices into the
// tile's records, one per check tile (gm x gn of them per workgroup tile).  Bad-line counts add up; a slice that could
// not locate its fault makes the check tile uncorrectable (2); otherwise it is corrected (1) if any slice corrected an
// element, and reports the first such slice's location and residuals (more than one corrected slice shows in the
// counts).  Slices are K ranges in ascending order, so with a verification cadence this is the order of the
// verifications.
template <int kUnused = 0>
__global__ __launch_bounds__(256) void tail_reduce_kernel(int M, int N, int bm, int bn, int tiles_m, int tiles_n,
                                                          int full_tiles, int splits, const float* __restrict__ partial,
                                                          float* __restrict__ C, int ldc, float alpha, float beta,
                                                          const hpcdnn_ft_status* __restrict__ slices, hpcdnn_ft_status* __restrict__ status,
                                                          int gm, int gn, int status_rows, int status_ld) {
    int tile_m, tile_n;
    tile_of_block(full_tiles + blockIdx.x, tiles_m, tiles_n, tile_m, tile_n);
    const int m0 = tile_m * bm, n0 = tile_n * bn;
    const size_t tile_elems = static_cast<size_t>(bm) * bn;
    const float* src = partial + static_cast<size_t>(blockIdx.x) * splits * tile_elems;
    const int groups_per_row = bn / 4;
    for (int g = threadIdx.x; g < 32 * groups_per_row; g += 256) {
        const int r = blockIdx.y * 32 + g / groups_per_row, c = (g % groups_per_row) * 4;
        const int row = m0 + r, col = n0 + c;
        if (row >= M || col >= N) continue;
        const size_t off = static_cast<size_t>(r) * bn + c;
        v4f s = *reinterpret_cast<const v4f*>(src + off);
        int z = 1;
        for (; z + 4 <= splits; z += 4) {  // four slices in flight, added in slice order
            v4f t[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) t[u] = *reinterpret_cast<const v4f*>(src + (z + u) * tile_elems + off);
#pragma unroll
            for (int u = 0; u < 4; ++u) s += t[u];
        }
        for (; z < splits; ++z) s += *reinterpret_cast<const v4f*>(src + z * tile_elems + off);
        const float sv[4] = {s.x, s.y, s.z, s.w};
        float* dst = C + static_cast<size_t>(row) * ldc + col;
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col + e < N) {
                const float t = alpha * sv[e];
                dst[e] = (beta == 0.f) ? t : __builtin_fmaf(beta, dst[e], t);
            }
    }
    if (slices && status && blockIdx.y == 0 && static_cast<int>(threadIdx.x) < gm * gn) {
        const int nct = gm * gn, ct = threadIdx.x, t = blockIdx.x;
        hpcdnn_ft_status out;
        out.flag = 0; out.row = -1; out.col = -1; out.n_bad_rows = 0; out.n_bad_cols = 0;
        out.row_residual = 0.f; out.col_residual = 0.f; out.max_clean_residual = 0.f;
        bool located = false;
        for (int z = 0; z < splits; ++z) {
            const hpcdnn_ft_status s = slices[(t * splits + z) * nct + ct];
            out.n_bad_rows += s.n_bad_rows;
            out.n_bad_cols += s.n_bad_cols;
            out.max_clean_residual = s.max_clean_residual > out.max_clean_residual ? s.max_clean_residual : out.max_clean_residual;
            if (s.flag == 2) out.flag = 2;
            if (s.flag == 1 && !located) {
                located = true;
                out.row = s.row; out.col = s.col; out.row_residual = s.row_residual; out.col_residual = s.col_residual;
            }
        }
        if (out.flag == 2) { out.row = -1; out.col = -1; out.row_residual = 0.f; out.col_residual = 0.f; }
        else if (located) out.flag = 1;
        const int srow = tile_m * gm + ct / gn, scol = tile_n * gn + ct % gn;
        if (srow < status_rows && scol < status_ld) status[srow * status_ld + scol] = out;
    }
}

// ---- ABFT pre-encode: the checksum vectors of the operands, one per row group (RM rows) / column group (CN
// columns), in one launch of 256-thread blocks that each cover kEncodeKB = 64 values of k: the first
// k_blocks * row_groups blocks encode A, the rest B (one block per 128 columns of B, i.e. 128 / CN column groups).  A
// group is a workgroup tile's rows or columns, or a wave tile's with wave-tile checksums.  (Blocks of 1024 threads
// over 256 values of k, the first layout, left a partial last round of blocks on the CUs - 3 us of a 4096-cubed call -
// and most CUs idle on small operands.)
//
// enc_a[g][k'] = sum over the rows m of row group g (m < M) of A[m][k]; zero for K <= k < enc_ld; k' is k with
// the order inside each group of 16 changed to 0, 8, 1, 9, ...  A thread owns 4 consecutive k and the RM / 16 rows of
// one of 16 row slices (a quarter wave per slice); the 16 partials are added in slice order, so the result does not
// depend on timing.
//
// enc_b[g][k] = sum over the columns n of column group g (n < N) of B[k][n]; zero for K <= k < enc_ld.  A half
// wave reads 128 columns of one k row (32 lanes x 4 columns) and owns 8 of the block's rows; CN / 4 neighbouring
// lanes share a column group.
//
// TA: A is given transposed (K rows of M floats, row length lda).  A row then holds a group's RM values side by side:
// the 16 lanes of a DPP row read them 16 at a time (64 contiguous bytes; the four rows of a wave four different k) and
// add their partial sums across the row; a block covers kEncodeKB values of k of one row group, a quarter per pass.
constexpr int kEncodeKB = 64;
template <int RM, int CN, bool TA = false, int KB = kEncodeKB>
__global__ __launch_bounds__(KB * 4) void abft_encode_kernel(int M, int N, int K, const float* __restrict__ A, int lda,
                                                             const float* __restrict__ B, int ldb,
                                                             float* __restrict__ enc_a, float* __restrict__ enc_b,
                                                             int enc_ld, int k_blocks, int row_groups, int col_groups) {
    static_assert(CN == 128 || CN == 64 || CN == 32, "column groups are 8, 16 or 32 lanes of a half wave");
    static_assert(RM % 16 == 0, "the rows of a group split evenly over 16 slices");
    static_assert(KB == 64 || KB == 256, "a row slice is a quarter wave (or a whole one)");
    constexpr int kSlices = 16, kRows = RM / kSlices, kSliceLanes = KB / 4;
    constexpr int kHalves = KB / 8, kRowsPerHalf = KB / kHalves;
    constexpr int kGroupLanes = CN / 4, kGroupsPer128 = 128 / CN;
    static_assert(kRowsPerHalf <= kGroupLanes, "every k row of a half wave has a lane of each group to write it");
    __shared__ v4f part[kSlices][kSliceLanes];
    const int a_blocks = k_blocks * row_groups;
    if (TA && static_cast<int>(blockIdx.x) < a_blocks) {
        static_assert(RM % 16 == 0, "a row group is read 16 values at a time");
        const int l16 = threadIdx.x & 15, krow = threadIdx.x >> 4;  // KB / 4 rows of k per pass
        const int group = blockIdx.x / k_blocks, m0 = group * RM;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const int k = (blockIdx.x % k_blocks) * KB + pass * (KB / 4) + krow;
            float t = 0.f;
            if (k < K) {
                const float* row = A + static_cast<int64_t>(k) * lda + m0;
                float v[RM / 16];
#pragma unroll
                for (int j = 0; j < RM / 16; ++j) v[j] = (m0 + l16 + 16 * j < M) ? row[l16 + 16 * j] : 0.f;
#pragma unroll
                for (int j = 0; j < RM / 16; ++j) t += v[j];
            }
            t = row16_allsum(t);
            if (l16 == 0 && k < enc_ld) {
                const int q = k & 15;  // k and k + 8 of a K step side by side, as below
                enc_a[static_cast<int64_t>(group) * enc_ld + (k & ~15) + (q & 7) * 2 + (q >> 3)] = t;
            }
        }
    } else if (static_cast<int>(blockIdx.x) < a_blocks) {
        const int lane = threadIdx.x % kSliceLanes, slice = threadIdx.x / kSliceLanes;
        const int group = blockIdx.x / k_blocks, m0 = group * RM;
        const int k = ((blockIdx.x % k_blocks) * kSliceLanes + lane) * 4;
        const float* base = A + static_cast<int64_t>(m0) * lda;
        // a group past the last row (the lower wave tiles of an edge tile) reads nothing and is all zeros
        const __amdgpu_buffer_rsrc_t rsrc = make_rsrc(base, m0 < M ? (static_cast<int64_t>(M - 1 - m0) * lda + K) * 4 : 0);
        v4f s = {0.f, 0.f, 0.f, 0.f};
        if (k < K && m0 < M) {
            v4f v[kRows];
#pragma unroll
            for (int r = 0; r < kRows; ++r) v[r] = buffer_load_v4f(rsrc, ((slice * kRows + r) * lda + k) * 4);
#pragma unroll
            for (int r = 0; r < kRows; ++r) s += v[r];
            // the group's tail beyond K holds the next row's first elements
            s.y = (k + 1 < K) ? s.y : 0.f;
            s.z = (k + 2 < K) ? s.z : 0.f;
            s.w = (k + 3 < K) ? s.w : 0.f;
        }
        part[slice][lane] = s;
        __syncthreads();
        if (slice == 0 && k < enc_ld) {
            v4f t = part[0][lane];
#pragma unroll
            for (int w = 1; w < kSlices; ++w) t += part[w][lane];
            // within each K step of 16, k and k + 8 sit side by side: the GEMM thread that stages rows k and
            // k + 8 of the B tile fetches both with one 8-byte load
            float* dst = enc_a + static_cast<int64_t>(group) * enc_ld + (k & ~15);
            const int q = k & 15, pos = (q & 7) * 2 + (q >> 3);
            dst[pos] = t.x;
            dst[pos + 2] = t.y;
            dst[pos + 4] = t.z;
            dst[pos + 6] = t.w;
        }
    } else {
        const int bid = blockIdx.x - a_blocks;
        const int lr = threadIdx.x & 31, half = threadIdx.x >> 5;
        const int tile_n = bid / k_blocks, n0 = tile_n * 128;
        const int kb = (bid % k_blocks) * KB;
        float s[kRowsPerHalf];
        v4f v[kRowsPerHalf];
#pragma unroll
        for (int i = 0; i < kRowsPerHalf; ++i) {
            const int k = kb + half + kHalves * i;
            const int kc = k < K ? k : K - 1;
            const float* base = B + static_cast<int64_t>(kc) * ldb + n0;
            v[i] = buffer_load_v4f(make_rsrc(base, static_cast<int64_t>(N - n0) * 4), lr * 16);
        }
#pragma unroll
        for (int i = 0; i < kRowsPerHalf; ++i) {
            const int k = kb + half + kHalves * i;
            float t = (v[i].x + v[i].y) + (v[i].z + v[i].w);
            t = k < K ? t : 0.f;
            // sum over the lanes of the column group; every lane of the group gets it
            t += dpp_mov<kDppXor1>(t);
            t += dpp_mov<kDppXor2>(t);
            t += dpp_mov<kDppHalfMirror>(t);
            if constexpr (kGroupLanes >= 16) t += dpp_mov<kDppMirror>(t);
            if constexpr (kGroupLanes >= 32) t += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, t), 0x401F));
            s[i] = t;
        }
        // lane l of a group writes the group's sum of k row l of this half wave
        const int in_group = lr % kGroupLanes, group = tile_n * kGroupsPer128 + lr / kGroupLanes;
        if (in_group < kRowsPerHalf) {
            float out = s[0];
#pragma unroll
            for (int i = 1; i < kRowsPerHalf; ++i) out = (in_group == i) ? s[i] : out;
            const int k = kb + half + kHalves * in_group;
            // (the last block of 128 columns may reach past the last column group)
            if (k < enc_ld && group < col_groups) enc_b[static_cast<int64_t>(group) * enc_ld + k] = out;
        }
    }
}

// ---- Pre-pass of the weighted-checksum locator: the two row sums of B per column group of CN columns,
//   enc_b[g][k]  = sum over the group's columns n of B[k][n]             (B e1, e1 = [1, 1, ...])
//   enc_bw[g][k] = sum over the group's columns n of (n' + 1) B[k][n]    (B e2, e2 = [1, 2, ...], n' counted inside the group)
// (kernel/ft_sgemm/README.md:16-26); zero for K <= k < enc_ld.  Nothing of A is needed.  Layout of the work as in the
// B half of abft_encode_kernel: 256-thread blocks over kEncodeKB values of k and 128 columns, a half wave per k row.
template <int CN, int KB = kEncodeKB>
__global__ __launch_bounds__(KB * 4) void abft_encode_weighted_kernel(int N, int K, const float* __restrict__ B, int ldb,
                                                                    float* __restrict__ enc_b, float* __restrict__ enc_bw,
                                                                    int enc_ld, int k_blocks, int col_groups) {
    static_assert(CN == 128 || CN == 64, "column groups are 16 or 32 lanes of a half wave");
    constexpr int kHalves = KB / 8, kRowsPerHalf = KB / kHalves;
    constexpr int kGroupLanes = CN / 4, kGroupsPer128 = 128 / CN;
    const int bid = blockIdx.x;
    const int lr = threadIdx.x & 31, half = threadIdx.x >> 5;
    const int tile_n = bid / k_blocks, n0 = tile_n * 128;
    const int kb = (bid % k_blocks) * KB;
    const int in_group = lr % kGroupLanes;
    const float w0 = static_cast<float>(in_group * 4 + 1);  // weight of this lane's first column
    float s[kRowsPerHalf], sw[kRowsPerHalf];
    v4f v[kRowsPerHalf];
#pragma unroll
    for (int i = 0; i < kRowsPerHalf; ++i) {
        const int k = kb + half + kHalves * i;
        const int kc = k < K ? k : K - 1;
        const float* base = B + static_cast<int64_t>(kc) * ldb + n0;
        v[i] = buffer_load_v4f(make_rsrc(base, static_cast<int64_t>(N - n0) * 4), lr * 16);
    }
#pragma unroll
    for (int i = 0; i < kRowsPerHalf; ++i) {
        const int k = kb + half + kHalves * i;
        float t = (v[i].x + v[i].y) + (v[i].z + v[i].w);
        float tw = __builtin_fmaf(v[i].x, w0, v[i].y * (w0 + 1.f)) + __builtin_fmaf(v[i].z, w0 + 2.f, v[i].w * (w0 + 3.f));
        t = k < K ? t : 0.f;
        tw = k < K ? tw : 0.f;
        // sums over the lanes of the column group; every lane of the group gets them
        t += dpp_mov<kDppXor1>(t);
        tw += dpp_mov<kDppXor1>(tw);
        t += dpp_mov<kDppXor2>(t);
        tw += dpp_mov<kDppXor2>(tw);
        t += dpp_mov<kDppHalfMirror>(t);
        tw += dpp_mov<kDppHalfMirror>(tw);
        t += dpp_mov<kDppMirror>(t);
        tw += dpp_mov<kDppMirror>(tw);
        if constexpr (kGroupLanes >= 32) {
            t += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, t), 0x401F));
            tw += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, tw), 0x401F));
        }
        s[i] = t;
        sw[i] = tw;
    }
    // lane l of a group writes the group's sums of k row l of this half wave
    const int group = tile_n * kGroupsPer128 + lr / kGroupLanes;
    if (in_group < kRowsPerHalf) {
        float out = s[0], outw = sw[0];
#pragma unroll
        for (int i = 1; i < kRowsPerHalf; ++i) {
            out = (in_group == i) ? s[i] : out;
            outw = (in_group == i) ? sw[i] : outw;
        }
        const int k = kb + half + kHalves * in_group;
        if (k < enc_ld && group < col_groups) {
            enc_b[static_cast<int64_t>(group) * enc_ld + k] = out;
            enc_bw[static_cast<int64_t>(group) * enc_ld + k] = outw;
        }
    }
}

}  // namespace hpcdnn
