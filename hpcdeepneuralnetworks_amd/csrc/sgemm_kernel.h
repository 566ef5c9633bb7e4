// Row-major FP32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32).
//
// One workgroup of 256 threads (4 waves) owns a BM x BN tile of C; wave w owns
// a (BM/WGM) x (BN/WGN) sub-tile made of 32x32 MFMA blocks whose accumulators
// stay in registers for the whole K loop.  Per K step of BK the A tile
// (BM x BK) and B tile (BK x BN) go HBM/L2 -> VGPR (16-byte loads, issued one
// K step ahead) -> LDS -> MFMA operands.
//
// LDS layout (floats):
//   A stage: [BM][BK + 4]   k contiguous, as in memory.  Lane (row r, half h)
//            reads 16 bytes = k {8g+4h .. 8g+4h+3}: one ds_read_b128 feeds four
//            MFMA k-steps.  Row stride BK+4 spreads 16 consecutive rows over
//            all banks.
//   B stage: [BK][BN + 8]   n contiguous, as in memory; lane (col c, half h)
//            reads B[8g+4h+q][c] with ds_read_b32.  Stride BN+8 puts the two
//            half-waves (rows 4 apart) on disjoint banks.
// The MFMA k index is a permutation of the memory k index (lane half h of
// k-step q in group g carries k = 8g+4h+q); A and B use the same permutation,
// so the contraction is unchanged.
//
// Accumulator layout of one 32x32 block (16 VGPRs): register v of lane l holds
// element (row 8*(v/4) + 4*(l/32) + v%4, col l%32).
//
// With FT = true the kernel is the fused online-ABFT variant: see the comment
// at "Online ABFT encode" in the main loop and "ABFT verification" after it.
#pragma once

#include "common.h"

namespace hpcdnn {

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
    int k_chunk;     // K range of one grid.z slice, a multiple of BK (>= K when not split)
    float* partial;  // split-K: [gridDim.z][M][N] raw accumulators; nullptr = write C directly
    int vec_a;       // every in-range 4-float group of A is 16-byte aligned
    int vec_b;
    // ABFT
    float tau;
    int fault_tile, fault_row, fault_col;
    float fault_delta;
    hpcdnn_ft_status* status;
};

constexpr int kGemmThreads = 256;
constexpr int kXcds = 8;
constexpr int kGroupM = 4;  // tile rows swept together so that co-resident tiles share A and B panels

template <int BM, int BN, int BK, int STAGES>
constexpr size_t gemm_lds_bytes() {
    return sizeof(float) * STAGES * (static_cast<size_t>(BM) * (BK + 4) + static_cast<size_t>(BK) * (BN + 8));
}

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

template <int BM, int BN, int BK, int WGM, int WGN, int STAGES, bool EDGE, bool FT, int MIN_BLOCKS>
__global__ __launch_bounds__(kGemmThreads, MIN_BLOCKS) void sgemm_kernel(const GemmArgs p) {
    static_assert(WGM * WGN == kGemmThreads / kWave, "four waves per workgroup");
    static_assert(BK % 8 == 0, "K step is consumed in groups of 8");
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(TM >= 1 && TN >= 1 && WM % 32 == 0 && WN % 32 == 0, "wave tile is made of 32x32 blocks");
    constexpr int AS = BK + 4, BS = BN + 8;
    constexpr int A_STAGE = BM * AS, B_STAGE = BK * BS;
    constexpr int A_V4_PER_ROW = BK / 4, B_V4_PER_ROW = BN / 4;
    constexpr int A_SLOTS = BM * BK / 4 / kGemmThreads, B_SLOTS = BK * BN / 4 / kGemmThreads;
    static_assert(A_SLOTS >= 1 && B_SLOTS >= 1, "every thread stages at least one 16-byte group of A and of B");
    static_assert(STAGES == 1 || STAGES == 2, "single or double buffered LDS");

    extern __shared__ __align__(16) float smem[];
    float* const As = smem;
    float* const Bs = smem + STAGES * A_STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave / WGN, wn = wave % WGN;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int kbeg = blockIdx.z * p.k_chunk;
    const int kend = (p.K - kbeg < p.k_chunk) ? p.K : kbeg + p.k_chunk;
    const int nkt = (kend - kbeg + BK - 1) / BK;

    // ---- staging slots: which 16-byte groups of the A and B tiles this thread moves
    int a_row[A_SLOTS], a_kc[A_SLOTS], b_row[B_SLOTS], b_nc[B_SLOTS];
    const float* a_ptr[A_SLOTS];
    const float* b_ptr[B_SLOTS];
#pragma unroll
    for (int s = 0; s < A_SLOTS; ++s) {
        const int idx = tid + s * kGemmThreads;
        a_row[s] = idx / A_V4_PER_ROW;
        a_kc[s] = (idx % A_V4_PER_ROW) * 4;
        a_ptr[s] = p.A + static_cast<size_t>(m0 + a_row[s]) * p.lda + (kbeg + a_kc[s]);
    }
#pragma unroll
    for (int s = 0; s < B_SLOTS; ++s) {
        const int idx = tid + s * kGemmThreads;
        b_row[s] = idx / B_V4_PER_ROW;
        b_nc[s] = (idx % B_V4_PER_ROW) * 4;
        b_ptr[s] = p.B + static_cast<size_t>(kbeg + b_row[s]) * p.ldb + (n0 + b_nc[s]);
    }

    v4f ra[A_SLOTS], rb[B_SLOTS];

    auto load_tile = [&](int k0) {  // k0: absolute k of the tile's first column; never touches memory outside A/B
#pragma unroll
        for (int s = 0; s < A_SLOTS; ++s) {
            if (!EDGE) {
                ra[s] = *reinterpret_cast<const v4f*>(a_ptr[s]);
            } else {
                v4f v = {0.f, 0.f, 0.f, 0.f};
                const int gk = k0 + a_kc[s];
                if (m0 + a_row[s] < p.M && gk < kend) {
                    if (p.vec_a && gk + 4 <= kend) {
                        v = *reinterpret_cast<const v4f*>(a_ptr[s]);
                    } else {
                        v.x = a_ptr[s][0];
                        if (gk + 1 < kend) v.y = a_ptr[s][1];
                        if (gk + 2 < kend) v.z = a_ptr[s][2];
                        if (gk + 3 < kend) v.w = a_ptr[s][3];
                    }
                }
                ra[s] = v;
            }
            a_ptr[s] += BK;
        }
#pragma unroll
        for (int s = 0; s < B_SLOTS; ++s) {
            if (!EDGE) {
                rb[s] = *reinterpret_cast<const v4f*>(b_ptr[s]);
            } else {
                v4f v = {0.f, 0.f, 0.f, 0.f};
                const int gn = n0 + b_nc[s];
                if (k0 + b_row[s] < kend && gn < p.N) {
                    if (p.vec_b && gn + 4 <= p.N) {
                        v = *reinterpret_cast<const v4f*>(b_ptr[s]);
                    } else {
                        v.x = b_ptr[s][0];
                        if (gn + 1 < p.N) v.y = b_ptr[s][1];
                        if (gn + 2 < p.N) v.z = b_ptr[s][2];
                        if (gn + 3 < p.N) v.w = b_ptr[s][3];
                    }
                }
                rb[s] = v;
            }
            b_ptr[s] += static_cast<size_t>(BK) * p.ldb;
        }
    };

    auto store_tile = [&](int stage) {
        float* as = As + stage * A_STAGE;
        float* bs = Bs + stage * B_STAGE;
#pragma unroll
        for (int s = 0; s < A_SLOTS; ++s) *reinterpret_cast<v4f*>(as + a_row[s] * AS + a_kc[s]) = ra[s];
#pragma unroll
        for (int s = 0; s < B_SLOTS; ++s) *reinterpret_cast<v4f*>(bs + b_row[s] * BS + b_nc[s]) = rb[s];
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // ABFT reference checksums (see abft comment below); dead code when !FT.
    double cc_ref[TN], cr_ref[TM];
#pragma unroll
    for (int j = 0; j < TN; ++j) cc_ref[j] = 0.0;
#pragma unroll
    for (int i = 0; i < TM; ++i) cr_ref[i] = 0.0;

    const int a_frag_off = (wm * WM + lr) * AS + lh * 4;
    const int b_frag_off = (lh * 4) * BS + wn * WN + lr;

    auto compute_tile = [&](int stage) {
        const float* as = As + stage * A_STAGE + a_frag_off;
        const float* bs = Bs + stage * B_STAGE + b_frag_off;
#pragma unroll
        for (int g = 0; g < BK / 8; ++g) {
            v4f a[TM];
            float b[TN][4];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = *reinterpret_cast<const v4f*>(as + i * 32 * AS + g * 8);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) b[j][q] = bs[(g * 8 + q) * BS + j * 32];
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][q], b[j][q], acc[i][j], 0, 0, 0);

            if constexpr (FT) {
                // Online ABFT encode (the reference forms e^T A and B e on its
                // global->shared staging registers with warp shuffles and adds
                // the rank-1 products into spare shared memory,
                // kernel/ft_sgemm/include/ft_sgemm_huge.cuh:442-474).  Here each
                // wave works on the operand fragments it already holds: for
                // its WM rows and WN columns and the 4 k values of its lane half,
                //   acs[q] = sum over the wave's rows of A[., k]     (e^T A)
                //   brs[q] = sum over the wave's columns of B[k, .]  (B e)
                // then cc += acs*B[k, n] (column n = lane) and cr += A[m, k]*brs
                // (row m = lane).  The 4-term partial is formed in FP32 and
                // added to an FP64 running sum so that the reference checksums
                // carry no drift of their own over a long K.
                float cc_lo[TN], cr_lo[TM];
#pragma unroll
                for (int j = 0; j < TN; ++j) cc_lo[j] = 0.f;
#pragma unroll
                for (int i = 0; i < TM; ++i) cr_lo[i] = 0.f;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float acs = a[0][q], brs = b[0][q];
#pragma unroll
                    for (int i = 1; i < TM; ++i) acs += a[i][q];
#pragma unroll
                    for (int j = 1; j < TN; ++j) brs += b[j][q];
                    acs = half32_allsum(acs);
                    brs = half32_allsum(brs);
#pragma unroll
                    for (int j = 0; j < TN; ++j) cc_lo[j] = __builtin_fmaf(acs, b[j][q], cc_lo[j]);
#pragma unroll
                    for (int i = 0; i < TM; ++i) cr_lo[i] = __builtin_fmaf(a[i][q], brs, cr_lo[i]);
                }
#pragma unroll
                for (int j = 0; j < TN; ++j) cc_ref[j] += static_cast<double>(cc_lo[j]);
#pragma unroll
                for (int i = 0; i < TM; ++i) cr_ref[i] += static_cast<double>(cr_lo[i]);
            }
        }
    };

    // ---- main loop: global loads run one K step ahead of the MFMAs
    if (nkt > 0) {
        load_tile(kbeg);
        store_tile(0);
        __syncthreads();
    }
    for (int kt = 0; kt < nkt; ++kt) {
        const bool more = (kt + 1 < nkt);
        if (more) load_tile(kbeg + (kt + 1) * BK);
        if (STAGES == 2) {
            compute_tile(kt & 1);
            if (more) store_tile((kt + 1) & 1);
            __syncthreads();
        } else {
            compute_tile(0);
            __syncthreads();
            if (more) store_tile(0);
            __syncthreads();
        }
    }

    // ---- ABFT verification: inject (testing aid), observe, compare, locate, correct
    if constexpr (FT) {
        // The staging buffers are free after the loop's last barrier; reuse them.
        double* const s_ccref = reinterpret_cast<double*>(smem);    // [WGM][BN] reference column checksums per wave row
        double* const s_crref = s_ccref + WGM * BN;                 // [WGN][BM] reference row checksums per wave column
        float* const s_ccobs = reinterpret_cast<float*>(s_crref + WGN * BM);  // [WGM][BN] observed column sums
        float* const s_crobs = s_ccobs + WGM * BN;                  // [WGN][BM] observed row sums
        float* const s_dr = s_crobs + WGN * BM;                     // [BM] row residuals, then [BN] column residuals
        int* const s_meta = reinterpret_cast<int*>(s_dr + BM + BN); // nbr, nbc, bad row, bad col, max clean (float bits)
        static_assert(gemm_lds_bytes<BM, BN, BK, STAGES>() >=
                          sizeof(double) * (WGM * BN + WGN * BM) + sizeof(float) * (WGM * BN + WGN * BM + BM + BN) + 32,
                      "verification scratch fits in the staging buffers");
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

        // Soft-error injection: one accumulator, after the K loop, before the checks
        // (run-time form of `t[2].x += error_inject`, ft_sgemm_huge.cuh:40,145).
        if (tile_linear == p.fault_tile) add_at(p.fault_row, p.fault_col, p.fault_delta);

        if (tid == 0) { s_meta[0] = 0; s_meta[1] = 0; s_meta[2] = -1; s_meta[3] = -1; s_meta[4] = 0; }

        // reference checksums: fold the two lane halves (disjoint k subsets), publish per wave
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const double t = cc_ref[j] + __shfl_xor(cc_ref[j], 32, kWave);
            if (lh == 0) s_ccref[wm * BN + wn * WN + j * 32 + lr] = t;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const double t = cr_ref[i] + __shfl_xor(cr_ref[i], 32, kWave);
            if (lh == 0) s_crref[wn * BM + wm * WM + i * 32 + lr] = t;
        }
        // observed column sums of the accumulators (ft_sgemm_huge.cuh:147-154): lane = column
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            float s = 0.f;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                float si = 0.f;
#pragma unroll
                for (int v = 0; v < 16; ++v) si += acc[i][j][v];
                s += si;
            }
            s += __shfl_xor(s, 32, kWave);
            if (lh == 0) s_ccobs[wm * BN + wn * WN + j * 32 + lr] = s;
        }
        // observed row sums (ft_sgemm_huge.cuh:156-171): register = row, summed over the 32 column lanes
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float s = acc[i][0][v];
#pragma unroll
                for (int j = 1; j < TN; ++j) s += acc[i][j][v];
                s = half32_allsum(s);
                if (lr == 0) s_crobs[wn * BM + wm * WM + i * 32 + 8 * (v / 4) + 4 * lh + (v % 4)] = s;
            }
        __syncthreads();

        // residual = reference - observed per line; |d| > tau marks the line (ft_sgemm_huge.cuh:200-271)
        const double tau = static_cast<double>(p.tau);
        for (int line = tid; line < BM + BN; line += kGemmThreads) {
            const bool is_row = line < BM;
            const int idx = is_row ? line : line - BM;
            double ref = 0.0, obs = 0.0;
            if (is_row) {
#pragma unroll
                for (int w = 0; w < WGN; ++w) { ref += s_crref[w * BM + idx]; obs += static_cast<double>(s_crobs[w * BM + idx]); }
            } else {
#pragma unroll
                for (int w = 0; w < WGM; ++w) { ref += s_ccref[w * BN + idx]; obs += static_cast<double>(s_ccobs[w * BN + idx]); }
            }
            const double d = ref - obs;
            if (fabs(d) > tau) {
                atomicAdd(&s_meta[is_row ? 0 : 1], 1);
                atomicMax(&s_meta[is_row ? 2 : 3], idx);
            } else {
                atomicMax(&s_meta[4], __float_as_int(static_cast<float>(fabs(d))));
            }
            if (is_row) s_dr[idx] = static_cast<float>(d);
            else s_dr[BM + idx] = static_cast<float>(d);   // column residuals follow the row residuals
        }
        __syncthreads();

        // locate: one faulty row x one faulty column (ft_sgemm_huge.cuh:273-296); correct with the signed
        // row residual (the reference's round(|residual|), :358, only fits its +1.0 test fault)
        const int nbr = s_meta[0], nbc = s_meta[1], bad_r = s_meta[2], bad_c = s_meta[3];
        int flag = 0;
        if (nbr == 1 && nbc == 1) {
            flag = 1;
            add_at(bad_r, bad_c, s_dr[bad_r]);
        } else if (nbr != 0 || nbc != 0) {
            flag = 2;
        }
        if (tid == 0 && p.status) {
            hpcdnn_ft_status st;
            st.flag = flag;
            st.row = (flag == 1) ? bad_r : -1;
            st.col = (flag == 1) ? bad_c : -1;
            st.n_bad_rows = nbr;
            st.n_bad_cols = nbc;
            st.row_residual = (flag == 1) ? s_dr[bad_r] : 0.f;
            st.col_residual = (flag == 1) ? s_dr[BM + bad_c] : 0.f;
            st.max_clean_residual = __int_as_float(s_meta[4]);
            p.status[tile_linear] = st;
        }
    }

    // ---- epilogue
    const int row_base = m0 + wm * WM + lh * 4;  // + i*32 + 8*(v/4) + v%4
    const int col_base = n0 + wn * WN + lr;      // + j*32

    if (p.partial) {
        float* out = p.partial + static_cast<size_t>(blockIdx.z) * p.M * p.N;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = row_base + i * 32 + 8 * (v / 4) + (v % 4);
                    const int col = col_base + j * 32;
                    if (!EDGE || (row < p.M && col < p.N)) out[static_cast<size_t>(row) * p.N + col] = acc[i][j][v];
                }
        return;
    }

    const float alpha = p.alpha, beta = p.beta;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = row_base + i * 32 + 8 * (v / 4) + (v % 4);
                const int col = col_base + j * 32;
                if (!EDGE || (row < p.M && col < p.N)) {
                    float* c = p.C + static_cast<size_t>(row) * p.ldc + col;
                    const float t = alpha * acc[i][j][v];
                    *c = (beta == 0.f) ? t : __builtin_fmaf(beta, *c, t);
                }
            }
}

// Fixed-order second phase of split-K: C = alpha * (ws[0] + ws[1] + ...) + beta*C.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(int M, int N, int splits, const float* __restrict__ ws,
                                                            float* __restrict__ C, int ldc, float alpha, float beta) {
    const int64_t total = static_cast<int64_t>(M) * N;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * 256;
    for (int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; e < total; e += stride) {
        float s = ws[e];
        for (int z = 1; z < splits; ++z) s += ws[static_cast<size_t>(z) * total + e];
        const int64_t r = e / N, c = e - r * N;
        float* dst = C + r * ldc + c;
        const float t = alpha * s;
        *dst = (beta == 0.f) ? t : __builtin_fmaf(beta, *dst, t);
    }
}

}  // namespace hpcdnn
