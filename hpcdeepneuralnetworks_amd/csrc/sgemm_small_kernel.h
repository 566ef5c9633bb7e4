// Row-major FP32 GEMM for problems too small to give every CU a 64 x 64 tile.
//
// One workgroup of four waves owns a (32 * TMB) x 32 tile of C, and the four waves split K between them: wave w
// multiplies K blocks w, w + 4, w + 8, ... (32 k values each) of the whole tile, so a 512 x 512 problem still puts
// four waves on each of 256 CUs.  The waves share no operands, so the main loop has no LDS traffic and no barriers:
// every lane loads its MFMA operands straight from memory,
//   A: lane (row i, half h) reads A[m0 + i][kb + 16 h .. kb + 16 h + 15], four 16-byte loads: the two halves of a
//      wave cover one 128-byte line of each row;
//   B: lane (half h, column j) reads B[kb + 16 h + t][n0 + j] for t = 0 .. 15: each load is one 128-byte line per half,
// and MFMA t of the block contracts k = kb + t (half 0) with k = kb + 16 + t (half 1).  The next block's loads are
// issued before the current block's MFMAs (two register sets).  At the end the four partial tiles meet in LDS and
// are added in wave order, so the result does not depend on timing; it does differ in the last bits from the large
// tiles' result, which add the products of one element in a different order.
//
// TA: A is given transposed (K rows of M floats, row length lda >= M).  Its operands are then fetched like B's: lane
// (half h, row i) reads At[kb + 16 h + t][m0 + i] for t = 0 .. 15, one 128-byte line per half and load; the MFMAs and
// their order are the same, so the result has the bits of the untransposed kernel.
#pragma once

#include "sgemm_kernel.h"

namespace hpcdnn {

constexpr int kSmallBK = 32;
constexpr int kSmallWaves = 4;
constexpr int kSmallThreads = kSmallWaves * kWave;

template <int TMB>
constexpr size_t small_lds_bytes() {
    return sizeof(float) * kSmallWaves * (32 * TMB) * 32;
}

template <int TMB, bool EDGE, int MIN_BLOCKS, bool TA = false>
__global__ __launch_bounds__(kSmallThreads, MIN_BLOCKS) void sgemm_small_kernel(const GemmArgs p) {
    constexpr int BM = 32 * TMB, BN = 32, BK = kSmallBK;
    constexpr int kRun = BK / 2;  // k values per lane half
    extern __shared__ __align__(16) float smem[];  // [waves][BM * BN] partial tiles

    const int tid = threadIdx.x;
    // the wave index steers scalar values (descriptors, loop bounds): tell the compiler it is wave-uniform
    const int lane = tid & (kWave - 1), wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int li = lane & 31, lh = lane >> 5;

    if (static_cast<int>(blockIdx.x) >= p.tiles_m * p.tiles_n) return;  // this kernel has no tail split: one workgroup per tile
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int kbeg = blockIdx.z * p.k_chunk;
    const int kend = (p.K - kbeg < p.k_chunk) ? p.K : kbeg + p.k_chunk;
    const int nb = (kend - kbeg + BK - 1) / BK;  // K blocks of this slice

    // Descriptors start at the tile's first element of the wave's current K block and end with the matrix: rows
    // m >= M of A read as 0.  They move on by four K blocks per trip.
    const int k_first = kbeg + wave * BK;
    // (TA: A^T is walked like B: rows k >= K read as 0, and columns m >= M, the next row or padding, only reach
    // accumulators of rows that are never stored)
    const float* a_base = TA ? p.A + static_cast<int64_t>(k_first) * p.lda + m0 : p.A + static_cast<int64_t>(m0) * p.lda + k_first;
    const float* b_base = p.B + static_cast<int64_t>(k_first) * p.ldb + n0;
    int64_t a_left = TA ? (static_cast<int64_t>(p.K - 1 - k_first) * p.lda + (p.M - m0)) * 4
                        : (static_cast<int64_t>(p.M - 1 - m0) * p.lda + (p.K - k_first)) * 4;
    int64_t b_left = (static_cast<int64_t>(p.K - 1 - k_first) * p.ldb + (p.N - n0)) * 4;
    const int64_t a_hop = TA ? static_cast<int64_t>(kSmallWaves * BK) * p.lda : kSmallWaves * BK;
    const int64_t b_hop = static_cast<int64_t>(kSmallWaves * BK) * p.ldb;
    const int at_voff = static_cast<int>((static_cast<unsigned>(kRun * lh) * p.lda + li) * 4u);  // TA; < 2^32 as for B
    const int at_row_bytes = p.lda * 4;

    int a_voff[TMB][4];
#pragma unroll
    for (int tm = 0; tm < TMB; ++tm)
#pragma unroll
        for (int c = 0; c < 4; ++c) a_voff[tm][c] = ((tm * 32 + li) * p.lda + kRun * lh + 4 * c) * 4;
    const int b_voff = static_cast<int>((static_cast<unsigned>(kRun * lh) * p.ldb + li) * 4u);  // < 2^32 for any accepted ldb
    const int b_row_bytes = p.ldb * 4;  // wave-uniform: row t of the run goes into the scalar offset of its load

    v4f ra[2][TMB][4];
    float rb[2][kRun];
    v16f acc[TMB];
#pragma unroll
    for (int tm = 0; tm < TMB; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[tm][v] = 0.f;

    // Loads of K block `blk` into register set S.  Every block but the slice's last one lies inside the matrix in
    // k; the last one may be partial: there the k values past the end are forced to 0 on both operands (A holds the
    // next row or padding there), and the rows of B are clamped to the last valid one before the load, so that no
    // load leaves the matrix.
    auto load = [&](auto set, int blk) {
        constexpr int S = decltype(set)::value;
        const __amdgpu_buffer_rsrc_t ar = make_rsrc(a_base, a_left), br = make_rsrc(b_base, b_left);
        if (EDGE && blk == nb - 1) {
            const int valid = kend - (kbeg + blk * BK);  // 1 .. 32 k values in this block
            const int mine = valid - kRun * lh;          // of this lane's run (may be <= 0)
            if constexpr (TA) {
#pragma unroll
                for (int t = 0; t < kRun; ++t) {
                    const int r = kRun * lh + t;
                    const int rc = r < valid ? r : valid - 1;
#pragma unroll
                    for (int tm = 0; tm < TMB; ++tm) {
                        const float v = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                                                      ar, static_cast<int>((static_cast<unsigned>(rc) * p.lda + tm * 32 + li) * 4u), 0, 0));
                        ra[S][tm][t / 4][t % 4] = (r < valid) ? v : 0.f;
                    }
                }
            } else {
#pragma unroll
                for (int tm = 0; tm < TMB; ++tm)
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        v4f v = buffer_load_v4f(ar, a_voff[tm][c]);
                        v.x = (4 * c + 0 < mine) ? v.x : 0.f;
                        v.y = (4 * c + 1 < mine) ? v.y : 0.f;
                        v.z = (4 * c + 2 < mine) ? v.z : 0.f;
                        v.w = (4 * c + 3 < mine) ? v.w : 0.f;
                        ra[S][tm][c] = v;
                    }
            }
#pragma unroll
            for (int t = 0; t < kRun; ++t) {
                const int r = kRun * lh + t;
                const int rc = r < valid ? r : valid - 1;
                const float v = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(br, static_cast<int>((static_cast<unsigned>(rc) * p.ldb + li) * 4u), 0, 0));
                rb[S][t] = (r < valid) ? v : 0.f;
            }
        } else {
            if constexpr (TA) {
                int soff = 0;  // one running scalar offset, as for B below
#pragma unroll
                for (int t = 0; t < kRun; ++t) {
#pragma unroll
                    for (int tm = 0; tm < TMB; ++tm)
                        ra[S][tm][t / 4][t % 4] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ar, at_voff + tm * 128, soff, 0));
                    soff += at_row_bytes;
                    asm volatile("" : "+s"(soff));
                }
            } else {
#pragma unroll
                for (int tm = 0; tm < TMB; ++tm)
#pragma unroll
                    for (int c = 0; c < 4; ++c) ra[S][tm][c] = buffer_load_v4f(ar, a_voff[tm][c]);
            }
            if constexpr (EDGE) {
                // one running scalar offset instead of sixteen live ones: this variant is short of scalar registers
                int soff = 0;
#pragma unroll
                for (int t = 0; t < kRun; ++t) {
                    rb[S][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(br, b_voff, soff, 0));
                    soff += b_row_bytes;
                    asm volatile("" : "+s"(soff));
                }
            } else {
#pragma unroll
                for (int t = 0; t < kRun; ++t)
                    rb[S][t] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(br, b_voff, t * b_row_bytes, 0));
            }
        }
    };
    auto hop = [&]() {
        if constexpr (TA) {
            a_base += a_hop;
            a_left -= a_hop * 4;
        } else {
            a_base += kSmallWaves * BK;
            a_left -= kSmallWaves * BK * 4;
        }
        b_base += b_hop;
        b_left -= b_hop * 4;
    };
    auto multiply = [&](auto set) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int t = 0; t < kRun; ++t)
#pragma unroll
            for (int tm = 0; tm < TMB; ++tm)
                acc[tm] = __builtin_amdgcn_mfma_f32_32x32x2f32(ra[S][tm][t / 4][t % 4], rb[S][t], acc[tm], 0, 0, 0);
    };

    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    if (wave < nb) {
        load(S0{}, wave);
        for (int blk = wave;; blk += 2 * kSmallWaves) {
            const bool more1 = blk + kSmallWaves < nb;
            if (more1) { hop(); load(S1{}, blk + kSmallWaves); }
            multiply(S0{});
            if (!more1) break;
            const bool more0 = blk + 2 * kSmallWaves < nb;
            if (more0) { hop(); load(S0{}, blk + 2 * kSmallWaves); }
            multiply(S1{});
            if (!more0) break;
        }
    }

    // ---- the four partial tiles meet in LDS; accumulator register v of lane (li, lh) is element
    // (8 * (v / 4) + 4 * lh + v % 4, li) of its 32 x 32 block
    float* mine = smem + wave * (BM * BN);
#pragma unroll
    for (int tm = 0; tm < TMB; ++tm)
#pragma unroll
        for (int v = 0; v < 16; ++v) mine[(tm * 32 + 8 * (v / 4) + 4 * lh + (v % 4)) * BN + li] = acc[tm][v];
    __syncthreads();

    const float alpha = p.alpha, beta = p.beta;
    float* const raw = p.partial ? p.partial + static_cast<size_t>(blockIdx.z) * p.M * p.N : nullptr;
#pragma unroll
    for (int r = 0; r < BM * BN / kSmallThreads; ++r) {
        const int e = tid + r * kSmallThreads;
        float s = smem[e];
#pragma unroll
        for (int w = 1; w < kSmallWaves; ++w) s += smem[w * (BM * BN) + e];
        const int row = m0 + e / BN, col = n0 + e % BN;
        if (EDGE && (row >= p.M || col >= p.N)) continue;
        if (raw) {
            raw[static_cast<size_t>(row) * p.N + col] = s;
        } else {
            float* dst = p.C + static_cast<size_t>(row) * p.ldc + col;
            const float t = alpha * s;
            *dst = (beta == 0.f) ? t : __builtin_fmaf(beta, *dst, t);
        }
    }
}

}  // namespace hpcdnn
