// Persistent variant of the plain SGEMM kernel for problems of several rounds of whole tiles (every tile full,
// K a multiple of 32).
//
// The tile-per-workgroup kernel drains its load pipeline at the end of a tile, stores C, and the next workgroup
// starts with an empty pipeline: with one or two workgroups per CU those phases line up across the whole chip, so
// the matrix cores idle while every CU waits for its first loads or for its stores.  On a short K (8192 x 8192 x
// 256: sixteen K steps per tile) that is a sixth of the run.
//
// Here one workgroup per CU (two of the 128 x 128 tile, which has the registers for it) walks the tiles id, id + grid, id + 2 grid, ... as one stream of K steps:
//   * the loads that run two K steps ahead cross over to the next tile's first steps, so the pipeline never
//     drains and a tile boundary costs only the move of the accumulators;
//   * the finished tile (times alpha) moves to a second register set, and its stores are handed out a few at a
//     time behind the MFMAs of the next tile's first eight K steps, like the other side instructions of the loop;
//     the last tile's stores go out after the loop.  With beta != 0 (template flag BETA; C is not read without
//     it) each group of stores is preceded, one K step earlier, by the loads of the old values it needs.
//     A tile whose accumulators leave too few registers for a full second set (192 x 256: 192 of 512) stores the
//     first IMM values of a finished tile at the boundary itself and hands out the rest (beta == 0 only).
// Same LDS layout, fragment layout, accumulator layout and K-step schedule as sgemm_kernel.h; the summation order
// of every element of C is the same as there, so both kernels give the same bits.
#pragma once

#include "sgemm_kernel.h"

namespace hpcdnn {

constexpr int kPersistDripSteps = 8;  // K steps over which a finished tile's stores are spread

// TA: the left operand is given transposed (K x M row-major), staged as in sgemm_kernel.h's TA kernels.
template <int BM, int BN, int WGM, int WGN, bool BETA, int IMM = 0, int PER_CU = 1, bool TA = false>
__global__ __launch_bounds__(WGM * WGN * kWave, PER_CU) void sgemm_persistent_kernel(const GemmArgs p) {
    constexpr int BK = kGemmBK;
    constexpr int kThreads = WGM * WGN * kWave;
    constexpr int WM = BM / WGM, WN = BN / WGN;
    constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile is made of 32x32 blocks");
    constexpr int AS = BK + 4, BS = b_stage_stride<BN>();
    constexpr int A_STAGE = BM * AS, B_STAGE = BK * BS;
    constexpr int A_V4_PER_ROW = BK / 4, B_V4_PER_ROW = BN / 4;
    constexpr int A_SLOTS = BM * BK / 4 / kThreads, B_SLOTS = BK * BN / 4 / kThreads;
    static_assert((BM * BK) % (4 * kThreads) == 0 && (BN * BK) % (4 * kThreads) == 0, "tiles split evenly over the threads");
    constexpr int NGL = A_SLOTS + B_SLOTS;  // global loads (and LDS writes) per thread per K step
    constexpr int NRD = TM + TN;            // fragment read groups per half K step
    constexpr int NMG = 4 * TM * TN;        // MFMAs per half K step
    constexpr int kStores = TM * TN * 16;   // stores per lane per tile
    constexpr int kDrip = kStores - IMM;    // of them handed out during the next tile
    constexpr int NPST = kDrip / kPersistDripSteps;
    static_assert(kDrip % kPersistDripSteps == 0, "the deferred stores of a tile split evenly over the drip steps");
    static_assert(!(BETA && IMM != 0), "stores at the boundary would wait for the old values of C");
    // K steps at the start of a tile that carry stores; with BETA group g is loaded in step g and stored in step g + 1
    constexpr int kDripSection = BETA ? kPersistDripSteps + 2 : kPersistDripSteps;

    extern __shared__ __align__(16) float smem[];
    float* const As = smem;
    float* const Bs = smem + 2 * A_STAGE;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int lr = lane & 31, lh = lane >> 5;
    const int wm = wave / WGN, wn = wave % WGN;

    const int total = p.tiles_m * p.tiles_n, stride = gridDim.x;
    const int nkt = p.K / BK;  // even, >= kPersistDripSteps + 2
    const float alpha = p.alpha, beta = p.beta;
    auto origin = [&](int t, int& m0, int& n0) {
        int tm, tn;
        tile_of_block(t, p.tiles_m, p.tiles_n, tm, tn);
        m0 = tm * BM;
        n0 = tn * BN;
    };
    int tile = blockIdx.x;  // the tile being multiplied
    int m0, n0;
    origin(tile, m0, n0);

    // ---- global -> register staging (two sets: K step t+1 waits in one while t+2 is on its way)
    const int64_t a_step = TA ? static_cast<int64_t>(BK) * p.lda : BK;
    const int64_t b_step = static_cast<int64_t>(BK) * p.ldb;
    auto a_origin = [&](int m) { return TA ? p.A + m : p.A + static_cast<int64_t>(m) * p.lda; };
    const float* a_base = a_origin(m0);  // of the K step the next load fetches
    const float* b_base = p.B + n0;
    const float* a_next = a_base;  // where the stream goes on after this tile's last K step (itself: harmless re-reads)
    const float* b_next = b_base;
    auto set_next = [&](int t) {
        if (t < total) {
            int nm0, nn0;
            origin(t, nm0, nn0);
            a_next = a_origin(nm0);
            b_next = p.B + nn0;
        }
    };
    set_next(tile + stride);
    int k_loaded = 0;

    int a_voff[A_SLOTS], a_lds[A_SLOTS];
    int b_voff[B_SLOTS], b_lds[B_SLOTS];
#pragma unroll
    for (int s = 0; s < A_SLOTS; ++s) {
        const int idx = tid + s * kThreads;
        if constexpr (TA) {
            const int k = (idx / 4) % BK, m = ((idx / (4 * BK)) * 4 + idx % 4) * 4;  // four m of one k (sgemm_kernel.h)
            a_voff[s] = (k * p.lda + m) * 4;
            a_lds[s] = m * AS + k;
        } else {
            const int row = idx / A_V4_PER_ROW, kc = (idx % A_V4_PER_ROW) * 4;
            a_voff[s] = (row * p.lda + kc) * 4;
            a_lds[s] = row * AS + kc;
        }
    }
#pragma unroll
    for (int s = 0; s < B_SLOTS; ++s) {
        const int idx = tid + s * kThreads;
        const int row = idx / B_V4_PER_ROW, nc = (idx % B_V4_PER_ROW) * 4;
        b_voff[s] = (row * p.ldb + nc) * 4;
        b_lds[s] = row * BS + nc;
    }
    v4f ra[2][A_SLOTS], rb[2][B_SLOTS];
    auto gload1 = [&](auto slot, auto part) {
        constexpr int S = decltype(slot)::value, P = decltype(part)::value;
        if constexpr (P < A_SLOTS) ra[S][P] = buffer_load_v4f(make_rsrc_unbounded(a_base), a_voff[P]);
        else rb[S][P - A_SLOTS] = buffer_load_v4f(make_rsrc_unbounded(b_base), b_voff[P - A_SLOTS]);
    };
    // after the loads of a K step: on to the next one, which after the tile's last step is the next tile's first
    auto gload_advance = [&]() {
        const bool more = k_loaded + BK < p.K;
        a_base = more ? a_base + a_step : a_next;
        b_base = more ? b_base + b_step : b_next;
        k_loaded = more ? k_loaded + BK : 0;
    };
    auto lstore1 = [&](auto slot, auto part, int stage) {
        constexpr int S = decltype(slot)::value, P = decltype(part)::value;
        if constexpr (P < A_SLOTS && TA) {
            float* const dst = As + stage * A_STAGE + a_lds[P];
            dst[0] = ra[S][P].x;
            dst[AS] = ra[S][P].y;
            dst[2 * AS] = ra[S][P].z;
            dst[3 * AS] = ra[S][P].w;
        } else if constexpr (P < A_SLOTS) {
            *reinterpret_cast<v4f*>(As + stage * A_STAGE + a_lds[P]) = ra[S][P];
        } else {
            *reinterpret_cast<v4f*>(Bs + stage * B_STAGE + b_lds[P - A_SLOTS]) = rb[S][P - A_SLOTS];
        }
    };

    // ---- LDS -> fragment registers -> MFMA
    v16f acc[TM][TN];   // the tile being multiplied
    float done[kDrip];  // the finished tile (times alpha), less its first IMM values: the stores that are going out
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
#pragma unroll
    for (int e = 0; e < kDrip; ++e) done[e] = 0.f;
    v4f fa[2][TM];
    float fb[2][TN][4];
    const int a_frag_off = (wm * WM + lr) * AS + lh * 4;
    const int b_frag_off = (lh * 4) * BS + wn * WN + lr;
    auto fread1 = [&](auto buf, auto part, int stage, int g) {
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
    auto mfma1 = [&](auto buf, auto idx) {
        constexpr int Bf = decltype(buf)::value, I = decltype(idx)::value;
        constexpr int q = I / (TM * TN), i = (I / TN) % TM, j = I % TN;
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[Bf][i][q], fb[Bf][j][q], acc[i][j], 0, 0, 0);
    };

    // ---- stores of the finished tile: descriptor at its corner (empty until there is one: the hardware drops
    // stores past the end of a descriptor), the lane's part of the address in one register, the row as a scalar
    // offset, the block column as an immediate.  Consecutive stores walk the column blocks of one row group, so
    // that they fill whole rows of the tile.
    // (the descriptor is rebuilt at every store from the corner's address, held as two scalars)
    unsigned done_lo = 0, done_hi = 0;
    int done_bytes = 0;
    const int ldc_bytes = p.ldc * 4;  // BM * ldc * 4 < 2^31 (checked by the host)
    const int lane_off = (wm * WM + lh * 4) * ldc_bytes + (wn * WN + lr) * 4;
    float old[2][NPST];  // BETA: old values of C for two groups of stores
    auto done_rsrc = [&]() {
        return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<float*>(static_cast<uint64_t>(done_hi) << 32 | done_lo), 0,
                                                 done_bytes, 0x00020000);
    };
    // deferred store number E of the tile: element v of block (i, j), which is store IMM + E of all of them
    auto pload1 = [&](auto idx) {
        constexpr int E = decltype(idx)::value, Q = E + IMM;
        constexpr int j = Q % TN, v = (Q / TN) % 16, i = Q / (TN * 16);
        constexpr int r = i * 32 + 8 * (v / 4) + (v % 4);
        old[(E / NPST) & 1][E % NPST] =
            __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(done_rsrc(), lane_off + j * 128, r * ldc_bytes, 0));
    };
    auto pstore1 = [&](auto idx) {
        constexpr int E = decltype(idx)::value, Q = E + IMM;
        constexpr int j = Q % TN, v = (Q / TN) % 16, i = Q / (TN * 16);
        constexpr int r = i * 32 + 8 * (v / 4) + (v % 4);
        float value = done[E];
        if constexpr (BETA) value = __builtin_fmaf(beta, old[(E / NPST) & 1][E % NPST], value);
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), done_rsrc(), lane_off + j * 128,
                                              r * ldc_bytes, 0);
    };

    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;

    // One K step, as in sgemm_kernel.h: first half multiplies fragment buffer 0 while it reads the second-half
    // fragments, fetches step t+2 into the free staging set and writes step t+1 to the other LDS stage (and, in a
    // drip step, hands out NPST stores of the finished tile); barrier; second half multiplies buffer 1 while it
    // reads the first-half fragments of step t+1.  `drip` = number of the step inside the tile's drip section, or -1.
    auto step = [&](auto sl_next, auto sl_free, auto stage, auto drip) {
        constexpr int st = decltype(stage)::value, D = decltype(drip)::value;
        constexpr int LD = (BETA && D >= 0 && D < kPersistDripSteps) ? D : -1;                    // group whose old values are fetched
        constexpr int ST = BETA ? ((D >= 1 && D <= kPersistDripSteps) ? D - 1 : -1) : D;            // group that is stored
        constexpr int NLD = LD >= 0 ? NPST : 0, NST = ST >= 0 ? NPST : 0;
        constexpr int NS0 = NRD + 2 * NGL + NLD + NST;
        static_for<NMG>([&](auto m) {
            constexpr int Mi = decltype(m)::value;
            mfma1(S0{}, m);
            constexpr int k_lo = (Mi * NS0 + NMG - 1) / NMG, k_hi = ((Mi + 1) * NS0 + NMG - 1) / NMG;
            static_for<k_hi - k_lo>([&](auto d) {
                constexpr int o = k_lo + decltype(d)::value;
                if constexpr (o < NRD) {
                    fread1(S1{}, std::integral_constant<int, o>{}, st, 1);
                } else if constexpr (o < NRD + NGL) {
                    gload1(sl_free, std::integral_constant<int, o - NRD>{});
                    if constexpr (o == NRD + NGL - 1) gload_advance();
                } else if constexpr (o < NRD + 2 * NGL) {
                    lstore1(sl_next, std::integral_constant<int, o - NRD - NGL>{}, st ^ 1);
                } else if constexpr (o < NRD + 2 * NGL + NLD) {
                    pload1(std::integral_constant<int, (LD >= 0 ? LD : 0) * NPST + o - NRD - 2 * NGL>{});
                } else {
                    pstore1(std::integral_constant<int, (ST >= 0 ? ST : 0) * NPST + o - NRD - 2 * NGL - NLD>{});
                }
            });
            __builtin_amdgcn_sched_barrier(0);
        });
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
        static_for<NMG>([&](auto m) {
            constexpr int Mi = decltype(m)::value;
            mfma1(S1{}, m);
            constexpr int k_lo = (Mi * NRD + NMG - 1) / NMG, k_hi = ((Mi + 1) * NRD + NMG - 1) / NMG;
            static_for<k_hi - k_lo>([&](auto d) {
                fread1(S0{}, std::integral_constant<int, k_lo + decltype(d)::value>{}, st ^ 1, 0);
            });
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // prologue of the stream: step 0 -> LDS stage 0, step 1 -> staging set 1, first-half fragments of step 0
    static_for<NGL>([&](auto s) { gload1(S0{}, s); });
    gload_advance();
    static_for<NGL>([&](auto s) { lstore1(S0{}, s, 0); });
    static_for<NGL>([&](auto s) { gload1(S1{}, s); });
    gload_advance();
    __syncthreads();
    static_for<NRD>([&](auto s) { fread1(S0{}, s, 0, 0); });

    for (;;) {
        static_for<kDripSection / 2>([&](auto h) {
            constexpr int H = decltype(h)::value;
            step(S1{}, S0{}, S0{}, std::integral_constant<int, 2 * H>{});
            step(S0{}, S1{}, S1{}, std::integral_constant<int, 2 * H + 1>{});
        });
        for (int kt = kDripSection; kt < nkt; kt += 2) {
            step(S1{}, S0{}, S0{}, std::integral_constant<int, -1>{});
            step(S0{}, S1{}, S1{}, std::integral_constant<int, -1>{});
        }
        // tile boundary: the stream is already inside the next tile (its step 0 is in LDS, step 1 in flight)
        const uint64_t corner = reinterpret_cast<uint64_t>(p.C + static_cast<int64_t>(m0) * p.ldc + n0);
        done_lo = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(corner));
        done_hi = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(corner >> 32));
        done_bytes = -1;
        static_for<kStores>([&](auto q) {
            constexpr int Q = decltype(q)::value;
            constexpr int j = Q % TN, v = (Q / TN) % 16, i = Q / (TN * 16);
            const float scaled = alpha * acc[i][j][v];
            if constexpr (Q < IMM) {
                constexpr int r = i * 32 + 8 * (v / 4) + (v % 4);
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, scaled), done_rsrc(), lane_off + j * 128,
                                                      r * ldc_bytes, 0);
            } else {
                done[Q - IMM] = scaled;
            }
        });
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
        tile += stride;
        if (tile >= total) break;
        origin(tile, m0, n0);
        a_next = a_base;  // default for the tile after this one: none
        b_next = b_base;
        set_next(tile + stride);
    }
    static_for<kPersistDripSteps>([&](auto g) {
        constexpr int G = decltype(g)::value;
        if constexpr (BETA) static_for<NPST>([&](auto q) { pload1(std::integral_constant<int, G * NPST + decltype(q)::value>{}); });
        static_for<NPST>([&](auto q) { pstore1(std::integral_constant<int, G * NPST + decltype(q)::value>{}); });
    });
}

}  // namespace hpcdnn
