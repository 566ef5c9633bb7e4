// The SGEMM tile table, one row per tile in the order of the tile index (hpcdnn_sgemm_tile_info, the `tile` argument of
// hpcdnn_sgemm_ex).  It is the counterpart of the reference's small/medium/large/tall/wide/huge shape table
// (kernel/ft_sgemm/code_gen/main.py:8-16), re-derived for 32x32 MFMA blocks and four or eight 64-lane waves per
// workgroup.  A row names its kind with one of six macros that the including file defines before expanding the list
// (sgemm.hip builds the table of untransposed kernels and the cost model's figures from it, sgemm_ta.hip the kernels
// for a transposed left operand), so the two tables cannot drift apart:
//   HPCDNN_TILE(BM, BN, WGM, WGN, OCC, EFF)                 tile-per-workgroup kernel only
//   HPCDNN_TILE_PERSISTENT(BM, BN, WGM, WGN, OCC, EFF)      + persistent kernel, one workgroup per CU
//   HPCDNN_TILE_PERSISTENT_TWO(BM, BN, WGM, WGN, OCC, EFF)  + persistent kernel, two workgroups per CU (64 accumulators per lane)
//   HPCDNN_TILE_PERSISTENT_BIG(BM, BN, WGM, WGN, OCC, EFF)  + persistent kernel that stores 64 of a finished tile's values at
//                                                             the tile boundary (192 accumulators per lane; beta == 0 only)
//   HPCDNN_TILE_DEEP(BM, BN, WGM, WGN, OCC, EFF, NSLOT)     tile-per-workgroup kernel with its loads NSLOT K steps ahead
//   HPCDNN_SMALL_TILE(TMB, OCC, EFF)                        32 TMB x 32 tile whose four waves split K
// BM x BN tile, WGM x WGN waves, OCC resident workgroups per CU the kernel is built for, EFF the fitted steady-state
// fraction of the FP32 MFMA peak of one CU (least-squares fit of plan_cost() in sgemm.hip to measured times of every
// tile over squares 256..6144 with K = n, 1024 and 256 and a set of skinny shapes on an MI355X).
#pragma once

#define HPCDNN_SGEMM_TILE_LIST                                                                                        \
    HPCDNN_TILE_PERSISTENT(256, 128, 2, 2, 2, 0.978f),     /* 0 huge (the ABFT tile) */                               \
    HPCDNN_TILE_PERSISTENT_TWO(128, 128, 2, 2, 2, 0.970f), /* 1 large */                                              \
    HPCDNN_TILE(128, 64, 2, 2, 2, 0.945f),                 /* 2 tall */                                               \
    HPCDNN_TILE(64, 128, 2, 2, 2, 0.939f),                 /* 3 wide */                                               \
    HPCDNN_TILE(64, 64, 2, 2, 4, 0.900f),                  /* 4 medium */                                             \
    HPCDNN_TILE_PERSISTENT_BIG(192, 256, 2, 2, 1, 0.964f), /* 5 6144-friendly: 32 x 24 tiles = 3 full rounds of 256 CUs */ \
    HPCDNN_TILE(256, 192, 2, 2, 1, 0.946f),                /* 6 */                                                    \
    HPCDNN_TILE_PERSISTENT(128, 256, 2, 2, 2, 0.987f),     /* 7 */                                                    \
    HPCDNN_TILE(256, 256, 2, 4, 1, 1.000f),                /* 8 giant, eight waves */                                 \
    HPCDNN_TILE(256, 128, 4, 2, 1, 1.000f),                /* 9 huge, eight waves */                                  \
    HPCDNN_TILE(256, 256, 4, 2, 1, 1.000f),                /* 10 giant, eight waves (4 x 2) */                        \
    /* 11 small: 32 x 32, K split between the four waves.  Every lane fetches its own operands, so the rate is set  \
       by the vector memory path, about half the matrix peak: for problems with too few 64 x 64 tiles to go round */ \
    HPCDNN_SMALL_TILE(1, 4, 0.50f),                                                                                   \
    /* 12 medium with its loads four K steps ahead: a 64-row tile moves 64 bytes per row and K step, and with one   \
       workgroup per CU two steps in flight do not cover the trip to HBM when A is long and read once.  Staged data \
       is so old when it is needed that the LDS writes lead the step and are done long before the barrier */         \
    HPCDNN_TILE_DEEP(64, 64, 2, 2, 4, 0.905f, 4),                                                                     \
    HPCDNN_TILE(192, 192, 2, 2, 1, 0.943f)                 /* 13 3072-friendly: 16 x 16 tiles = one full round of 256 CUs */
