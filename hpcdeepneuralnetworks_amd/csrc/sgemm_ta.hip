// SGEMM kernels for a transposed left operand (A^T given as a K x M row-major matrix), in a translation unit of their
// own so that they compile beside the others.  The table is built from the same tile list as the one in sgemm.hip
// (sgemm_tiles.h).
#include "gemm_host.h"
#include "sgemm_persistent_kernel.h"
#include "sgemm_small_kernel.h"
#include "sgemm_tiles.h"

namespace hpcdnn {

namespace {
struct TaKernels {
    int bm, bn;
    void (*plain)(const GemmArgs);
    void (*edge)(const GemmArgs);
    void (*persistent)(const GemmArgs);       // as in sgemm.hip's table: beta == 0, beta != 0, or nullptr
    void (*persistent_beta)(const GemmArgs);
};

#define HPCDNN_TA_(BM, BN, WGM, WGN, OCC, NSLOT, PERSISTENT, PERSISTENT_BETA)                      \
    {                                                                                            \
        BM, BN, sgemm_kernel<BM, BN, WGM, WGN, false, 0, OCC, NSLOT, 0, false, true>,            \
            sgemm_kernel<BM, BN, WGM, WGN, true, 0, OCC, NSLOT, 0, false, true>, PERSISTENT, PERSISTENT_BETA \
    }
// the kinds of sgemm_tiles.h (IMM: stores at the tile boundary, PER_CU: persistent workgroups per CU, as in sgemm.hip)
#define HPCDNN_TA_PERSISTENT_(BM, BN, WGM, WGN, OCC, PER_CU)                                                         \
    HPCDNN_TA_(BM, BN, WGM, WGN, OCC, 2, (sgemm_persistent_kernel<BM, BN, WGM, WGN, false, 0, PER_CU, true>),        \
               (sgemm_persistent_kernel<BM, BN, WGM, WGN, true, 0, PER_CU, true>))
#define HPCDNN_TILE(BM, BN, WGM, WGN, OCC, EFF) HPCDNN_TA_(BM, BN, WGM, WGN, OCC, 2, nullptr, nullptr)
#define HPCDNN_TILE_PERSISTENT(BM, BN, WGM, WGN, OCC, EFF) HPCDNN_TA_PERSISTENT_(BM, BN, WGM, WGN, OCC, 1)
#define HPCDNN_TILE_PERSISTENT_TWO(BM, BN, WGM, WGN, OCC, EFF) HPCDNN_TA_PERSISTENT_(BM, BN, WGM, WGN, OCC, 2)
#define HPCDNN_TILE_PERSISTENT_BIG(BM, BN, WGM, WGN, OCC, EFF) \
    HPCDNN_TA_(BM, BN, WGM, WGN, OCC, 2, (sgemm_persistent_kernel<BM, BN, WGM, WGN, false, 64, 1, true>), nullptr)
#define HPCDNN_TILE_DEEP(BM, BN, WGM, WGN, OCC, EFF, NSLOT) HPCDNN_TA_(BM, BN, WGM, WGN, OCC, NSLOT, nullptr, nullptr)
#define HPCDNN_SMALL_TILE(TMB, OCC, EFF) \
    {32 * TMB, 32, sgemm_small_kernel<TMB, false, OCC, true>, sgemm_small_kernel<TMB, true, OCC, true>, nullptr, nullptr}

const TaKernels kTaKernels[] = {HPCDNN_SGEMM_TILE_LIST};
}  // namespace

void (*sgemm_ta_kernel(int tile, int bm, int bn, bool edge))(const GemmArgs) {
    if (tile < 0 || tile >= static_cast<int>(sizeof(kTaKernels) / sizeof(kTaKernels[0]))) return nullptr;
    const TaKernels& k = kTaKernels[tile];
    if (k.bm != bm || k.bn != bn) return nullptr;
    return edge ? k.edge : k.plain;
}

void (*sgemm_ta_persistent_kernel(int tile, int bm, int bn, bool beta))(const GemmArgs) {
    if (tile < 0 || tile >= static_cast<int>(sizeof(kTaKernels) / sizeof(kTaKernels[0]))) return nullptr;
    const TaKernels& k = kTaKernels[tile];
    if (k.bm != bm || k.bn != bn) return nullptr;
    return beta ? k.persistent_beta : k.persistent;
}

}  // namespace hpcdnn
