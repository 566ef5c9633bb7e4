// SGEMM kernels for a transposed left operand (A^T given as a K x M row-major matrix), in a translation unit of their
// own so that they compile beside the others.  Row i of the table is tile i of the table in sgemm.hip; the 32 x 32
// tile, whose lanes fetch their own operands, has no such variant.
#include "gemm_host.h"
#include "sgemm_persistent_kernel.h"

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
#define HPCDNN_TA(BM, BN, WGM, WGN, OCC, NSLOT) HPCDNN_TA_(BM, BN, WGM, WGN, OCC, NSLOT, nullptr, nullptr)
// (IMM: stores at the tile boundary, PER_CU: persistent workgroups per CU, both as for the same tile in sgemm.hip)
#define HPCDNN_TA_PERSISTENT(BM, BN, WGM, WGN, OCC, PER_CU)                                                          \
    HPCDNN_TA_(BM, BN, WGM, WGN, OCC, 2, (sgemm_persistent_kernel<BM, BN, WGM, WGN, false, 0, PER_CU, true>),        \
               (sgemm_persistent_kernel<BM, BN, WGM, WGN, true, 0, PER_CU, true>))

const TaKernels kTaKernels[] = {
    HPCDNN_TA_PERSISTENT(256, 128, 2, 2, 2, 1),  // 0
    HPCDNN_TA_PERSISTENT(128, 128, 2, 2, 2, 2),  // 1
    HPCDNN_TA(128, 64, 2, 2, 2, 2),   // 2
    HPCDNN_TA(64, 128, 2, 2, 2, 2),   // 3
    HPCDNN_TA(64, 64, 2, 2, 4, 2),    // 4
    HPCDNN_TA_(192, 256, 2, 2, 1, 2, (sgemm_persistent_kernel<192, 256, 2, 2, false, 64, 1, true>), nullptr),  // 5
    HPCDNN_TA(256, 192, 2, 2, 1, 2),  // 6
    HPCDNN_TA_PERSISTENT(128, 256, 2, 2, 2, 1),  // 7
    HPCDNN_TA(256, 256, 2, 4, 1, 2),  // 8
    HPCDNN_TA(256, 128, 4, 2, 1, 2),  // 9
    HPCDNN_TA(256, 256, 4, 2, 1, 2),  // 10
    {32, 32, nullptr, nullptr, nullptr, nullptr},  // 11
    HPCDNN_TA(64, 64, 2, 2, 4, 4),    // 12
    HPCDNN_TA(192, 192, 2, 2, 1, 2),  // 13
};
}  // namespace

void (*sgemm_ta_kernel(int tile, int bm, int bn, bool edge))(const GemmArgs) {
    if (tile < 0 || tile >= static_cast<int>(sizeof(kTaKernels) / sizeof(kTaKernels[0]))) return nullptr;
    const TaKernels& k = kTaKernels[tile];
    if (k.bm != bm || k.bn != bn) return nullptr;  // the two tables have drifted apart
    return edge ? k.edge : k.plain;
}

void (*sgemm_ta_persistent_kernel(int tile, int bm, int bn, bool beta))(const GemmArgs) {
    if (tile < 0 || tile >= static_cast<int>(sizeof(kTaKernels) / sizeof(kTaKernels[0]))) return nullptr;
    const TaKernels& k = kTaKernels[tile];
    if (k.bm != bm || k.bn != bn) return nullptr;
    return beta ? k.persistent_beta : k.persistent;
}

}  // namespace hpcdnn
