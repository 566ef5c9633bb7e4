// SGEMM kernels for a transposed left operand (A^T given as a K x M row-major matrix), in a translation unit of their
// own so that they compile beside the others.  Row i of the table is tile i of the table in sgemm.hip; the 32 x 32
// tile, whose lanes fetch their own operands, has no such variant.
#include "gemm_host.h"

namespace hpcdnn {

namespace {
struct TaKernels {
    int bm, bn;
    void (*plain)(const GemmArgs);
    void (*edge)(const GemmArgs);
};

#define HPCDNN_TA(BM, BN, WGM, WGN, OCC, NSLOT)                                                   \
    {                                                                                            \
        BM, BN, sgemm_kernel<BM, BN, WGM, WGN, false, 0, OCC, NSLOT, 0, false, true>,            \
            sgemm_kernel<BM, BN, WGM, WGN, true, 0, OCC, NSLOT, 0, false, true>                  \
    }

const TaKernels kTaKernels[] = {
    HPCDNN_TA(256, 128, 2, 2, 2, 2),  // 0
    HPCDNN_TA(128, 128, 2, 2, 2, 2),  // 1
    HPCDNN_TA(128, 64, 2, 2, 2, 2),   // 2
    HPCDNN_TA(64, 128, 2, 2, 2, 2),   // 3
    HPCDNN_TA(64, 64, 2, 2, 4, 2),    // 4
    HPCDNN_TA(192, 256, 2, 2, 1, 2),  // 5
    HPCDNN_TA(256, 192, 2, 2, 1, 2),  // 6
    HPCDNN_TA(128, 256, 2, 2, 2, 2),  // 7
    HPCDNN_TA(256, 256, 2, 4, 1, 2),  // 8
    HPCDNN_TA(256, 128, 4, 2, 1, 2),  // 9
    HPCDNN_TA(256, 256, 4, 2, 1, 2),  // 10
    {32, 32, nullptr, nullptr},       // 11
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

}  // namespace hpcdnn
