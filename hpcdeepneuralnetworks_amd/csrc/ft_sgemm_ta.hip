// ABFT-SGEMM kernels for a transposed left operand (A^T given as a K x M row-major matrix: the reference family's
// column-major operands), in a translation unit of their own so that they compile beside the others.  Row i of the
// table is tile class i of the table in ft_sgemm.hip, with the same wave layouts.
#include "gemm_host.h"

namespace hpcdnn {

namespace {
#define HPCDNN_FT_TA_KERNEL_(BM, BN, WM_, WN_, FT, GRAN, CAD)                                              \
    FtKernel {                                                                                             \
        sgemm_kernel<BM, BN, WM_, WN_, false, FT, 1, 2, GRAN, CAD, true>,                                  \
            sgemm_kernel<BM, BN, WM_, WN_, true, FT, 1, 2, GRAN, CAD, true>, WM_ * WN_ * kWave,            \
            gemm_lds_bytes<BM, BN, FT, WM_ * WN_ * kWave, WM_, WN_, GRAN>()                                \
    }
#define HPCDNN_FT_TA_KERNEL(BM, BN, WM_, WN_, GRAN, CAD) HPCDNN_FT_TA_KERNEL_(BM, BN, WM_, WN_, 2, GRAN, CAD)
#define HPCDNN_FT_TA_FUSED(BM, BN, CAD) HPCDNN_FT_TA_KERNEL_(BM, BN, 2, 2, 1, 0, CAD)
#define HPCDNN_FT_TA_NONE \
    FtKernel { nullptr, nullptr, 0, 0 }

struct FtTaClass {
    int bm, bn;
    // checksum vectors from the workspace: per workgroup tile, per wave tile, per workgroup tile with verification
    // cadence; checksum vectors formed in the main loop (four waves, as in ft_sgemm.hip): per workgroup tile, and
    // with verification cadence
    FtKernel kind[5];
};
const FtTaClass kFtTaClasses[HPCDNN_FT_NUM_CLASSES] = {
    {256, 128, {HPCDNN_FT_TA_KERNEL(256, 128, 2, 4, 0, false), HPCDNN_FT_TA_KERNEL(256, 128, 2, 4, 1, false), HPCDNN_FT_TA_KERNEL(256, 128, 2, 4, 0, true),
                 HPCDNN_FT_TA_FUSED(256, 128, false), HPCDNN_FT_TA_FUSED(256, 128, true)}},
    {128, 128, {HPCDNN_FT_TA_KERNEL(128, 128, 2, 2, 0, false), HPCDNN_FT_TA_KERNEL(128, 128, 2, 2, 1, false), HPCDNN_FT_TA_KERNEL(128, 128, 2, 2, 0, true),
                 HPCDNN_FT_TA_FUSED(128, 128, false), HPCDNN_FT_TA_FUSED(128, 128, true)}},
    {64, 128, {HPCDNN_FT_TA_KERNEL(64, 128, 2, 2, 0, false), HPCDNN_FT_TA_KERNEL(64, 128, 2, 2, 1, false), HPCDNN_FT_TA_NONE,
                HPCDNN_FT_TA_FUSED(64, 128, false), HPCDNN_FT_TA_NONE}},
    {128, 64, {HPCDNN_FT_TA_KERNEL(128, 64, 2, 2, 0, false), HPCDNN_FT_TA_NONE, HPCDNN_FT_TA_NONE, HPCDNN_FT_TA_FUSED(128, 64, false), HPCDNN_FT_TA_NONE}},
    {64, 64, {HPCDNN_FT_TA_KERNEL(64, 64, 2, 2, 0, false), HPCDNN_FT_TA_NONE, HPCDNN_FT_TA_NONE, HPCDNN_FT_TA_FUSED(64, 64, false), HPCDNN_FT_TA_NONE}},
};
}  // namespace

FtKernel ft_ta_kernel(int tile_class, int bm, int bn, int kind) {
    if (tile_class < 0 || tile_class >= HPCDNN_FT_NUM_CLASSES || kind < 0 || kind > 4) return HPCDNN_FT_TA_NONE;
    const FtTaClass& c = kFtTaClasses[tile_class];
    if (c.bm != bm || c.bn != bn) return HPCDNN_FT_TA_NONE;  // the two tables have drifted apart
    return c.kind[kind];
}

EncodeFn ft_ta_encode(int rows, int cols) {
    // the check tiles of the classes above, at either granularity
    if (rows == 256 && cols == 128) return abft_encode_kernel<256, 128, true>;
    if (rows == 128 && cols == 32) return abft_encode_kernel<128, 32, true>;
    if (rows == 128 && cols == 128) return abft_encode_kernel<128, 128, true>;
    if (rows == 64 && cols == 64) return abft_encode_kernel<64, 64, true>;
    if (rows == 64 && cols == 128) return abft_encode_kernel<64, 128, true>;
    if (rows == 32 && cols == 64) return abft_encode_kernel<32, 64, true>;
    if (rows == 128 && cols == 64) return abft_encode_kernel<128, 64, true>;
    return nullptr;
}

}  // namespace hpcdnn
