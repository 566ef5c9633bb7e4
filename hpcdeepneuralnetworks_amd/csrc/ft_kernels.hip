// The ABFT-SGEMM kernels of ONE tile class for ONE operand layout: compiled once per (class, layout) pair with
// -DHPCDNN_FT_CLASS=0..4 -DHPCDNN_FT_TA=0|1, so that the instantiations build side by side.  Every class has every
// kind (the reference ships an ABFT kernel with the in-loop check for every shape of its table,
// kernel/ft_sgemm/code_gen/main.py:8-16, kernel/ft_sgemm/sgemm.cu:186-192, kernel/ft_sgemm/include/ft_sgemm_large.cuh:337,
// ft_sgemm_tall.cuh:18): checksum vectors formed in the main loop or read from the workspace, one checksum pair per
// workgroup tile or per wave tile, one verification or one every check_interval values of k.
#include "gemm_host.h"

#if !defined(HPCDNN_FT_CLASS) || !defined(HPCDNN_FT_TA)
#error "compile with -DHPCDNN_FT_CLASS=<0..4> -DHPCDNN_FT_TA=<0|1>"
#endif

namespace hpcdnn {

namespace {
constexpr FtGeom kGeom = kFtGeom[HPCDNN_FT_CLASS];
constexpr bool kTa = HPCDNN_FT_TA != 0;

// the kernels without a workspace run four waves (2 x 2), those with one the class's own wave layout (ft_sgemm.hip)
// (two staging sets in every class: the ABFT loop with four of them, tried on the 64-column classes for the products that
// stream an operand from memory, measured 10-20 % slower on every shape)
constexpr int kSlots = 2;

template <int FT, int GRAN, bool CAD>
FtKernel make_kernel() {
    constexpr int WGM = FT == 1 ? 2 : kGeom.wgm, WGN = FT == 1 ? 2 : kGeom.wgn;
    // The classes below 256 x 128 run four waves per workgroup and are built for two workgroups per CU, which cover each
    // other's prologue, verification and epilogue: their kernels are held to the 256 registers per lane that this takes
    // (the cadence kernels of the 128 x 128 class had grown to 268 and ran alone on their CU: +25 % instead of +17 %).
    // (the 256 x 128 class has 128 accumulators per lane in its four-wave kernels: one workgroup per CU)
    constexpr int kMinBlocks = HPCDNN_FT_CLASS == 0 ? 1 : 2;
    return FtKernel{sgemm_kernel<kGeom.bm, kGeom.bn, WGM, WGN, false, FT, kMinBlocks, kSlots, GRAN, CAD, kTa>,
                    sgemm_kernel<kGeom.bm, kGeom.bn, WGM, WGN, true, FT, kMinBlocks, kSlots, GRAN, CAD, kTa>, WGM * WGN * kWave,
                    gemm_lds_bytes<kGeom.bm, kGeom.bn, FT, WGM * WGN * kWave, WGM, WGN, GRAN>()};
}
}  // namespace

#define HPCDNN_FT_PASTE_(a, b, c, d) a##b##c##d
#define HPCDNN_FT_PASTE(a, b, c, d) HPCDNN_FT_PASTE_(a, b, c, d)

FtKernel HPCDNN_FT_PASTE(ft_kernel_c, HPCDNN_FT_CLASS, _ta, HPCDNN_FT_TA)(int kind) {
    switch (kind) {
        case kFtFused: return make_kernel<1, 0, false>();
        case kFtFusedCad: return make_kernel<1, 0, true>();
        case kFtPre: return make_kernel<2, 0, false>();
        case kFtPreCad: return make_kernel<2, 0, true>();
        case kFtWave: return make_kernel<2, 1, false>();
        case kFtWaveCad: return make_kernel<2, 1, true>();
        case kFtWeighted: return make_kernel<3, 0, false>();
        default: return FtKernel{nullptr, nullptr, 0, 0};
    }
}

// the pre-pass over both operands for this class's check tiles at either granularity
EncodeFn HPCDNN_FT_PASTE(ft_encode_c, HPCDNN_FT_CLASS, _ta, HPCDNN_FT_TA)(bool wave) {
    if (wave) return abft_encode_kernel<kGeom.bm / kGeom.wgm, kGeom.bn / kGeom.wgn, kTa>;
    return abft_encode_kernel<kGeom.bm, kGeom.bn, kTa>;
}

}  // namespace hpcdnn
