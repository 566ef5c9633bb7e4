// Host-side helpers shared by the SGEMM and ABFT-SGEMM entry points.
#pragma once

#include <mutex>

#include "sgemm_kernel.h"

namespace hpcdnn {

constexpr int kMaxLda = (1 << 21) - 64;    // 256 * lda * 4 < 2^31
constexpr int kMaxLdb = (1 << 25) - 1024;  // 16 * ldb * 4 + row < 2^31
constexpr int kMaxLdc = (1 << 21) - 64;    // 256 * ldc * 4 + row < 2^31

// ta: A is given transposed, K rows of M floats (row length lda >= M, at most kMaxLdb: a K step is 16 of its rows)
inline int check_gemm_args(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                           bool ta = false) {
    if (M < 0 || N < 0 || K < 0) return HPCDNN_ERR_INVALID_VALUE;
    const int a_cols = ta ? M : K;
    if (lda < (a_cols > 1 ? a_cols : 1) || ldb < (N > 1 ? N : 1) || ldc < (N > 1 ? N : 1)) return HPCDNN_ERR_INVALID_VALUE;
    if (M > 0 && N > 0 && !C) return HPCDNN_ERR_INVALID_VALUE;
    if (M > 0 && N > 0 && K > 0 && (!A || !B)) return HPCDNN_ERR_INVALID_VALUE;
    if ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B) | reinterpret_cast<uintptr_t>(C)) & 3u)
        return HPCDNN_ERR_INVALID_VALUE;
    // byte offsets inside one tile are 32-bit: 256 rows of A and of C, 16 rows of B
    if (lda > (ta ? kMaxLdb : kMaxLda) || ldb > kMaxLdb || ldc > kMaxLdc) return HPCDNN_ERR_INVALID_VALUE;
    return HPCDNN_OK;
}

inline GemmArgs make_args(int M, int N, int K, const float* A, int lda, const float* B, int ldb, float* C, int ldc,
                          float alpha, float beta, int bm, int bn) {
    GemmArgs a{};
    a.M = M; a.N = N; a.K = K;
    a.A = A; a.lda = lda; a.B = B; a.ldb = ldb; a.C = C; a.ldc = ldc;
    a.alpha = alpha; a.beta = beta;
    a.tiles_m = static_cast<int>(ceil_div(M, bm));
    a.tiles_n = static_cast<int>(ceil_div(N, bn));
    a.k_chunk = static_cast<int>(ceil_div(K > 0 ? K : 1, kGemmBK)) * kGemmBK;
    a.partial = nullptr;
    a.n_faults = 0;
    a.full_tiles = a.tiles_m * a.tiles_n;
    a.tail_split = 1;
    return a;
}

// The ragged-tile kernel masks the K tail and the columns past N; full tiles with K a multiple of the K step
// (per slice, which k_chunk guarantees for all but the last) skip that work.
inline bool needs_edge(const GemmArgs& a, int bm, int bn, int bk) {
    return !(a.M % bm == 0 && a.N % bn == 0 && a.K % bk == 0);
}

// The kernel of tile `tile` (bm x bn, as a cross-check of the index) for a transposed left operand, or nullptr when
// the tile has none (sgemm_ta.hip).
void (*sgemm_ta_kernel(int tile, int bm, int bn, bool edge))(const GemmArgs);
// Its persistent kernel (beta == 0 or beta != 0 variant), or nullptr; only tiles whose untransposed kernel has one
void (*sgemm_ta_persistent_kernel(int tile, int bm, int bn, bool beta))(const GemmArgs);

// An ABFT kernel: full-tile and ragged-tile instantiation, its workgroup size and LDS need
struct FtKernel {
    void (*plain)(const GemmArgs);
    void (*edge)(const GemmArgs);
    int threads;
    size_t lds;
};
typedef void (*EncodeFn)(int, int, int, const float*, int, const float*, int, float*, float*, int, int, int, int);

// ABFT tile classes: workgroup tile and the wave layout of the kernels that read their checksum vectors from the
// workspace (the wave tile, (bm / wgm) x (bn / wgn), is the check tile of wave-tile granularity)
struct FtGeom {
    int bm, bn, wgm, wgn;
};
constexpr FtGeom kFtGeom[HPCDNN_FT_NUM_CLASSES] = {{256, 128, 2, 4}, {128, 128, 2, 2}, {64, 128, 2, 2}, {128, 64, 2, 2}, {64, 64, 2, 2}};

// Kernel kinds of a class.  Fused: checksum vectors formed in the main loop (no workspace); pre: read from the
// workspace the pre-pass filled; wave: pre, with one checksum pair per wave tile; cad: with a verification every
// check_interval values of k; weighted: the weighted-checksum locator (two row sums of B from the workspace).
enum FtKind { kFtFused = 0, kFtFusedCad, kFtPre, kFtPreCad, kFtWave, kFtWaveCad, kFtWeighted, kFtKinds };

// One getter pair per (class, operand layout): each lives in its own translation unit (ft_kernels.hip compiled with
// -DHPCDNN_FT_CLASS / -DHPCDNN_FT_TA).  _ta1: the left operand is given transposed (K rows of M floats).
#define HPCDNN_FT_DECLARE(c)                  \
    FtKernel ft_kernel_c##c##_ta0(int kind);  \
    FtKernel ft_kernel_c##c##_ta1(int kind);  \
    EncodeFn ft_encode_c##c##_ta0(bool wave); \
    EncodeFn ft_encode_c##c##_ta1(bool wave);
HPCDNN_FT_DECLARE(0)
HPCDNN_FT_DECLARE(1)
HPCDNN_FT_DECLARE(2)
HPCDNN_FT_DECLARE(3)
HPCDNN_FT_DECLARE(4)
#undef HPCDNN_FT_DECLARE

// Kernels that use more than the default 64 KiB of LDS must opt in once per device.
inline int enable_lds(void (*fn)(const GemmArgs), size_t bytes) {
    if (bytes <= 64 * 1024) return HPCDNN_OK;
    struct Done {
        const void* fn;
        int device;
    };
    static std::mutex mu;
    static Done done[512] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return static_cast<int>(e);
    std::lock_guard<std::mutex> lock(mu);
    const void* key = reinterpret_cast<const void*>(fn);
    for (const Done& d : done)
        if (d.fn == key && d.device == dev) return HPCDNN_OK;
    e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
    if (e != hipSuccess) return static_cast<int>(e);
    for (Done& d : done)
        if (!d.fn) { d = Done{key, dev}; break; }  // a full table only costs a repeated call
    return HPCDNN_OK;
}

}  // namespace hpcdnn
