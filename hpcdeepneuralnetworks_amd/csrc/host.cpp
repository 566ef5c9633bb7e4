// Host-only entry points: version/error strings, workspace sizing, and the
// CPU GEMM validator the reference ships with its drivers.
#include <hip/hip_runtime_api.h>

#include "hpcdnn.h"

namespace hpcdnn {
size_t sdot_workspace_bytes();
size_t sgemm_workspace_bytes(int M, int N, int K);
size_t ft_workspace_bytes(int M, int N, int K);
size_t ft_cm_nt_workspace_bytes(int M, int N, int K);
size_t sgemv_workspace_bytes(int M, int N);
size_t offline_ft_workspace_bytes(int M, int N, int K);
}  // namespace hpcdnn

extern "C" const char* hpcdnn_version(void) { return "hpcdnn 0.1 (gfx950)"; }

extern "C" const char* hpcdnn_error_string(int code) {
    switch (code) {
        case HPCDNN_OK: return "success";
        case HPCDNN_ERR_INVALID_VALUE: return "invalid argument";
        case HPCDNN_ERR_WORKSPACE: return "workspace missing or too small";
        case HPCDNN_ERR_NOT_READY: return "one-time set-up needed: make one call outside stream capture first";
        default: return hipGetErrorString(static_cast<hipError_t>(code));
    }
}

extern "C" size_t hpcdnn_workspace_bytes(int op, int M, int N, int K) {
    switch (op) {
        case HPCDNN_OP_SGEMM: return hpcdnn::sgemm_workspace_bytes(M, N, K);
        case HPCDNN_OP_SDOT: return hpcdnn::sdot_workspace_bytes();
        case HPCDNN_OP_FT_SGEMM: return hpcdnn::ft_workspace_bytes(M, N, K);
        case HPCDNN_OP_FT_SGEMM_CM_NT: return hpcdnn::ft_cm_nt_workspace_bytes(M, N, K);
        case HPCDNN_OP_SGEMV: return hpcdnn::sgemv_workspace_bytes(M, N);
        case HPCDNN_OP_OFFLINE_FT_SGEMM: return hpcdnn::offline_ft_workspace_bytes(M, N, K);
        default: return 0;
    }
}

// utils/utils.cu:93-103 of the reference: i-j-k order, float accumulator,
// square, ld = n, C = alpha*(A*B) + beta*C.  Host pointers; validation aid only.
extern "C" void hpcdnn_cpu_gemm(float alpha, float beta, const float* mat1, const float* mat2, int n, float* mat3) {
    for (int i = 0; i < n; ++i) {
        const float* arow = mat1 + static_cast<size_t>(i) * n;
        float* crow = mat3 + static_cast<size_t>(i) * n;
        for (int j = 0; j < n; ++j) {
            float temp = 0.0f;
            for (int k = 0; k < n; ++k) temp += arow[k] * mat2[static_cast<size_t>(k) * n + j];
            crow[j] = alpha * temp + beta * crow[j];
        }
    }
}
