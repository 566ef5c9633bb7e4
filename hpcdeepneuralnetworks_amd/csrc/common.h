// Shared device/host helpers for the gfx950 kernels (wave64 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "hpcdnn.h"

namespace hpcdnn {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kWave = 64;

inline int launch_status() {
    hipError_t e = hipGetLastError();
    return (e == hipSuccess) ? HPCDNN_OK : static_cast<int>(e);
}

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Compute units of the current device (256 on an MI355X); 256 when no device can be queried.
inline int device_cus() {
    constexpr int kMaxDevices = 64;
    static int cus[kMaxDevices] = {};  // written once per device with the same value: racing threads agree
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
    if (cus[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
        cus[dev] = n;
    }
    return cus[dev];
}

// ---- counter-based RNG: splitmix64 finaliser of seed*golden + index ------
__host__ __device__ inline uint64_t mix64(uint64_t z) {
    z ^= z >> 30; z *= 0xBF58476D1CE4E5B9ull;
    z ^= z >> 27; z *= 0x94D049BB133111EBull;
    z ^= z >> 31;
    return z;
}

__host__ __device__ inline float uniform_pm1(uint64_t seed, uint64_t idx) {
    uint64_t z = mix64(seed * 0x9E3779B97F4A7C15ull + idx + 0x632BE59BD9B4E019ull);
    int32_t v = static_cast<int32_t>(z >> 40) - (1 << 23);
    return static_cast<float>(v) * (1.0f / 8388608.0f);
}

// ---- cross-lane primitives (DPP / swizzle; no LDS traffic) ----------------
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
}

constexpr int kDppXor1 = 0xB1;        // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;        // quad_perm [2,3,0,1]
constexpr int kDppHalfMirror = 0x141; // lane i <-> 7-i inside each 8
constexpr int kDppMirror = 0x140;     // lane i <-> 15-i inside each 16
constexpr int kDppBcast15 = 0x142;    // lane 15 of each row -> next row
constexpr int kDppBcast31 = 0x143;    // lane 31 -> rows 2,3

// Sum over the 16 lanes of each DPP row; every lane of the row gets the sum.
__device__ __forceinline__ float row16_allsum(float v) {
    v += dpp_mov<kDppXor1>(v);
    v += dpp_mov<kDppXor2>(v);
    v += dpp_mov<kDppHalfMirror>(v);
    v += dpp_mov<kDppMirror>(v);
    return v;
}

// Sum over each 32-lane half of the wave; every lane of the half gets the sum.
__device__ __forceinline__ float half32_allsum(float v) {
    v = row16_allsum(v);
    // swap with lane ^ 16: bit-mask swizzle, and=0x1f or=0 xor=0x10
    v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
    return v;
}

// Value of lane (l ^ X) for X = 1, 2 (DPP quad permutes) or 4, 8, 16 (bit-mask swizzles).
template <int X>
__device__ __forceinline__ float lane_xor(float v) {
    static_assert(X == 1 || X == 2 || X == 4 || X == 8 || X == 16, "partner inside a 32-lane half");
    if constexpr (X == 1) return dpp_mov<kDppXor1>(v);
    else if constexpr (X == 2) return dpp_mov<kDppXor2>(v);
    else return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x1F | (X << 10)));
}

// Transposing sum over each 32-lane half of the wave.  On entry every lane holds N values (N = 16 or 32); on return
// v[0] of lane l holds the sum over the lanes of its half of value l % N.  Each stage halves the values a lane keeps
// and doubles the lanes summed into them (lane bit b decides which of a pair stays and which travels), so the whole
// costs N - 1 additions per lane instead of 5 N for N separate all-reduces.  The order of the additions is fixed.
template <int N>
__device__ __forceinline__ void half32_transpose_sum(float (&v)[N], int lane) {
    static_assert(N == 16 || N == 32, "16 or 32 values per lane");
    auto stage = [&](auto bit, auto count) {
        constexpr int B = decltype(bit)::value, C = decltype(count)::value;
        const bool up = (lane >> B) & 1;
        float send[C / 2];
#pragma unroll
        for (int i = 0; i < C / 2; ++i) {
            send[i] = up ? v[2 * i] : v[2 * i + 1];
            v[i] = up ? v[2 * i + 1] : v[2 * i];
        }
#pragma unroll
        for (int i = 0; i < C / 2; ++i) send[i] = lane_xor<(1 << B)>(send[i]);
#pragma unroll
        for (int i = 0; i < C / 2; ++i) v[i] += send[i];
    };
    using std::integral_constant;
    stage(integral_constant<int, 0>{}, integral_constant<int, N>{});
    stage(integral_constant<int, 1>{}, integral_constant<int, N / 2>{});
    stage(integral_constant<int, 2>{}, integral_constant<int, N / 4>{});
    stage(integral_constant<int, 3>{}, integral_constant<int, N / 8>{});
    if constexpr (N == 32) stage(integral_constant<int, 4>{}, integral_constant<int, 2>{});
    else v[0] += lane_xor<16>(v[0]);
}

// Maximum over each 32-lane half of the wave; every lane of the half gets it.
__device__ __forceinline__ float half32_allmax(float v) {
    v = __builtin_fmaxf(v, dpp_mov<kDppXor1>(v));
    v = __builtin_fmaxf(v, dpp_mov<kDppXor2>(v));
    v = __builtin_fmaxf(v, dpp_mov<kDppHalfMirror>(v));
    v = __builtin_fmaxf(v, dpp_mov<kDppMirror>(v));
    return __builtin_fmaxf(v, lane_xor<16>(v));
}

// Sum over the whole wave; the total is valid in lane 63 only.
__device__ __forceinline__ float wave_sum_lane63(float v) {
    v = row16_allsum(v);
    v += dpp_mov<kDppBcast15, 0xa>(v);
    v += dpp_mov<kDppBcast31, 0xc>(v);
    return v;
}

// ---- buffer addressing --------------------------------------------------
// Raw buffer descriptor over [base, base + bytes), bytes >= 0: loads past the end return 0.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const float* base, int64_t bytes) {
    // bytes >= 0.  Clamped to 2^32 - 1 by looking at the upper half only: the value is wave-uniform, and a 32-bit
    // compare stays on the scalar unit (a 64-bit signed one would occupy the vector unit the MFMAs need).
    unsigned hi = static_cast<unsigned>(static_cast<uint64_t>(bytes) >> 32);
    asm volatile("" : "+s"(hi));  // keeps the compiler from fusing the test below back into a 64-bit compare
    const unsigned lo = static_cast<unsigned>(bytes);
    const unsigned clipped = hi != 0u ? 0xFFFFFFFFu : lo;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, static_cast<int>(clipped), 0x00020000);
}

// Descriptor without an end, for accesses known to stay inside the allocation.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc_unbounded(const float* base) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, -1, 0x00020000);
}

__device__ __forceinline__ v4f buffer_load_v4f(__amdgpu_buffer_rsrc_t rsrc, int byte_offset) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 0);
    return __builtin_bit_cast(v4f, v);
}

// Four consecutive floats from an address that is only 4-byte aligned and differs from lane to lane (a buffer
// descriptor wants a wave-uniform base: with a per-lane one the compiler loops over the lanes).
__device__ __forceinline__ v4f load_v4f_words(const float* p) {
    struct __attribute__((aligned(4))) words {
        float x, y, z, w;
    };
    const words t = *reinterpret_cast<const words*>(p);
    return v4f{t.x, t.y, t.z, t.w};
}

// The same with the non-temporal hint, for data that is read once (aux bit 1 of the raw buffer instructions).
__device__ __forceinline__ v4f buffer_load_v4f_nt(__amdgpu_buffer_rsrc_t rsrc, int byte_offset) {
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    const v4u v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 2);
    return __builtin_bit_cast(v4f, v);
}

// Fixed-order sum of many slices, C = alpha * (ws[0] + ws[1] + ...) + beta * C with ws = [splits][M][N] (N a multiple
// of 4, 16-byte aligned): the second phase of split-K SGEMM and of the transposed SGEMV.  Four lanes share a group of four
// consecutive elements, each adds a quarter of the slices in slice order (up to 32 16-byte loads in flight, so
// 128 slices cost one trip to memory where a lane that walks them eight at a time makes eight), and the four partial
// sums are combined as
// (q0 + q1) + (q2 + q3) by exchanges with lane ^ 16 and lane ^ 32: a fixed order, the same bits on every run.
// A wave covers 16 groups (256 contiguous bytes per slice) x 4 quarters; a block is kWaves waves (one when there are
// so few elements that blocks of four would leave most CUs without one).
template <int kWaves = 4>
__global__ __launch_bounds__(64 * kWaves) void splitk_reduce_wide_kernel(int M, int N, int splits, const float* __restrict__ ws,
                                                                 float* __restrict__ C, int ldc, float alpha, float beta) {
    const int64_t total = static_cast<int64_t>(M) * N;
    const int lane = threadIdx.x & (kWave - 1);
    const int q = lane >> 4;
    const int64_t e = (static_cast<int64_t>(blockIdx.x) * (16 * kWaves) + (threadIdx.x / kWave) * 16 + (lane & 15)) * 4;
    const int per = (splits + 3) / 4;
    const int z0 = q * per, z1 = (z0 + per < splits) ? z0 + per : splits;
    v4f s = {0.f, 0.f, 0.f, 0.f};
    if (e < total) {
        // all of a lane's slices in one batch when they are few, else 32 at a time
        auto add_slices = [&](auto batch) {
            constexpr int kBatch = decltype(batch)::value;
            for (int z = z0; z < z1; z += kBatch) {
                v4f t[kBatch];
#pragma unroll
                for (int u = 0; u < kBatch; ++u)
                    t[u] = (z + u < z1) ? *reinterpret_cast<const v4f*>(ws + static_cast<size_t>(z + u) * total + e) : v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int u = 0; u < kBatch; ++u) s += t[u];
            }
        };
        if (per <= 8) add_slices(std::integral_constant<int, 8>{});
        else add_slices(std::integral_constant<int, 32>{});
    }
    float sv[4] = {s.x, s.y, s.z, s.w};
    const int x32_addr = (lane ^ 32) * 4;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        sv[c] += lane_xor<16>(sv[c]);
        sv[c] += __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(x32_addr, __builtin_bit_cast(int, sv[c])));
    }
    if (q == 0 && e < total) {
        const int64_t r = e / N, c0 = e - r * N;
        float* dst = C + r * ldc + c0;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float t = alpha * sv[c];
            dst[c] = (beta == 0.f) ? t : __builtin_fmaf(beta, dst[c], t);
        }
    }
}

// Launch of the kernel above: one-wave blocks while blocks of four waves would number fewer than the CUs.
inline void launch_splitk_reduce_wide(int M, int N, int splits, const float* ws, float* C, int ldc, float alpha, float beta,
                                      int cus, hipStream_t stream) {
    const int64_t total = static_cast<int64_t>(M) * N;
    if (total < static_cast<int64_t>(cus) * 256)
        splitk_reduce_wide_kernel<1><<<static_cast<int>((total + 63) / 64), 64, 0, stream>>>(M, N, splits, ws, C, ldc, alpha, beta);
    else
        splitk_reduce_wide_kernel<4><<<static_cast<int>((total + 255) / 256), 256, 0, stream>>>(M, N, splits, ws, C, ldc, alpha, beta);
}

}  // namespace hpcdnn
