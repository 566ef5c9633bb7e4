// SAXPY, SDOT and the seeded fill kernels: HBM-bandwidth-bound streams.
//
// Layout: contiguous FP32 vectors.  Algorithmic traffic: SAXPY 12 B/element
// (two loads, one store), SDOT 8 B/element (two loads).  Launch shapes follow
// what the HBM3E stacks of this part sustain: for the read+write stream of
// SAXPY many one-wave workgroups, 8 bytes per lane (a grid-stride loop
// that runs once unless n exceeds the grid cap), reach ~7.1 TB/s where
// long-running grid-stride blocks stay near 4.6 TB/s; for the read-only stream
// of SDOT one workgroup per CU walks one contiguous slice of both vectors with
// four 16-byte loads per vector in flight (~7.2 TB/s against ~6.0 TB/s
// grid-stride).
// All streaming accesses carry the non-temporal hint.
#include "common.h"

namespace hpcdnn {

constexpr int kVecThreads = 256;

// ------------------------------------------------------------------ SAXPY --
// Stands in for saxpy / saxpy3 / _saxpy (kernel/saxpy/saxpy.cu:15-48).  The
// reference's f128 kernels need n % 4 == 0 and 16-byte alignment; here any n
// and any pair of pointers with the same alignment modulo 8 take the vector
// kernel (a leading and a trailing single element are done by two lanes of
// block 0), and the rest takes the dword kernel.
//
// One wave per workgroup and 8 bytes per lane: a wave moves 512 contiguous
// bytes of x and of y.  The memory system sustains more the smaller and the
// shorter-lived the waves are (n = 2^28, 12 B/element: 16 bytes per lane in
// 256-thread workgroups 6.4 TB/s, in 64-thread workgroups 6.65, 8 bytes per
// lane in 64-thread workgroups 7.1): the requests then reach the DRAM
// channels in address order at the pace the dispatcher launches waves, which
// at 512 bytes per wave is just below what the channels can take (4 bytes per
// lane is bound by the wave launch rate at 3.6 TB/s).  Loads carry the
// non-temporal hint, stores write through (sc0 sc1 nt): measured 1-3 % over
// non-temporal stores alone, and less dependent on where x and y lie.
constexpr int kSaxpyThreads = 64;
constexpr int64_t kSaxpySegment = int64_t{1} << 29;  // elements per launch: byte offsets stay below 2^31
constexpr int kAuxNt = 2;            // cache-policy bits of the raw buffer instructions on gfx950: sc0 = 1, nt = 2, sc1 = 16
constexpr int kAuxWriteThroughNt = 19;

// One launch covers `nbytes` (a multiple of 8, at most 4 * kSaxpySegment) of x and y from 8-byte aligned xb, yb.
// The whole byte offset of a lane goes into the vector offset of one descriptor over the segment: rebasing the
// descriptor per wave, or moving the wave's part into the scalar offset, measured 3 % slower.  Lanes past the end
// load zeros and their stores are dropped by the descriptor's range check.
// extra bit 0: also do the single element in front of the segment (xb[-1]); bit 1: the one behind it.
__global__ __launch_bounds__(kSaxpyThreads) void saxpy_vec2_kernel(unsigned nbytes, float alpha, const float* __restrict__ xb,
                                                                   float* __restrict__ yb, int extra) {
    typedef float v2f __attribute__((ext_vector_type(2)));
    typedef unsigned v2u __attribute__((ext_vector_type(2)));
    const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(xb), 0, nbytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t ry = __builtin_amdgcn_make_buffer_rsrc(yb, 0, nbytes, 0x00020000);
    const unsigned off = blockIdx.x * (kSaxpyThreads * 8) + threadIdx.x * 8;
    const v2f xv = __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(rx, off, 0, kAuxNt));
    const v2f yv = __builtin_bit_cast(v2f, __builtin_amdgcn_raw_buffer_load_b64(ry, off, 0, kAuxNt));
    v2f r;
    r.x = __builtin_fmaf(alpha, xv.x, yv.x);
    r.y = __builtin_fmaf(alpha, xv.y, yv.y);
    __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(v2u, r), ry, off, 0, kAuxWriteThroughNt);
    if (blockIdx.x == 0 && extra != 0 && threadIdx.x < 2) {
        const int64_t t = threadIdx.x == 0 ? -1 : static_cast<int64_t>(nbytes >> 2);
        if (extra & (1 << threadIdx.x)) yb[t] = __builtin_fmaf(alpha, xb[t], yb[t]);
    }
}

__global__ __launch_bounds__(kVecThreads) void saxpy_dword_kernel(int64_t n, float alpha, const float* __restrict__ x,
                                                                  float* __restrict__ y) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kVecThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kVecThreads + threadIdx.x; i < n; i += stride)
        y[i] = __builtin_fmaf(alpha, x[i], y[i]);
}

// ------------------------------------------------------------------- SDOT --
// Stands in for _sdot (grid-stride + shared-memory tree + float atomicAdd,
// kernel/sdot/sdot.cu:9-36) and for the sdot + reduction multi-launch chain
// (:38-67).  One launch, no float atomics: every block publishes one partial,
// and block 0 collects the partials and adds them in index order, so the result
// is reproducible bit for bit.
//
// Workspace layout: [0] epoch (uint32: the number of calls completed on this
// workspace), [64..] two 64-bit words per block, each holding the epoch tag of
// the call that wrote it in its upper half and one half of the block's double
// partial in its lower half.
constexpr int kSdotMaxBlocks = 4096;
constexpr int kSdotVecBlocks = 256;  // one workgroup per CU of an MI355X: fewest tickets and partials, full bandwidth
constexpr size_t kSdotPartialOffset = 64;

__device__ __forceinline__ double block_sum_to_thread0(double v, double* lds) {
    // lanes -> wave via bpermute shuffles (tail of the kernel, not hot)
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
    __syncthreads();
    double s = 0.0;
    if (threadIdx.x == 0) {
#pragma unroll
        for (int w = 0; w < kVecThreads / kWave; ++w) s += lds[w];
    }
    return s;
}

constexpr int kSdotSpinLimit = 1 << 20;  // polls before block 0 gives up on a block (about a second)

template <int UNROLL, bool VEC>
__global__ __launch_bounds__(kVecThreads) void sdot_kernel(int64_t n, const float* __restrict__ x,
                                                           const float* __restrict__ y, float* __restrict__ out,
                                                           unsigned int* epoch, unsigned long long* slots) {
    __shared__ double lds[kVecThreads / kWave];
    __shared__ unsigned int s_tag;
    // this call's number: one more than the calls completed on this workspace (read now, needed after the sums)
    unsigned int tag = 0;
    if (threadIdx.x == 0) tag = __hip_atomic_load(epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u;
    float acc[UNROLL][4];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc[u][0] = acc[u][1] = acc[u][2] = acc[u][3] = 0.0f;

    if (VEC) {
        // workgroup b owns the contiguous slice [b*per, (b+1)*per) of 16-byte groups
        const int64_t n4 = n >> 2;
        const v4f* __restrict__ x4 = reinterpret_cast<const v4f*>(x);
        const v4f* __restrict__ y4 = reinterpret_cast<const v4f*>(y);
        const int64_t per = (n4 + gridDim.x - 1) / gridDim.x;
        const int64_t beg = static_cast<int64_t>(blockIdx.x) * per;
        const int64_t end = (beg + per < n4) ? beg + per : n4;
        int64_t i = beg + threadIdx.x;
        for (; i + (UNROLL - 1) * kVecThreads < end; i += UNROLL * kVecThreads) {
            v4f xv[UNROLL], yv[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) xv[u] = __builtin_nontemporal_load(&x4[i + u * kVecThreads]);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) yv[u] = __builtin_nontemporal_load(&y4[i + u * kVecThreads]);
            __builtin_amdgcn_sched_barrier(0);  // all 2*UNROLL loads are in flight before the first FMA waits
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                acc[u][0] = __builtin_fmaf(xv[u].x, yv[u].x, acc[u][0]);
                acc[u][1] = __builtin_fmaf(xv[u].y, yv[u].y, acc[u][1]);
                acc[u][2] = __builtin_fmaf(xv[u].z, yv[u].z, acc[u][2]);
                acc[u][3] = __builtin_fmaf(xv[u].w, yv[u].w, acc[u][3]);
            }
        }
        for (; i < end; i += kVecThreads) {
            const v4f xv = x4[i], yv = y4[i];
            acc[0][0] = __builtin_fmaf(xv.x, yv.x, acc[0][0]);
            acc[0][1] = __builtin_fmaf(xv.y, yv.y, acc[0][1]);
            acc[0][2] = __builtin_fmaf(xv.z, yv.z, acc[0][2]);
            acc[0][3] = __builtin_fmaf(xv.w, yv.w, acc[0][3]);
        }
        if (blockIdx.x == 0) {
            const int64_t t = (n4 << 2) + threadIdx.x;
            if (t < n) acc[0][0] = __builtin_fmaf(x[t], y[t], acc[0][0]);
        }
    } else {
        const int64_t stride = static_cast<int64_t>(gridDim.x) * kVecThreads;
        for (int64_t i = static_cast<int64_t>(blockIdx.x) * kVecThreads + threadIdx.x; i < n; i += stride)
            acc[0][0] = __builtin_fmaf(x[i], y[i], acc[0][0]);
    }

    // Fixed-order combine of this lane's accumulators, in double from here on.
    double v = 0.0;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
        v += (static_cast<double>(acc[u][0]) + static_cast<double>(acc[u][1])) +
             (static_cast<double>(acc[u][2]) + static_cast<double>(acc[u][3]));
    const double block_total = block_sum_to_thread0(v, lds);

    // Cross-block hand-off without cache-wide fences (a device-scope release/acquire fence writes back and
    // invalidates the whole L2 of the XCD, which costs a streaming kernel a quarter of its bandwidth) and without a
    // chain of dependent read-modify-writes (exchange, ticket, read-back: three trips to the point of coherence, which
    // is most of a short call).  Every block stores its partial as two device-scope 64-bit words, each tagged with
    // this call's number; block 0 polls the words of every block until both carry the tag - a word is written whole,
    // so a matching tag means its payload is this call's - and adds the partials in index order.  No value of a
    // partial is special: stale words are told apart by their tag, which differs from call to call.  Hardware
    // assumption: device-scope (sc1) stores and loads of an aligned 64-bit word are single accesses at the point of
    // coherence shared by the XCDs.  Every block but block 0 ends without waiting; block 0 waits for blocks that are
    // running or will run once a CU is free, and gives up (NaN result) after a bounded number of polls.
    if (threadIdx.x == 0) {
        const unsigned long long bits = __builtin_bit_cast(unsigned long long, block_total);
        const unsigned long long tag_hi = static_cast<unsigned long long>(tag) << 32;
        __hip_atomic_store(&slots[2 * blockIdx.x], tag_hi | (bits & 0xffffffffull), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&slots[2 * blockIdx.x + 1], tag_hi | (bits >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_tag = tag;
    }
    if (blockIdx.x != 0) return;
    __syncthreads();
    const unsigned int want = s_tag;
    double s = 0.0;
    int missing = 0;
    for (unsigned int b = threadIdx.x; b < gridDim.x; b += kVecThreads) {
        unsigned long long lo = 0, hi = 0;
        int spin = 0;
        for (; spin < kSdotSpinLimit; ++spin) {
            lo = __hip_atomic_load(&slots[2 * b], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            hi = __hip_atomic_load(&slots[2 * b + 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (static_cast<unsigned int>(lo >> 32) == want && static_cast<unsigned int>(hi >> 32) == want) break;
            __builtin_amdgcn_s_sleep(1);
        }
        missing += spin == kSdotSpinLimit;
        s += __builtin_bit_cast(double, (hi << 32) | (lo & 0xffffffffull));
    }
    missing = __syncthreads_or(missing);  // (also the barrier before lds is reused)
    const double total = block_sum_to_thread0(s, lds);
    if (threadIdx.x == 0) {
        *out = missing ? __builtin_nanf("") : static_cast<float>(total);
        __hip_atomic_store(epoch, want, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // the next stream-ordered call is number want + 1
    }
}

// ------------------------------------------------------------------ fills --
__global__ __launch_bounds__(kVecThreads) void fill_uniform_kernel(float* __restrict__ dst, int64_t n, uint64_t seed) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kVecThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kVecThreads + threadIdx.x; i < n; i += stride)
        dst[i] = uniform_pm1(seed, static_cast<uint64_t>(i));
}

__global__ __launch_bounds__(kVecThreads) void fill_uniform_matrix_kernel(float* __restrict__ dst, int rows, int cols,
                                                                          int ld, uint64_t seed) {
    const int64_t total = static_cast<int64_t>(rows) * cols;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kVecThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kVecThreads + threadIdx.x; i < total; i += stride) {
        const int64_t r = i / cols, c = i - r * cols;
        dst[r * ld + c] = uniform_pm1(seed, static_cast<uint64_t>(i));
    }
}

__global__ __launch_bounds__(kVecThreads) void zero_words_kernel(uint32_t* __restrict__ dst, int64_t nwords) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kVecThreads;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * kVecThreads + threadIdx.x; i < nwords; i += stride) dst[i] = 0u;
}

// ------------------------------------------------------------- launch glue --
static int stream_grid(int64_t work_items, int blocks_per_cu) {
    int64_t want = ceil_div(work_items, kVecThreads);
    int64_t cap = static_cast<int64_t>(device_cus()) * blocks_per_cu;
    if (want < 1) want = 1;
    return static_cast<int>(want < cap ? want : cap);
}

}  // namespace hpcdnn

using namespace hpcdnn;

extern "C" int hpcdnn_saxpy(int64_t n, float alpha, const float* x, float* y, void* stream) {
    if (n < 0 || (n > 0 && (!x || !y))) return HPCDNN_ERR_INVALID_VALUE;
    if (n == 0) return HPCDNN_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 3u) return HPCDNN_ERR_INVALID_VALUE;
    // the vector kernel pairs elements on 8-byte boundaries: x and y must agree modulo 8
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) ^ reinterpret_cast<uintptr_t>(y)) & 7u) == 0;
    if (aligned) {
        // a leading element when both pointers are 4 bytes off an 8-byte boundary, pairs, a trailing element
        const int head = static_cast<int>((reinterpret_cast<uintptr_t>(x) >> 2) & 1);
        const int64_t pairs = (n - head) >> 1;
        const bool tail = head + 2 * pairs < n;
        const float* xb = x + head;
        float* yb = y + head;
        int64_t done = 0;
        do {
            const int64_t left = 2 * pairs - done;
            const int64_t count = left < kSaxpySegment ? left : kSaxpySegment;
            const bool last = done + count == 2 * pairs;
            const int extra = ((done == 0 && head) ? 1 : 0) | ((last && tail) ? 2 : 0);
            const unsigned nbytes = static_cast<unsigned>(count * 4);
            const int64_t grid = count > 0 ? ceil_div(count * 4, kSaxpyThreads * 8) : 1;
            saxpy_vec2_kernel<<<static_cast<int>(grid), kSaxpyThreads, 0, s>>>(nbytes, alpha, xb + done, yb + done, extra);
            done += count;
        } while (done < 2 * pairs);
    } else {
        const int grid = stream_grid(n, 16);
        saxpy_dword_kernel<<<grid, kVecThreads, 0, s>>>(n, alpha, x, y);
    }
    return launch_status();
}

extern "C" int hpcdnn_sdot(int64_t n, const float* x, const float* y, float* out, void* ws, size_t ws_bytes,
                           void* stream) {
    if (n < 0 || !out || (n > 0 && (!x || !y))) return HPCDNN_ERR_INVALID_VALUE;
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 3u) return HPCDNN_ERR_INVALID_VALUE;
    if (!ws || ws_bytes < hpcdnn_workspace_bytes(HPCDNN_OP_SDOT, 0, 0, 0)) return HPCDNN_ERR_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(ws) & 7u) return HPCDNN_ERR_INVALID_VALUE;  // the block partials are doubles
    hipStream_t s = static_cast<hipStream_t>(stream);
    unsigned int* ticket = static_cast<unsigned int*>(ws);  // the epoch word
    unsigned long long* partials = reinterpret_cast<unsigned long long*>(static_cast<char*>(ws) + kSdotPartialOffset);
    const bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15u) == 0;
    if (aligned) {
        // one slice of >= 4096 elements per workgroup, 256 workgroups at most: a function of n only, so the
        // summation order (and the result's bits) do not depend on the device
        int64_t grid = ceil_div((n >> 2) + 1, 1024);
        if (grid > kSdotVecBlocks) grid = kSdotVecBlocks;
        sdot_kernel<4, true><<<static_cast<int>(grid), kVecThreads, 0, s>>>(n, x, y, out, ticket, partials);
    } else {
        int64_t grid = ceil_div(n + 1, 1024);
        if (grid > kSdotVecBlocks) grid = kSdotVecBlocks;
        sdot_kernel<1, false><<<static_cast<int>(grid), kVecThreads, 0, s>>>(n, x, y, out, ticket, partials);
    }
    return launch_status();
}

extern "C" int hpcdnn_workspace_init(void* ws, size_t ws_bytes, void* stream) {
    if (ws_bytes == 0) return HPCDNN_OK;
    if (!ws || (reinterpret_cast<uintptr_t>(ws) & 3u) || (ws_bytes & 3u)) return HPCDNN_ERR_INVALID_VALUE;
    const int64_t words = static_cast<int64_t>(ws_bytes / 4);
    zero_words_kernel<<<stream_grid(words, 8), kVecThreads, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint32_t*>(ws), words);
    return launch_status();
}

extern "C" int hpcdnn_fill_uniform(float* dst, int64_t n, uint64_t seed, void* stream) {
    if (n < 0 || (n > 0 && !dst)) return HPCDNN_ERR_INVALID_VALUE;
    if (n == 0) return HPCDNN_OK;
    fill_uniform_kernel<<<stream_grid(n, 8), kVecThreads, 0, static_cast<hipStream_t>(stream)>>>(dst, n, seed);
    return launch_status();
}

extern "C" int hpcdnn_fill_uniform_matrix(float* dst, int rows, int cols, int ld, uint64_t seed, void* stream) {
    if (rows < 0 || cols < 0 || ld < cols || (rows > 0 && cols > 0 && !dst)) return HPCDNN_ERR_INVALID_VALUE;
    if (rows == 0 || cols == 0) return HPCDNN_OK;
    const int64_t total = static_cast<int64_t>(rows) * cols;
    fill_uniform_matrix_kernel<<<stream_grid(total, 8), kVecThreads, 0, static_cast<hipStream_t>(stream)>>>(
        dst, rows, cols, ld, seed);
    return launch_status();
}

namespace hpcdnn {
size_t sdot_workspace_bytes() { return kSdotPartialOffset + sizeof(double) * kSdotMaxBlocks; }
}  // namespace hpcdnn
