// Two bare streaming kernels that measure what the memory system delivers to the simplest possible consumer: a
// read-only pass (16-byte loads folded into one word per workgroup) and a copy.  The benchmark reports them next to
// the library's kernels, so that a kernel's distance from the published peak can be split into what no kernel gets
// and what this kernel loses.  No counterpart in the reference.

#include "ahq_device.h"
#include "ahq_host.h"

namespace ahq {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
constexpr int kDiagThreads = 256;
constexpr int kDiagUnroll = 4;

template <bool NT>
__global__ __launch_bounds__(kDiagThreads) void diag_read_kernel(const u32x4* __restrict__ x, int64_t nvec,
                                                                 uint32_t* __restrict__ out) {
    uint32_t acc = 0;
    const int64_t stride = (int64_t)gridDim.x * kDiagThreads * kDiagUnroll;
    for (int64_t base = (int64_t)blockIdx.x * kDiagThreads * kDiagUnroll + threadIdx.x; base < nvec; base += stride) {
        u32x4 v[kDiagUnroll];
#pragma unroll
        for (int u = 0; u < kDiagUnroll; ++u) {
            const int64_t i = base + (int64_t)u * kDiagThreads;
            v[u] = i >= nvec ? u32x4{0u, 0u, 0u, 0u} : NT ? __builtin_nontemporal_load(x + i) : x[i];
        }
#pragma unroll
        for (int u = 0; u < kDiagUnroll; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
#pragma unroll
    for (int m = kWave / 2; m >= 1; m >>= 1) acc ^= __shfl_xor(acc, m, kWave);
    __shared__ uint32_t part[kDiagThreads / kWave];
    if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t r = 0;
        for (int w = 0; w < kDiagThreads / kWave; ++w) r ^= part[w];
        out[blockIdx.x] = r;
    }
}

__global__ __launch_bounds__(kDiagThreads) void diag_copy_kernel(const u32x4* __restrict__ x, u32x4* __restrict__ y,
                                                                 int64_t nvec) {
    const int64_t stride = (int64_t)gridDim.x * kDiagThreads * kDiagUnroll;
    for (int64_t base = (int64_t)blockIdx.x * kDiagThreads * kDiagUnroll + threadIdx.x; base < nvec; base += stride) {
        u32x4 v[kDiagUnroll];
#pragma unroll
        for (int u = 0; u < kDiagUnroll; ++u) {
            const int64_t i = base + (int64_t)u * kDiagThreads;
            if (i < nvec) v[u] = __builtin_nontemporal_load(x + i);
        }
#pragma unroll
        for (int u = 0; u < kDiagUnroll; ++u) {
            const int64_t i = base + (int64_t)u * kDiagThreads;
            if (i < nvec) __builtin_nontemporal_store(v[u], y + i);
        }
    }
}

}  // namespace ahq

using namespace ahq;

extern "C" int ahq_diag_read(const void* x, size_t bytes, int32_t workgroups, int32_t nontemporal, uint32_t* out,
                             void* stream) {
    if (!x || !out) return set_error("null argument"), AHQ_ERR_INVALID;
    if (bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(x) & 15u)) return set_error("x must be 16-byte aligned and a multiple of 16 bytes long"), AHQ_ERR_INVALID;
    if (workgroups < 1 || workgroups > 65536) return set_error("workgroups must be in 1..65536"), AHQ_ERR_INVALID;
    if (bytes == 0) return AHQ_OK;
    if (nontemporal)
        hipLaunchKernelGGL(diag_read_kernel<true>, dim3((unsigned)workgroups), dim3(kDiagThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<const u32x4*>(x), (int64_t)(bytes / 16), out);
    else
        hipLaunchKernelGGL(diag_read_kernel<false>, dim3((unsigned)workgroups), dim3(kDiagThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<const u32x4*>(x), (int64_t)(bytes / 16), out);
    return check_launch("ahq_diag_read");
}

extern "C" int ahq_diag_copy(const void* x, void* y, size_t bytes, int32_t workgroups, void* stream) {
    if (!x || !y) return set_error("null argument"), AHQ_ERR_INVALID;
    if (bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(x) & 15u) || (reinterpret_cast<uintptr_t>(y) & 15u))
        return set_error("x and y must be 16-byte aligned and a multiple of 16 bytes long"), AHQ_ERR_INVALID;
    if (workgroups < 1 || workgroups > 65536) return set_error("workgroups must be in 1..65536"), AHQ_ERR_INVALID;
    if (bytes == 0) return AHQ_OK;
    hipLaunchKernelGGL(diag_copy_kernel, dim3((unsigned)workgroups), dim3(kDiagThreads), 0, static_cast<hipStream_t>(stream),
                       static_cast<const u32x4*>(x), static_cast<u32x4*>(y), (int64_t)(bytes / 16));
    return check_launch("ahq_diag_copy");
}
