// Dense fp16 matrix-vector product, the comparator of the LUT matvec: y[n] = sum_k W[n][k] x[k]
// for a dense weight stored as W^T [n][k] (what lutgemm_dequantize writes with transposed = 1).
// Plain bandwidth-bound streaming: one wavefront per output row at a time, 16-byte non-temporal
// loads of the row with several in flight per lane, the activations re-read through the cache,
// products accumulated in fp32 (v_dot2_f32_f16), cross-lane sum, one fp16 store.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "kernels.h"

namespace lutgemm_kernels {

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc)
{
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, w), __builtin_bit_cast(half2_t, x), acc, false);
}

// (vector elements are copied to scalars first: a bit cast applied to an element expression of
// an ext_vector picks element 0 whichever element is named)
__device__ __forceinline__ float dot8(const u32x4 &w, const u32x4 &x, float acc)
{
    const uint32_t w0 = w.x, w1 = w.y, w2 = w.z, w3 = w.w;
    const uint32_t x0 = x.x, x1 = x.y, x2 = x.z, x3 = x.w;
    return dot2(w3, x3, dot2(w2, x2, dot2(w1, x1, dot2(w0, x0, acc))));
}

constexpr int kInFlight = 8;  // 16-byte loads per lane before the first use

__global__ __launch_bounds__(256) void dense_gemv_kernel(const u32x4 *wt, const u32x4 *x, __half *y, int k8, int n)
{
    const int lane = threadIdx.x & 63;
    const int wave = (int)((blockIdx.x * blockDim.x + threadIdx.x) >> 6);
    const int nwaves = (int)((gridDim.x * blockDim.x) >> 6);
    for (int row = wave; row < n; row += nwaves) {
        const u32x4 *wr = wt + (size_t)row * k8;
        float acc = 0.f;
        int c = lane;
        for (; c + (kInFlight - 1) * 64 < k8; c += kInFlight * 64) {
            u32x4 w[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; u++) w[u] = __builtin_nontemporal_load(wr + c + u * 64);
#pragma unroll
            for (int u = 0; u < kInFlight; u++) acc = dot8(w[u], x[c + u * 64], acc);
        }
        for (; c < k8; c += 64) acc = dot8(__builtin_nontemporal_load(wr + c), x[c], acc);
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1) acc += __shfl_xor(acc, s, 64);
        if (lane == 0) y[row] = __float2half_rn(acc);
    }
}

}  // namespace

hipError_t launch_dense_gemv(const void *wt, const void *x, void *y, int k, int n, int compute_units, hipStream_t stream)
{
    // sixteen wavefronts per compute unit, each walking rows wave, wave + total, ...
    const int blocks = compute_units * 4;
    hipLaunchKernelGGL(dense_gemv_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<const u32x4 *>(wt),
                       static_cast<const u32x4 *>(x), static_cast<__half *>(y), k / 8, n);
    return hipGetLastError();
}

}  // namespace lutgemm_kernels
