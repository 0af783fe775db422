// The batch kernel as a work list, like lut_matvec_multi_kernel: up to kMaxFused independent
// batches (same planes, offset and scale layout, same wavefronts per workgroup; each with its own
// weight, rows and k-split) share one grid, entry i owning the workgroups first_block[i] ..
// first_block[i + 1] - 1 (workgroup body: batch_body.h).  A kernel of its own beside the one for a
// single batch: the larger kernel arguments cost a launch one to two microseconds.
#include "batch_body.h"

namespace lutgemm_kernels {
namespace {

template <int Q, bool OFF, int GSUB, int W, bool TWO>
__global__ __launch_bounds__(W * 64) __attribute__((aligned(16384))) void lut_batch_multi_kernel(MultiMatvecArgs m)
{
    int i = 0;
    while (i + 1 < m.count && (int)blockIdx.x >= m.first_block[i + 1]) i++;   // scalar: at most 31 steps
    batch_workgroup<Q, OFF, GSUB, W, TWO>(m.entry[i], blockIdx.x - (unsigned)m.first_block[i]);
}

template <int Q, bool OFF, int GSUB, int W, bool TWO>
struct LaunchMany {
    static hipError_t run(const MultiMatvecArgs &m, int workgroups, int waves, hipStream_t stream)
    {
        static std::atomic<unsigned long long> allowed{0};
        const hipError_t e = allow_batch_lds<Q, OFF, GSUB>(&lut_batch_multi_kernel<Q, OFF, GSUB, W, TWO>, allowed);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((lut_batch_multi_kernel<Q, OFF, GSUB, W, TWO>), dim3(workgroups), dim3(waves * kLanes),
                           batch_lds_bytes(waves, GSUB, Q + (OFF ? 1 : 0)), stream, m);
        return hipGetLastError();
    }
};

}  // namespace

hipError_t launch_batch_multi(int q, int has_offset, int gsub, const MultiMatvecArgs &m, int workgroups, int waves,
                              hipStream_t stream)
{
    if (m.count < 1 || m.count > kMaxFused) return hipErrorInvalidValue;
    bool two = false;   // some entry has more rows than the workgroups have wavefronts
    for (int i = 0; i < m.count; i++) {
        if (m.entry[i].rows < 1 || m.entry[i].rows > kBatchRows) return hipErrorInvalidValue;
        two = two || m.entry[i].rows > waves;
    }
    return dispatch_batch<LaunchMany>(q, has_offset, gsub, two, m, workgroups, waves, stream);
}

}  // namespace lutgemm_kernels
