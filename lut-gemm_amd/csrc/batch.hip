// The batch kernel for one batch: 3..16 activation rows against a packed BCQ weight in one pass
// over its tiles (workgroup body and description: batch_body.h).
#include "batch_body.h"

namespace lutgemm_kernels {
namespace {

template <int Q, bool OFF, int GSUB, int W, bool TWO>
__global__ __launch_bounds__(W * 64) __attribute__((aligned(16384))) void lut_batch_kernel(MatvecArgs a)
{
    batch_workgroup<Q, OFF, GSUB, W, TWO>(a, blockIdx.x);
}

template <int Q, bool OFF, int GSUB, int W, bool TWO>
struct LaunchOne {
    static hipError_t run(const MatvecArgs &a, int workgroups, int waves, hipStream_t stream)
    {
        static std::atomic<unsigned long long> allowed{0};
        const hipError_t e = allow_batch_lds<Q, OFF, GSUB>(&lut_batch_kernel<Q, OFF, GSUB, W, TWO>, allowed);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL((lut_batch_kernel<Q, OFF, GSUB, W, TWO>), dim3(workgroups), dim3(waves * kLanes),
                           batch_lds_bytes(waves, GSUB, Q + (OFF ? 1 : 0)), stream, a);
        return hipGetLastError();
    }
};

}  // namespace

hipError_t launch_batch(int q, int has_offset, int gsub, const MatvecArgs &a, int workgroups, int waves, hipStream_t stream)
{
    if (a.rows < 1 || a.rows > kBatchRows) return hipErrorInvalidValue;
    return dispatch_batch<LaunchOne>(q, has_offset, gsub, a.rows > waves, a, workgroups, waves, stream);
}

}  // namespace lutgemm_kernels
