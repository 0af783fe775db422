// kernels.h -- the matmul entry points of the reference's C++ API (lutGEMM/include/kernels.h:26-33),
// header only, on top of the C ABI of this library.  Every batch size streams the packed weight (one
// and two rows through the table-lookup kernels, three and more through the batch kernel, 16 rows per
// pass; the reference dequantises and calls a dense GEMM for m > 1, lutGEMM/src/kernels.cu:73-79),
// the offset is applied for every m, no memset of the output is needed, and `algo` is accepted
// and ignored exactly as in the reference (mv_fp16.hpp:121).  Work is issued on the default stream
// and is asynchronous, as in the reference; failures throw std::runtime_error.
#ifndef KERNELS_H
#define KERNELS_H

#include "nQWeight_fp16.h"

namespace lutGEMM {

// weight first: input fp16 [kSize][n], output fp16 [mSize][n] (n vectors stored as columns)
inline void matmul(void *output, nQWeight_fp16 &nqW, void *input, int n, int algo = 0)
{
    (void)algo;
    detail::check(lutgemm_matvec_cols(nqW.handle(), input, output, n, nullptr), "lutGEMM::matmul");
}

// input first: input fp16 [m][kSize], output fp16 [m][mSize]
inline void matmul(void *output, void *input, nQWeight_fp16 &nqW, int m, int algo = 0)
{
    (void)algo;
    detail::check(lutgemm_matvec(nqW.handle(), input, output, m, nullptr), "lutGEMM::matmul");
}

// The OPTQ 3-bit comparison kernels of the reference (lutGEMM/src/kernels.cu:40-54) use a different
// weight format and are not part of this library.
inline void matmul_gptq(int, int, int, void *, void *, void *, void *, void *)
{
    throw std::runtime_error("lutGEMM::matmul_gptq: the OPTQ baseline kernel is not provided by this library");
}
inline void matmul_gptq_faster(int, int, int, void *, void *, void *, void *, void *)
{
    throw std::runtime_error("lutGEMM::matmul_gptq_faster: the OPTQ baseline kernel is not provided by this library");
}

}  // namespace lutGEMM
#endif  // KERNELS_H
