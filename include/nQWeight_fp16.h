// nQWeight_fp16.h -- the packed BCQ weight container of the reference's C++ API, on top of the
// C ABI of this library (lutgemm_c.h).  Header only.
//
// Same class name, namespace, public data members (in the same order) and member functions as
// lutGEMM/include/nQWeight_fp16.h:27-52 of the reference, so that a caller written against it
// recompiles unchanged.  What differs, on purpose:
//   * bWeight / alpha / q_bias point at DEVICE memory whose tiling is private to the library
//     (sign tiles, scale tiles; q_bias is non-null iff the weight has an offset and points into
//     the scale tiles).  Indexing them directly is not part of the contract.
//   * group_size is always kSize / num_groups (the reference computes it from an uninitialised
//     field, lutGEMM/src/nQWeight_fp16.cu:63); the destructor frees every allocation exactly once
//     (the reference frees alpha twice and leaks bWeight, :101-105); a default-constructed object
//     is empty and safe to destroy.
//   * dequantisation takes the group index per weight and includes the offset (the reference's
//     kernels drop q_bias, lutGEMM/src/cuda/kernels/dequant_fp16.hpp:54-80).
//   * failures throw std::runtime_error (the reference checks no status at all).
#ifndef N_Q_WEIGHT_FP16_H
#define N_Q_WEIGHT_FP16_H

#include <hip/hip_runtime_api.h>

#include <stdexcept>
#include <string>

#include "lutgemm_c.h"

namespace lutGEMM {

class nQWeight_fp16;

void dequantize_gpu(nQWeight_fp16 &nqw, void *d_fW, int algo = 0);
void dequantize_cpu(nQWeight_fp16 &nqw, void *fW);

namespace detail {
inline void check(int status, const char *what)
{
    if (status != LUTGEMM_OK)
        throw std::runtime_error(std::string(what) + ": " + lutgemm_status_string(status) + ": " +
                                 lutgemm_last_error());
}
inline void check_hip(hipError_t e, const char *what)
{
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}
}  // namespace detail

class nQWeight_fp16 {
public:
    unsigned int *bWeight = nullptr;  // device: sign tiles of Weight[kSize/32][nb][mSize]
    void *alpha = nullptr;            // device: scale tiles of alpha[num_alpha_groups][nb][mSize]
    void *q_bias = nullptr;           // device, non-null iff q_bias[num_alpha_groups][mSize] was given
    int num_groups = 0;
    int group_size = 0;
    int mSize = 0;
    int kSize = 0;
    int nb = 0;
    bool is_row_wise_quantize = false;

    nQWeight_fp16() {}

    /* host arrays: uint32 bW[kSize/32][nb][mSize], float A[num_alpha_groups][nb][mSize],
       float q_bias[num_alpha_groups][mSize] or nullptr */
    nQWeight_fp16(unsigned int *bW, float *A, int row, int col, int num_bits, bool is_row_wise_quantize,
                  int num_alpha_groups = 1, float *q_bias = nullptr)
    {
        parsing(bW, A, row, col, num_bits, is_row_wise_quantize, num_alpha_groups, q_bias);
    }

    nQWeight_fp16(const nQWeight_fp16 &) = delete;
    nQWeight_fp16 &operator=(const nQWeight_fp16 &) = delete;

    // (row, col) = (kSize, mSize) when is_row_wise_quantize is false, (mSize, kSize) when true,
    // as in lutGEMM/src/nQWeight_fp16.cu:69-76.  Re-parsing releases the previous weight.
    void parsing(unsigned int *bW, float *A, int row, int col, int num_bits, bool is_row_wise_quantize,
                 int num_alpha_groups = 1, float *q_bias = nullptr)
    {
        release();
        this->is_row_wise_quantize = is_row_wise_quantize;
        nb = num_bits;
        num_groups = num_alpha_groups;
        if (is_row_wise_quantize) {
            mSize = row;
            kSize = col;
        } else {
            mSize = col;
            kSize = row;
        }
        group_size = num_alpha_groups > 0 ? kSize / num_alpha_groups : 0;
        detail::check(lutgemm_weight_create(bW, A, q_bias, kSize, mSize, num_bits, num_alpha_groups, &handle_),
                      "nQWeight_fp16::parsing");
        void *s = nullptr, *a = nullptr, *z = nullptr;
        detail::check(lutgemm_weight_device_ptrs(handle_, &s, &a, &z), "nQWeight_fp16::parsing");
        bWeight = static_cast<unsigned int *>(s);
        alpha = a;
        this->q_bias = z;
    }

    ~nQWeight_fp16() { release(); }

    // Dense fp16 weight in a device buffer owned by this object (the reference hands out a
    // process-wide scratch, lutGEMM/src/cuda/tmpWeight.hpp:28-35): [kSize][mSize], or
    // [mSize][kSize] for a row-wise weight.  Valid until the next call or until the object dies.
    // Both values of onGPU run the device kernel; the result is complete when the call returns.
    void *getDequantiedWeight(bool onGPU = true)
    {
        (void)onGPU;
        if (!dense_)
            detail::check_hip(hipMalloc(&dense_, sizeof(unsigned short) * (size_t)mSize * (size_t)kSize),
                              "getDequantiedWeight");
        dequantize_gpu(*this, dense_);
        return dense_;
    }

    lutgemm_weight *handle() const { return handle_; }

    // ---- additions without counterpart in the reference ----
    // Write the packed weight to a file / replace this object's weight by a packed file's
    // (no packing work on load).  A loaded weight is column-wise (is_row_wise_quantize = false).
    void save(const char *path) const { detail::check(lutgemm_weight_save(handle_, path), "nQWeight_fp16::save"); }
    void load(const char *path)
    {
        release();
        detail::check(lutgemm_weight_load(path, &handle_), "nQWeight_fp16::load");
        lutgemm_weight_info_t info;
        detail::check(lutgemm_weight_info(handle_, &info), "nQWeight_fp16::load");
        is_row_wise_quantize = false;
        kSize = info.k;
        mSize = info.n;
        nb = info.q;
        num_groups = info.num_groups;
        group_size = info.group_size;
        void *s = nullptr, *a = nullptr, *z = nullptr;
        detail::check(lutgemm_weight_device_ptrs(handle_, &s, &a, &z), "nQWeight_fp16::load");
        bWeight = static_cast<unsigned int *>(s);
        alpha = a;
        q_bias = z;
    }
    // Measure launch plans on the device and keep the fastest (the default plan comes from a model).
    void autotune() { detail::check(lutgemm_weight_autotune(handle_, nullptr), "nQWeight_fp16::autotune"); }

private:
    void release()
    {
        if (handle_) lutgemm_weight_destroy(handle_);
        if (dense_) (void)hipFree(dense_);
        handle_ = nullptr;
        dense_ = nullptr;
        bWeight = nullptr;
        alpha = nullptr;
        q_bias = nullptr;
    }
    lutgemm_weight *handle_ = nullptr;
    void *dense_ = nullptr;
};

// d_fW: device buffer of mSize*kSize halves; synchronises the device like the reference does
// (lutGEMM/src/nQWeight_fp16.cu:29-35).
inline void dequantize_gpu(nQWeight_fp16 &nqw, void *d_fW, int algo)
{
    (void)algo;
    detail::check(lutgemm_dequantize(nqw.handle(), d_fW, nqw.is_row_wise_quantize ? 1 : 0, nullptr),
                  "dequantize_gpu");
    detail::check_hip(hipDeviceSynchronize(), "dequantize_gpu");
}

// fW: HOST buffer of mSize*kSize halves.  Same values as dequantize_gpu (computed on the device and
// copied back); stands for the host loop of lutGEMM/src/nQWeight_fp16.cu:38-59.
inline void dequantize_cpu(nQWeight_fp16 &nqw, void *fW)
{
    void *d = nullptr;
    const size_t bytes = sizeof(unsigned short) * (size_t)nqw.mSize * (size_t)nqw.kSize;
    detail::check_hip(hipMalloc(&d, bytes), "dequantize_cpu");
    try {
        dequantize_gpu(nqw, d);
        detail::check_hip(hipMemcpy(fW, d, bytes, hipMemcpyDeviceToHost), "dequantize_cpu");
    } catch (...) {
        (void)hipFree(d);
        throw;
    }
    (void)hipFree(d);
}

}  // namespace lutGEMM
#endif  // N_Q_WEIGHT_FP16_H
