// A caller written against the reference's C++ API, compiled against this library's headers:
//   #include "lutGEMM";  nqW.parsing(bW, alpha, K, N, NUM_BITS, false, num_groups, q_bias);
//   lutGEMM::matmul((void*)C, (void*)A, nqW, M);
// It mirrors the reference's only test, tests/opt/fp16/int3_col_wise_matmul_fp16.cu: same input
// generators (makeRandomInput / makeRandomAlpha / makeRandomWeight, :185-215), same dense weight
// (dequantizeFrom_qW, :235-244), same timing protocol (1 warm-up + 16 timed calls, each followed by a
// device synchronise, min/max/avg in ms, :120-133) -- and, unlike it, checks the numbers: the result
// against a double-precision dense product, the mean error as checkOutputMeanError (:163-172) defines it.
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "lutGEMM"

namespace {

bool rand_bool() { return rand() > (RAND_MAX / 2); }
double rand_fp64(double max = 1.0)
{
    const double sign[] = {-1.0, 1.0};
    return sign[rand_bool()] * rand() / RAND_MAX * rand() / RAND_MAX * max;
}
float rand_fp32(float max = 1.0f) { return (float)(rand_fp64() * max); }

struct Timer {
    std::vector<double> ms;
    std::chrono::steady_clock::time_point t0;
    void start() { t0 = std::chrono::steady_clock::now(); }
    void end() { ms.push_back(std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count()); }
    double min() const { return *std::min_element(ms.begin(), ms.end()); }
    double max() const { return *std::max_element(ms.begin(), ms.end()); }
    double mean() const { double s = 0; for (double v : ms) s += v; return s / ms.size(); }
};

#define HIP_OK(call)                                                                   \
    do {                                                                               \
        hipError_t e_ = (call);                                                        \
        if (e_ != hipSuccess) {                                                        \
            fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));          \
            exit(2);                                                                   \
        }                                                                              \
    } while (0)

// One problem in the reference test's shape: M activations, N outputs, K inputs, NUM_BITS planes.
int run_case(int M, int N, int K, int NUM_BITS, int A_GROUP_SIZE, bool with_q_bias, bool check, int iter)
{
    const int num_groups = K / A_GROUP_SIZE;
    std::vector<uint32_t> bW((size_t)K / 32 * NUM_BITS * N);
    std::vector<float> alpha((size_t)num_groups * NUM_BITS * N), q_bias((size_t)num_groups * N);
    std::vector<float> input((size_t)M * K);
    for (auto &v : input) v = rand_fp32();
    for (int g = 0; g < num_groups; g++)
        for (int n = 0; n < N; n++) {
            q_bias[(size_t)g * N + n] = rand_fp32() / (1 << NUM_BITS);
            for (int b = 0; b < NUM_BITS; b++)
                alpha[((size_t)g * NUM_BITS + b) * N + n] = rand_fp32() / (1 << b);
        }
    for (int n = 0; n < N; n++)
        for (int b = 0; b < NUM_BITS; b++)
            for (int k = 0; k < K; k += 32) {
                uint32_t s = 0;
                for (int t = 0; t < 32; t++)
                    if (rand_bool()) s |= 1u << t;
                bW[((size_t)(k / 32) * NUM_BITS + b) * N + n] = s;
            }

    lutGEMM::nQWeight_fp16 nqW;
    nqW.parsing(bW.data(), alpha.data(), K, N, NUM_BITS, false, num_groups, with_q_bias ? q_bias.data() : nullptr);
    if (nqW.mSize != N || nqW.kSize != K || nqW.nb != NUM_BITS || nqW.num_groups != num_groups ||
        nqW.group_size != A_GROUP_SIZE || (nqW.q_bias != nullptr) != with_q_bias) {
        fprintf(stderr, "container fields wrong\n");
        return 1;
    }

    std::vector<_Float16> h_in((size_t)M * K), h_out((size_t)M * N);
    for (size_t i = 0; i < h_in.size(); i++) h_in[i] = (_Float16)input[i];
    _Float16 *d_input, *d_nq_output;
    HIP_OK(hipMalloc((void **)&d_input, h_in.size() * 2));
    HIP_OK(hipMalloc((void **)&d_nq_output, h_out.size() * 2));
    HIP_OK(hipMemcpy(d_input, h_in.data(), h_in.size() * 2, hipMemcpyHostToDevice));

    // lutgemm_latency
    Timer tm;
    lutGEMM::matmul((void *)d_nq_output, (void *)d_input, nqW, M);
    HIP_OK(hipDeviceSynchronize());
    for (int i = 0; i < iter; i++) {
        tm.start();
        lutGEMM::matmul((void *)d_nq_output, (void *)d_input, nqW, M);
        HIP_OK(hipDeviceSynchronize());
        tm.end();
    }
    printf("LUT-GEMM [INT%d, FP16, FP16] M=%d N=%d K=%d g=%d q_bias=%d\tlatency min : %.5fms, max : %.5fms, avg:%.5f\n",
           NUM_BITS, M, N, K, A_GROUP_SIZE, (int)with_q_bias, tm.min(), tm.max(), tm.mean());

    int bad = 0;
    if (check) {
        HIP_OK(hipMemcpy(h_out.data(), d_nq_output, h_out.size() * 2, hipMemcpyDeviceToHost));
        // dense weight from the fp16-rounded container contents, product in double
        double err_sum = 0, err_max = 0;
        std::vector<double> W((size_t)K);
        for (int n = 0; n < N; n++) {
            for (int k = 0; k < K; k++) {
                int g = k / A_GROUP_SIZE;
                double w = with_q_bias ? (double)(float)(_Float16)q_bias[(size_t)g * N + n] : 0.0;
                for (int b = 0; b < NUM_BITS; b++) {
                    double a = (double)(float)(_Float16)alpha[((size_t)g * NUM_BITS + b) * N + n];
                    bool plus = (bW[((size_t)(k / 32) * NUM_BITS + b) * N + n] >> (k % 32)) & 1u;
                    w += plus ? a : -a;
                }
                W[k] = w;
            }
            for (int m = 0; m < M; m++) {
                double y = 0;
                for (int k = 0; k < K; k++) y += (double)(float)h_in[(size_t)m * K + k] * W[k];
                double got = (double)(float)h_out[(size_t)m * N + n];
                double err = std::fabs(got - y);
                double ulp = std::ldexp(1.0, (int)std::floor(std::log2(std::max(std::fabs(y), std::ldexp(1.0, -14)))) - 10);
                err_sum += err;
                err_max = std::max(err_max, err);
                if (!(err <= 2 * ulp + 1e-3)) bad++;
            }
        }
        printf("  mean |error| = %.3e  max |error| = %.3e  out of tolerance: %d of %d\n", err_sum / ((double)M * N),
               err_max, bad, M * N);
    }
    HIP_OK(hipFree(d_input));
    HIP_OK(hipFree(d_nq_output));
    return bad;
}

}  // namespace

int main(int argc, char **argv)
{
    const bool full = argc > 1 && std::string(argv[1]) == "full";
    int bad = 0;
    // small checked cases: both overload families are exercised through the same container
    bad += run_case(1, 512, 1024, 3, 128, false, true, 4);
    bad += run_case(1, 1000, 2048, 4, 128, true, true, 4);
    bad += run_case(3, 384, 1024, 2, 64, true, true, 4);
    {
        // weight-first overload: input [K][n], output [N][n]
        const int K = 1024, N = 256, n = 2, q = 2, g = 128;
        std::vector<uint32_t> bW((size_t)K / 32 * q * N);
        for (auto &v : bW) v = (uint32_t)rand() * 2654435761u;
        std::vector<float> alpha((size_t)(K / g) * q * N, 0.25f);
        lutGEMM::nQWeight_fp16 nqW(bW.data(), alpha.data(), K, N, q, false, K / g, nullptr);
        std::vector<_Float16> x((size_t)K * n), y_cols((size_t)N * n), y_rows((size_t)n * N), xr((size_t)n * K);
        for (int k = 0; k < K; k++)
            for (int c = 0; c < n; c++) xr[(size_t)c * K + k] = x[(size_t)k * n + c] = (_Float16)rand_fp32();
        _Float16 *dx, *dxr, *dy, *dyr;
        HIP_OK(hipMalloc((void **)&dx, x.size() * 2));
        HIP_OK(hipMalloc((void **)&dxr, xr.size() * 2));
        HIP_OK(hipMalloc((void **)&dy, y_cols.size() * 2));
        HIP_OK(hipMalloc((void **)&dyr, y_rows.size() * 2));
        HIP_OK(hipMemcpy(dx, x.data(), x.size() * 2, hipMemcpyHostToDevice));
        HIP_OK(hipMemcpy(dxr, xr.data(), xr.size() * 2, hipMemcpyHostToDevice));
        lutGEMM::matmul((void *)dy, nqW, (void *)dx, n);
        lutGEMM::matmul((void *)dyr, (void *)dxr, nqW, n);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipMemcpy(y_cols.data(), dy, y_cols.size() * 2, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(y_rows.data(), dyr, y_rows.size() * 2, hipMemcpyDeviceToHost));
        int diff = 0;
        for (int j = 0; j < N; j++)
            for (int c = 0; c < n; c++) diff += (float)y_cols[(size_t)j * n + c] != (float)y_rows[(size_t)c * N + j];
        printf("weight-first overload vs input-first overload: %d differing outputs\n", diff);
        bad += diff;
        // dense weight through the container API
        _Float16 *dW = (_Float16 *)nqW.getDequantiedWeight(true);
        std::vector<_Float16> hW((size_t)K * N), hW2((size_t)K * N);
        HIP_OK(hipMemcpy(hW.data(), dW, hW.size() * 2, hipMemcpyDeviceToHost));
        lutGEMM::dequantize_cpu(nqW, hW2.data());
        int wbad = 0;
        for (int k = 0; k < K; k++)
            for (int j = 0; j < N; j++) {
                float w = 0;
                for (int b = 0; b < q; b++) w += ((bW[((size_t)(k / 32) * q + b) * N + j] >> (k % 32)) & 1u) ? 0.25f : -0.25f;
                wbad += (float)hW[(size_t)k * N + j] != w || (float)hW2[(size_t)k * N + j] != w;
            }
        printf("getDequantiedWeight / dequantize_cpu: %d wrong weights\n", wbad);
        bad += wbad;
        // additions to the container: packed file round trip and measured plan keep the results
        {
            const char *path = "/tmp/lutgemm_dropin_test.lutw";
            nqW.save(path);
            lutGEMM::nQWeight_fp16 loaded;
            loaded.load(path);
            loaded.autotune();
            std::remove(path);
            int ldiff = loaded.kSize != K || loaded.mSize != N || loaded.nb != q || loaded.num_groups != K / g;
            lutGEMM::matmul((void *)dy, (void *)dxr, loaded, n);
            HIP_OK(hipDeviceSynchronize());
            std::vector<_Float16> y2((size_t)n * N);
            HIP_OK(hipMemcpy(y2.data(), dy, y2.size() * 2, hipMemcpyDeviceToHost));
            // another plan changes the summation order only: unit scales and these activations leave
            // the results within one fp16 step
            for (size_t i = 0; i < y2.size(); i++)
                ldiff += std::fabs((float)y2[i] - (float)y_rows[i]) > 4e-3f * std::fmax(1.f, std::fabs((float)y_rows[i]));
            printf("save / load / autotune: %d differing outputs\n", ldiff);
            bad += ldiff;
        }
        HIP_OK(hipFree(dx)); HIP_OK(hipFree(dxr)); HIP_OK(hipFree(dy)); HIP_OK(hipFree(dyr));
    }
    {
        lutGEMM::nQWeight_fp16 empty;  // default-constructed objects are safe to destroy
    }
    if (full) {
        // the reference test's own shape and protocol: H = 7168, M = 1, N = 4H, K = H, g = 128, with q_bias
        const int H = 7168;
        for (int q : {8, 4, 3}) bad += run_case(1, 4 * H, H, q, 128, true, q == 3, 16);
    }
    printf(bad ? "DROPIN FAILED (%d)\n" : "DROPIN OK\n", bad);
    return bad ? 1 : 0;
}
