/* Memory-safety check of the CPU oracle (oracle/lutgemm_oracle.c) under -fsanitize=address,undefined,
 * built and run by tests/test_sanitizers.py: every entry point on exactly sized heap arrays of a
 * ragged shape, so that an index outside an array aborts the run.  Checker of the checker only. */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

void orc_f2h_array(const float *src, uint16_t *dst, long count);
void orc_pack_signs(const int8_t *signs, uint32_t *bW, int K, int q, int N);
void orc_dequantize_cpu(const uint32_t *bW, const uint16_t *alpha, int K, int N, int q, int group_size, int row_wise, uint16_t *fW);
void orc_matmul_cpu(const uint16_t *x, const uint16_t *fW, int M, int N, int K, float *out);
void orc_matvec_f64(const uint32_t *bW, const uint16_t *alpha, const uint16_t *zoff, const uint16_t *x, int M, int K, int N, int q,
                    int group_size, double *y);
void orc_dense_weight_f64(const uint32_t *bW, const uint16_t *alpha, const uint16_t *zoff, int K, int N, int q, int group_size, double *W);
void orc_lut256_f64(const uint16_t *x8, double *lut);
void orc_ref_kernel_fp16(const uint32_t *bW, const uint16_t *alpha, const uint16_t *zoff, const uint16_t *x, int K, int N, int q,
                         int group_size, int fused, uint16_t *y);

static unsigned long long st = 88172645463325252ull;
static unsigned rnd(void) { st ^= st << 13; st ^= st >> 7; st ^= st << 17; return (unsigned)(st >> 20); }

int main(void)
{
    const int shapes[][5] = {{64, 6, 1, 1, 0}, {128, 10, 3, 2, 1}, {256, 34, 4, 4, 1}, {512, 2, 8, 8, 0}};   /* K N q groups offset */
    for (unsigned c = 0; c < sizeof(shapes) / sizeof(shapes[0]); c++) {
        const int K = shapes[c][0], N = shapes[c][1], q = shapes[c][2], G = shapes[c][3], off = shapes[c][4], M = 2;
        int8_t *sg = malloc((size_t)K * q * N);
        uint32_t *bW = malloc((size_t)(K / 32) * q * N * 4);
        float *af = malloc((size_t)G * q * N * 4), *zf = malloc((size_t)G * N * 4), *xf = malloc((size_t)M * K * 4);
        uint16_t *a = malloc((size_t)G * q * N * 2), *z = malloc((size_t)G * N * 2), *x = malloc((size_t)M * K * 2);
        for (long i = 0; i < (long)K * q * N; i++) sg[i] = (rnd() & 1) ? 1 : -1;
        for (long i = 0; i < (long)G * q * N; i++) af[i] = 0.02f * (float)(rnd() % 1000) / 1000.f;
        for (long i = 0; i < (long)G * N; i++) zf[i] = 0.01f * ((float)(rnd() % 2001) - 1000.f) / 1000.f;
        for (long i = 0; i < (long)M * K; i++) xf[i] = ((float)(rnd() % 2001) - 1000.f) / 500.f;
        orc_pack_signs(sg, bW, K, q, N);
        orc_f2h_array(af, a, (long)G * q * N);
        orc_f2h_array(zf, z, (long)G * N);
        orc_f2h_array(xf, x, (long)M * K);
        uint16_t *fW = malloc((size_t)K * N * 2), *fWt = malloc((size_t)K * N * 2), *yr = malloc((size_t)N * 2);
        float *yf = malloc((size_t)M * N * 4);
        double *y = malloc((size_t)M * N * 8), *W = malloc((size_t)K * N * 8), lut[256];
        const int g = K / G;
        orc_dequantize_cpu(bW, a, K, N, q, g, 0, fW);
        orc_dequantize_cpu(bW, a, K, N, q, g, 1, fWt);
        orc_matmul_cpu(x, fW, M, N, K, yf);
        orc_matvec_f64(bW, a, off ? z : NULL, x, M, K, N, q, g, y);
        orc_dense_weight_f64(bW, a, off ? z : NULL, K, N, q, g, W);
        orc_lut256_f64(x, lut);
        if (N % 2 == 0 && g % 64 == 0) {
            orc_ref_kernel_fp16(bW, a, off ? z : NULL, x, K, N, q, g, 1, yr);
            orc_ref_kernel_fp16(bW, a, off ? z : NULL, x, K, N, q, g, 0, yr);
        }
        free(sg); free(bW); free(af); free(zf); free(xf); free(a); free(z); free(x); free(fW); free(fWt); free(yr); free(yf); free(y); free(W);
    }
    printf("oracle under sanitizers: ok\n");
    return 0;
}
