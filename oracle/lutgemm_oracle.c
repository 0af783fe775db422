/*
 * CPU oracle for the BCQ LUT matvec path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithms of the reference implementation
 * (paths below are relative to the reference tree).  It is the checker that the GPU
 * library is compared against; nothing in the shipped library may link, load or call
 * it.  Only tests, the smoke check and the benchmark's cpu_baseline leg use it.
 *
 * Reference being restated (the CUDA sources cannot be compiled without nvcc and
 * cuda_fp16.h, so no binary of the reference exists next to this file):
 *   container layout      lutGEMM/include/nQWeight_fp16.h:27-52
 *   ingest (float->half)  lutGEMM/src/nQWeight_fp16.cu:60-91
 *   dequantize_cpu        lutGEMM/src/nQWeight_fp16.cu:38-59
 *   LUT kernels           lutGEMM/src/cuda/kernels/mv_fp16.hpp:25-97
 *                         lutGEMM/src/cuda/kernels/mv_fp16_bias.hpp:24-118
 *   dispatch rule         lutGEMM/src/kernels.cu:56-71
 *   packing / dense W /   tests/opt/fp16/int3_col_wise_matmul_fp16.cu:163-244
 *   dense truth / error
 *   RTN -> BCQ            examples/rtn_parameter.py:77-96
 *
 * Parity status of every exported function is "pinned": each one is checked in
 * tests/test_oracle.py against something it does not itself compute (numpy float16,
 * numpy unpackbits + dense matmul, closed forms, brute force on tiny inputs); the order of
 * the fp16 operations in orc_ref_kernel_fp16 is pinned in tests/test_oracle_ref_kernel.py by
 * known answers worked out by hand from the reference source, where binary16 rounding makes
 * every other order give a different number, and by a thread-by-thread transcription of the
 * CUDA kernels in numpy.float16 that must agree bit for bit.
 *
 * Layout conventions (reference names in brackets):
 *   K [kSize]  reduction length, multiple of 32
 *   N [mSize]  number of outputs
 *   q [nb]     number of sign bit-planes
 *   G [num_groups], group length gs = K / G along k
 *   bW    uint32 [K/32][q][N]   bit t of bW[w][b][n] <=> sign of weight k = 32 w + t, 1 = +1
 *   alpha fp16   [G][q][N]
 *   zoff  fp16   [G][N]  or NULL   [q_bias]
 *   W[k][n] = sum_b alpha[k/gs][b][n] * s(b,k,n) + zoff[k/gs][n]
 *   y[n]    = sum_k x[k] * W[k][n]
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

/* ------------------------------------------------------------------------------------
 * IEEE binary16 <-> binary32/64, round to nearest even.  The double-source routine is the
 * definition; the float-source bit routine is the fast path used in the timed baseline
 * and is pinned against the definition and against numpy.float16 in the tests.
 * ---------------------------------------------------------------------------------- */
float orc_h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {
            /* subnormal: value = man * 2^-24 */
            float f = (float)man * 5.9604644775390625e-08f;
            memcpy(&bits, &f, 4);
            bits |= sign;
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

uint16_t orc_d2h(double d)
{
    uint16_t sign = signbit(d) ? 0x8000u : 0u;
    if (isnan(d)) return (uint16_t)(sign | 0x7e00u);
    double a = fabs(d);
    if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u); /* rounds to infinity */
    if (a == 0.0) return sign;
    int e;
    (void)frexp(a, &e); /* a = f * 2^e, f in [0.5,1) -> floor(log2 a) = e-1 */
    int le = e - 1;
    if (le < -14) le = -14;               /* subnormal range shares the quantum 2^-24 */
    double quantum = ldexp(1.0, le - 10); /* spacing of halves in this binade */
    double r = nearbyint(a / quantum);    /* exact scaling; RNE in the default mode */
    /* r in [0, 2048]; r == 2048 means carry into the next binade */
    uint32_t ri = (uint32_t)r;
    uint32_t bits;
    if (le == -14 && ri < 1024u) {
        bits = ri; /* subnormal or zero */
    } else {
        if (ri == 2048u) {
            ri = 1024u;
            le += 1;
        }
        bits = ((uint32_t)(le + 15) << 10) + (ri - 1024u);
    }
    return (uint16_t)(sign | bits);
}

uint16_t orc_f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); /* >= 65520 */
    if (x < 0x38800000u) {                                   /* < 2^-14: subnormal */
        if (x < 0x33000000u) return sign;                    /* < 2^-25 */
        uint32_t e = x >> 23;                                /* 102..112 */
        uint32_t m = (x & 0x7fffffu) | 0x800000u;            /* 24-bit significand */
        uint32_t shift = 126u - e;                           /* 14..24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (x >> 23) - 112u;
    uint32_t m = x & 0x7fffffu;
    uint32_t h = (e << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

void orc_f2h_array(const float *src, uint16_t *dst, long count)
{
    for (long i = 0; i < count; i++) dst[i] = orc_f2h(src[i]);
}

void orc_d2h_array(const double *src, uint16_t *dst, long count)
{
    for (long i = 0; i < count; i++) dst[i] = orc_d2h(src[i]);
}

void orc_h2f_array(const uint16_t *src, float *dst, long count)
{
    for (long i = 0; i < count; i++) dst[i] = orc_h2f(src[i]);
}

/* ------------------------------------------------------------------------------------
 * Bit packing exactly as the reference's only packer does it
 * (tests/opt/fp16/int3_col_wise_matmul_fp16.cu:200-215): signs[K][q][N] in {+1,-1},
 * bit t of bW[k/32][b][n] is set iff signs[k+t][b][n] == +1.
 * ---------------------------------------------------------------------------------- */
void orc_pack_signs(const int8_t *signs, uint32_t *bW, int K, int q, int N)
{
    for (int n = 0; n < N; n++)
        for (int b = 0; b < q; b++)
            for (int k = 0; k < K; k += 32) {
                uint32_t s = 0;
                for (int t = 0; t < 32; t++)
                    if (signs[((long)(k + t) * q + b) * N + n] > 0) s |= 1u << t;
                bW[((long)(k / 32) * q + b) * N + n] = s;
            }
}

/* ------------------------------------------------------------------------------------
 * dequantize_cpu, lutGEMM/src/nQWeight_fp16.cu:38-59: k outer, output inner, plane
 * innermost; float accumulate of +/-alpha; one float->half per weight; the offset is
 * NOT applied (the reference ignores q_bias here).  row_wise selects fW[n*K+k] instead
 * of fW[k*N+n].  group_size is passed explicitly because the reference derives it from
 * an uninitialised field; K/num_groups is what its kernels use (mv_fp16.hpp:104).
 * ---------------------------------------------------------------------------------- */
void orc_dequantize_cpu(const uint32_t *bW, const uint16_t *alpha, int K, int N, int q,
                        int group_size, int row_wise, uint16_t *fW)
{
    for (int k = 0; k < K; k++) {
        for (int n = 0; n < N; n++) {
            float tmp = 0.0f;
            for (int b = 0; b < q; b++) {
                float a = orc_h2f(alpha[((long)(k / group_size) * q + b) * N + n]);
                if ((bW[((long)(k / 32) * q + b) * N + n] >> (k % 32)) & 1u)
                    tmp += a;
                else
                    tmp -= a;
            }
            if (row_wise)
                fW[(long)n * K + k] = orc_f2h(tmp);
            else
                fW[(long)k * N + n] = orc_f2h(tmp);
        }
    }
}

/* Same loop nest with OpenMP over k; reports the threads it used. */
int orc_dequantize_cpu_omp(const uint32_t *bW, const uint16_t *alpha, int K, int N, int q,
                           int group_size, uint16_t *fW)
{
    int used = 1;
#if defined(_OPENMP)
#pragma omp parallel
    {
#pragma omp single
        used = omp_get_num_threads();
#pragma omp for schedule(static)
        for (int k = 0; k < K; k++) {
            for (int n = 0; n < N; n++) {
                float tmp = 0.0f;
                for (int b = 0; b < q; b++) {
                    float a = orc_h2f(alpha[((long)(k / group_size) * q + b) * N + n]);
                    if ((bW[((long)(k / 32) * q + b) * N + n] >> (k % 32)) & 1u)
                        tmp += a;
                    else
                        tmp -= a;
                }
                fW[(long)k * N + n] = orc_f2h(tmp);
            }
        }
    }
#else
    orc_dequantize_cpu(bW, alpha, K, N, q, group_size, 0, fW);
#endif
    return used;
}

/* Dense weight including the offset, as the test's dequantizeFrom_qW defines it
 * (tests/opt/fp16/int3_col_wise_matmul_fp16.cu:235-244), in double: W[k][n]. */
void orc_dense_weight_f64(const uint32_t *bW, const uint16_t *alpha, const uint16_t *zoff,
                          int K, int N, int q, int group_size, double *W)
{
    for (int k = 0; k < K; k++) {
        int g = k / group_size;
        for (int n = 0; n < N; n++) {
            double w = zoff ? (double)orc_h2f(zoff[(long)g * N + n]) : 0.0;
            for (int b = 0; b < q; b++) {
                double a = (double)orc_h2f(alpha[((long)g * q + b) * N + n]);
                if ((bW[((long)(k / 32) * q + b) * N + n] >> (k % 32)) & 1u)
                    w += a;
                else
                    w -= a;
            }
            W[(long)k * N + n] = w;
        }
    }
}

/* matmul_cpu, tests/opt/fp16/int3_col_wise_matmul_fp16.cu:174-183: float triple loop,
 * (m, n) outer and k inner, float accumulator.  W is the dense fp16 matrix [K][N]. */
void orc_matmul_cpu(const uint16_t *x, const uint16_t *fW, int M, int N, int K, float *out)
{
    for (int m = 0; m < M; m++)
        for (int n = 0; n < N; n++) {
            float acc = 0.0f;
            for (int k = 0; k < K; k++)
                acc += orc_h2f(x[(long)m * K + k]) * orc_h2f(fW[(long)k * N + n]);
            out[(long)m * N + n] = acc;
        }
}

/* Same result definition with OpenMP over n; reports the threads it used. */
int orc_matmul_cpu_omp(const uint16_t *x, const uint16_t *fW, int M, int N, int K, float *out)
{
    int used = 1;
#if defined(_OPENMP)
#pragma omp parallel
    {
#pragma omp single
        used = omp_get_num_threads();
        for (int m = 0; m < M; m++) {
#pragma omp for schedule(static)
            for (int n = 0; n < N; n++) {
                float acc = 0.0f;
                for (int k = 0; k < K; k++)
                    acc += orc_h2f(x[(long)m * K + k]) * orc_h2f(fW[(long)k * N + n]);
                out[(long)m * N + n] = acc;
            }
        }
    }
#else
    orc_matmul_cpu(x, fW, M, N, K, out);
#endif
    return used;
}

/* ------------------------------------------------------------------------------------
 * The mathematical truth of the path: double accumulation over the fp16-rounded inputs,
 * y[m][n] = sum_k x[m][k] * (sum_b alpha*s + zoff).  Evaluated group by group as
 * sum_g ( sum_b alpha[g][b][n] * T[g][b][n] + zoff[g][n] * X[g] ) with
 * T = sum_{k in g} s*x and X = sum_{k in g} x, all in double (exact reordering of a
 * finite double sum up to rounding ~1e-16 relative).
 * ---------------------------------------------------------------------------------- */
void orc_matvec_f64(const uint32_t *bW, const uint16_t *alpha, const uint16_t *zoff,
                    const uint16_t *x, int M, int K, int N, int q, int group_size, double *y)
{
    int G = K / group_size;
    double *xf = (double *)malloc(sizeof(double) * (size_t)K);
    double *T = (double *)malloc(sizeof(double) * (size_t)N);
    for (int m = 0; m < M; m++) {
        for (int k = 0; k < K; k++) xf[k] = (double)orc_h2f(x[(long)m * K + k]);
        double *ym = y + (long)m * N;
        for (int n = 0; n < N; n++) ym[n] = 0.0;
        for (int g = 0; g < G; g++) {
            int k0 = g * group_size;
            double X = 0.0;
            for (int k = k0; k < k0 + group_size; k++) X += xf[k];
            for (int b = 0; b < q; b++) {
                for (int n = 0; n < N; n++) T[n] = 0.0;
                for (int k = k0; k < k0 + group_size; k++) {
                    const uint32_t *row = bW + ((long)(k / 32) * q + b) * N;
                    int sh = k % 32;
                    double xp = xf[k];
                    for (int n = 0; n < N; n++) T[n] += ((row[n] >> sh) & 1u) ? xp : -xp;
                }
                const uint16_t *ar = alpha + ((long)g * q + b) * N;
                for (int n = 0; n < N; n++) ym[n] += (double)orc_h2f(ar[n]) * T[n];
            }
            if (zoff) {
                const uint16_t *zr = zoff + (long)g * N;
                for (int n = 0; n < N; n++) ym[n] += (double)orc_h2f(zr[n]) * X;
            }
        }
    }
    free(xf);
    free(T);
}

/* ------------------------------------------------------------------------------------
 * The 256-entry partial-sum table of one 8-activation chunk (mv_fp16.hpp:36-60 in exact
 * arithmetic): lut[idx] = sum_j (2*bit_j(idx) - 1) * x[j].
 * ---------------------------------------------------------------------------------- */
void orc_lut256_f64(const uint16_t *x8, double *lut)
{
    for (int idx = 0; idx < 256; idx++) {
        double s = 0.0;
        for (int j = 0; j < 8; j++) {
            double v = (double)orc_h2f(x8[j]);
            s += ((idx >> j) & 1) ? v : -v;
        }
        lut[idx] = s;
    }
}

/* ------------------------------------------------------------------------------------
 * Op-for-op fp16 emulation of the reference GPU kernels, so that "the reference kernel's
 * error" can be reported without CUDA.  Every fp16 operation is computed exactly in
 * double and rounded once to binary16 (sums and products of two halves are exact in
 * double, so this is the correctly rounded result).
 *   k_tile = 64 without offset  (mv_fp16.hpp:121-128 picks _nqmv<64>)
 *   k_tile = 32 with offset     (mv_fp16_bias.hpp:143-150 picks _nqmv_bias<32>)
 * The per-k-tile atomicAdd(half2) into the zeroed output (mv_fp16.hpp:95, kernels.cu:66)
 * is applied in ascending k-tile order; the hardware order is not deterministic.
 * fused != 0 models `o += a * t` contracted to one fp16 FMA, fused == 0 a rounded
 * multiply followed by a rounded add; the compiler may pick either.
 * The group index is taken per k-tile block exactly as the kernels do
 * (mv_fp16.hpp:70), which is only meaningful when group_size is a multiple of k_tile.
 * ---------------------------------------------------------------------------------- */
static inline uint16_t h_add(uint16_t a, uint16_t b)
{
    return orc_d2h((double)orc_h2f(a) + (double)orc_h2f(b));
}
static inline uint16_t h_mul(uint16_t a, uint16_t b)
{
    return orc_d2h((double)orc_h2f(a) * (double)orc_h2f(b));
}
static inline uint16_t h_fma(uint16_t a, uint16_t b, uint16_t c)
{
    /* a*b is exact in double (22 significant bits); the sum may round in double before
       the final rounding to half only when the exponents differ by more than 30, where
       the small term cannot move a half-precision result across a rounding boundary
       except at exact ties, which the long double sum below resolves. */
    long double p = (long double)orc_h2f(a) * (long double)orc_h2f(b);
    return orc_d2h((double)(p + (long double)orc_h2f(c)));
}

static void ref_build_lut(const uint16_t *x, int k_tile, uint16_t *lut /* [k_tile/8][256] */)
{
    const int tables = k_tile / 8;
    const int lut_x_size = 256 / tables; /* 256 threads per block */
    int s0 = 0;
    while ((1 << s0) < lut_x_size) s0++;
    const uint16_t two = 0x4000, one = 0x3c00, mone = 0xbc00;
    for (int ty = 0; ty < tables; ty++) {
        const uint16_t *inp = x + ty * 8;
        uint16_t *t = lut + ty * 256;
        for (int lx = 0; lx < lut_x_size; lx++) {
            /* unary plus on the first product, then left-to-right fp16 adds */
            uint16_t base = h_mul(((lx >> 0) & 1) ? one : mone, inp[0]);
            for (int j = 1; j < 8; j++)
                base = h_add(base, h_mul(((lx >> j) & 1) ? one : mone, inp[j]));
            t[lx] = base;
        }
        for (int s = s0; s < 8; s++) {
            uint16_t iv = h_mul(two, inp[s]);
            for (int lx = 0; lx < lut_x_size; lx++)
                for (int i = (1 << s); i < (1 << (s + 1)); i += lut_x_size)
                    t[i + lx] = h_add(t[i + lx - (1 << s)], iv);
        }
    }
}

void orc_ref_kernel_fp16(const uint32_t *bW, const uint16_t *alpha, const uint16_t *zoff,
                         const uint16_t *x, int K, int N, int q, int group_size, int fused,
                         uint16_t *y)
{
    const int k_tile = zoff ? 32 : 64;
    const int tables = k_tile / 8;
    uint16_t *lut = (uint16_t *)malloc(sizeof(uint16_t) * (size_t)tables * 256);
    for (int n = 0; n < N; n++) y[n] = 0;
    for (int by = 0; by * k_tile < K; by++) {
        ref_build_lut(x + (long)by * k_tile, k_tile, lut);
        const uint32_t *W = bW + (long)by * (k_tile / 32) * q * N;
        int g = (by * k_tile) / group_size;
        for (int n = 0; n < N; n++) {
            uint16_t o = 0;
            if (zoff) {
                uint16_t t = 0;
                for (int kt = 0; kt < k_tile / 32; kt++)
                    for (int i = 0; i < 4; i++) t = h_add(t, lut[(kt * 4 + i) * 256 + 255]);
                uint16_t a = zoff[(long)g * N + n];
                o = fused ? h_fma(a, t, o) : h_add(o, h_mul(a, t));
            }
            for (int b = 0; b < q; b++) {
                uint16_t a = alpha[((long)g * q + b) * N + n];
                uint16_t t = 0;
                for (int kt = 0; kt < k_tile / 32; kt++) {
                    uint32_t w = W[((long)kt * q + b) * N + n];
                    for (int i = 0; i < 4; i++)
                        t = h_add(t, lut[(kt * 4 + i) * 256 + ((w >> (8 * i)) & 255u)]);
                }
                o = fused ? h_fma(a, t, o) : h_add(o, h_mul(a, t));
            }
            y[n] = h_add(y[n], o); /* atomicAdd(half2) on a zeroed output */
        }
    }
    free(lut);
}

/* ------------------------------------------------------------------------------------
 * Uniform (round-to-nearest) codes expressed as BCQ with an offset,
 * examples/rtn_parameter.py:77-96: w = s*(c - z0), c = sum_i 2^i bit_i  ==>
 *   alpha_i = s * 2^i / 2,  sign_i = 2*bit_i - 1,  offset = sum_i alpha_i - s*z0.
 * Inputs: codes[K][N] (0..2^q-1), scale[G][N], zero[G][N] as float.  Outputs in the
 * container's host-side input layout: bW[K/32][q][N], alpha[G][q][N], off[G][N] (float).
 * ---------------------------------------------------------------------------------- */
void orc_rtn_to_bcq(const uint8_t *codes, const float *scale, const float *zero, int K, int N,
                    int q, int group_size, uint32_t *bW, float *alpha, float *off)
{
    int G = K / group_size;
    memset(bW, 0, sizeof(uint32_t) * (size_t)(K / 32) * q * N);
    for (int k = 0; k < K; k++)
        for (int n = 0; n < N; n++) {
            unsigned c = codes[(long)k * N + n];
            for (int b = 0; b < q; b++)
                if ((c >> b) & 1u) bW[((long)(k / 32) * q + b) * N + n] |= 1u << (k % 32);
        }
    for (int g = 0; g < G; g++)
        for (int n = 0; n < N; n++) {
            float s = scale[(long)g * N + n];
            float sum = 0.0f;
            for (int b = 0; b < q; b++) {
                float a = s * 0.5f * (float)(1u << b);
                alpha[((long)g * q + b) * N + n] = a;
                sum += a;
            }
            off[(long)g * N + n] = sum - s * zero[(long)g * N + n];
        }
}

/* ------------------------------------------------------------------------------------
 * Error figures: mean |a-b| as the reference's dead checker would print
 * (tests/opt/fp16/int3_col_wise_matmul_fp16.cu:163-172), plus max-abs and relative L2.
 * out[0]=mean abs, out[1]=max abs, out[2]=||a-b||2/||b||2.
 * ---------------------------------------------------------------------------------- */
void orc_error_stats(const uint16_t *a_h, const double *b, long count, double *out)
{
    double sum = 0.0, mx = 0.0, num = 0.0, den = 0.0;
    for (long i = 0; i < count; i++) {
        double d = fabs((double)orc_h2f(a_h[i]) - b[i]);
        sum += d;
        if (d > mx) mx = d;
        num += d * d;
        den += b[i] * b[i];
    }
    out[0] = count ? sum / (double)count : 0.0;
    out[1] = mx;
    out[2] = den > 0.0 ? sqrt(num / den) : 0.0;
}
