// gfx950 (CDNA4, wave64) kernels of the BCQ table-lookup matvec.
//
// What the reference computes with kernel::_nqmv / kernel::_nqmv_bias
// (lutGEMM/src/cuda/kernels/mv_fp16.hpp:25-97, mv_fp16_bias.hpp:24-118) is computed here by a
// different decomposition, designed for 64-lane wavefronts and the LDS of a CDNA compute unit:
//
//  * One workgroup owns `waves` batches of 32 outputs and a contiguous range of 512-wide
//    k-blocks.  For each k-block it builds ONE table set in LDS: 64 tables (one per 8-k chunk)
//    of 256 fp32 partial sums, laid out [entry 0..255][lane 0..63].  Lane L only ever reads
//    column L, so every lookup of a wavefront hits 64 different dwords in 64 different bank
//    slots: the lookups are bank-conflict free for any sign data.
//  * Lane L of every wavefront works on chunk L of the k-block ("k across lanes").  Its sign
//    bytes for 32 outputs x q planes arrive as 2q fully coalesced 16-byte loads.  A lookup is
//    one v_perm_b32 (byte -> LDS address), one ds_read_b32 and one FMA whose scale operand is
//    broadcast from the lane of the same row that holds it (DPP), accumulating in fp32.
//  * After the last k-block the 64 per-lane partial sums of each output are reduced across the
//    wavefront in a fixed order.  With more than one k-split the workgroups of a column tile
//    write fp32 partials and the last one to finish adds them in ascending split order, so the
//    result is deterministic and no memset or atomic accumulation of y is needed.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <type_traits>
#include <utility>

#include "kernels.h"
#include "layout.h"

namespace lutgemm_kernels {
using namespace lutgemm_layout;

namespace {

constexpr int kTableFloats = 256 * kLanes;  // one table set: 64 KiB

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// compile-time loop: body(std::integral_constant<int, I>) for I in [0, N)
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&body, std::integer_sequence<int, Is...>)
{
    (body(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&body)
{
    static_for_impl(body, std::make_integer_sequence<int, N>{});
}

__device__ __forceinline__ float lds_lookup(const float *lds, uint32_t byte_addr)
{
    return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(lds) + byte_addr);
}

// a * v + acc with `a` taken from another lane of the same DPP row / half row / quad.
// CTRL is the DPP control word, BANKS the bank mask (which 4-lane groups of a row take part;
// the others see a == 0 and leave acc unchanged).
template <int CTRL, int BANKS>
__device__ __forceinline__ float fma_bcast(float a, float v, float acc)
{
    int ab = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), CTRL, 0xf, BANKS, BANKS == 0xf);
    return __builtin_fmaf(__builtin_bit_cast(float, ab), v, acc);
}

constexpr int kRowBcast = 0x150;  // DPP control of row_newbcast:0

// acc += scale(output I, slot BO) * v, the scale coming from the lane that holds it.
//   GSUB 1: lane I%16 of the row, register slot I/16
//   GSUB 2: lane I%8 of each half row (two masked instructions), slot I/8
//   GSUB 4: lane I%4 of each quad, slot I/4
template <int GSUB, int QO, int I, int BO, int NSC>
__device__ __forceinline__ float scaled_add(const float (&sc)[NSC], float v, float acc)
{
    if constexpr (GSUB == 1) {
        return fma_bcast<kRowBcast + (I % 16), 0xf>(sc[(I / 16) * QO + BO], v, acc);
    } else if constexpr (GSUB == 2) {
        const float s = sc[(I / 8) * QO + BO];
        acc = fma_bcast<kRowBcast + (I % 8), 0x3>(s, v, acc);
        return fma_bcast<kRowBcast + 8 + (I % 8), 0xc>(s, v, acc);
    } else {
        return fma_bcast<(I % 4) * 0x55, 0xf>(sc[(I / 4) * QO + BO], v, acc);
    }
}

// Build one quarter (entries qtr*64 .. qtr*64+63, qtr wave-uniform) of this lane's 256-entry
// table from its 8 activations f[0..7]:  entry(idx) = sum_j (bit_j(idx) ? +f[j] : -f[j]).
// Split as (bits 6,7 fixed by qtr) + (bits 3..5) + (bits 0..2) so no entry is more than a
// few fp32 additions away from the inputs.  One code path for all quarters: only `top` and
// the base address depend on qtr.
__device__ __forceinline__ void build_quarter(float *col, int qtr, const float (&f)[8])
{
    float lo[8];
#pragma unroll
    for (int t = 0; t < 8; t++)
        lo[t] = ((t & 1) ? f[0] : -f[0]) + ((t & 2) ? f[1] : -f[1]) + ((t & 4) ? f[2] : -f[2]);
    const float top = ((qtr & 1) ? f[6] : -f[6]) + ((qtr & 2) ? f[7] : -f[7]);
    float *q = col + qtr * (64 * kLanes);
#pragma unroll
    for (int h = 0; h < 8; h++) {
        const float hi =
            top + (((h & 1) ? f[3] : -f[3]) + ((h & 2) ? f[4] : -f[4]) + ((h & 4) ? f[5] : -f[5]));
#pragma unroll
        for (int t = 0; t < 8; t++) q[(h * 8 + t) * kLanes] = hi + lo[t];
    }
}

template <int Q, int QO, int GSUB>
struct TileRegs {
    u32x4 sign[2 * Q];
    uint32_t scale[GSUB * QO];
};

template <int Q, int QO, int GSUB>
__device__ __forceinline__ void load_tile(TileRegs<Q, QO, GSUB> &r, const u32x4 *signs,
                                          const uint32_t *scales, size_t tile, int lane)
{
    const uint32_t *cp = scales + (tile * kLanes + lane) * (size_t)(GSUB * QO);
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) r.scale[d] = __builtin_nontemporal_load(cp + d);
    const u32x4 *sp = signs + tile * (size_t)(2 * Q * kLanes) + lane;
#pragma unroll
    for (int u = 0; u < 2 * Q; u++) r.sign[u] = __builtin_nontemporal_load(sp + u * kLanes);
}

// This lane's 8 activations of k-block ts as fp32 (zero beyond k).
__device__ __forceinline__ void load_activations(const __half *x, int x_stride, int k, int ts, int lane,
                                                 float (&f)[8])
{
    const int kpos = (ts * kLanes + lane) * kChunk;
    if (kpos < k) {
        if (x_stride == 1) {
            const uint4 raw = *reinterpret_cast<const uint4 *>(x + kpos);
            const __half *hp = reinterpret_cast<const __half *>(&raw);
#pragma unroll
            for (int j = 0; j < 8; j++) f[j] = __half2float(hp[j]);
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) f[j] = __half2float(x[(size_t)(kpos + j) * x_stride]);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) f[j] = 0.f;
    }
}

// Rebuild the table set for this lane's chunk.  Two barriers: the first makes sure every
// lookup into the previous table set has completed, the second publishes the new one.
__device__ __forceinline__ void build_tables(float *table, const float (&f)[8], int lane, int wave,
                                             int waves)
{
    __syncthreads();
    float *col = table + lane;
    for (int task = wave; task < 4; task += waves) build_quarter(col, task, f);
    __syncthreads();
}

// All lookups of one tile (32 outputs x Q planes for this lane's chunk) into acc.
template <int Q, bool OFF, int GSUB>
__device__ __forceinline__ void process_tile(const TileRegs<Q, Q + (OFF ? 1 : 0), GSUB> &t,
                                             const float *table, uint32_t lane_off, float chunk_sum,
                                             float (&acc)[kBatch])
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    constexpr int NSC = 2 * GSUB * QO;  // scales held per lane
    float sc[NSC];
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) {
        const __half2 h2 = *reinterpret_cast<const __half2 *>(&t.scale[d]);
        sc[2 * d] = __low2float(h2);
        sc[2 * d + 1] = __high2float(h2);
    }

    // offset term: q_bias[group][out] * (sum of this lane's 8 activations)
    if constexpr (OFF) {
        static_for<kBatch>([&](auto I) {
            acc[I] = scaled_add<GSUB, QO, I, Q, NSC>(sc, chunk_sum, acc[I]);
        });
    }

    static_for<2 * Q>([&](auto U) {
        constexpr int b = U / 2, h = U % 2;
        const u32x4 w4 = t.sign[U];
        const uint32_t w[4] = {w4.x, w4.y, w4.z, w4.w};
        static_for<16>([&](auto P) {
            constexpr int i = h * 16 + P;
            // address = entry * 256 + lane * 4: sign byte -> address byte 1,
            // lane_off -> address byte 0, upper bytes zero
            constexpr uint32_t sel = 0x0c0c0400u | ((uint32_t)(P % 4) << 8);
            const uint32_t addr = __builtin_amdgcn_perm(w[P / 4], lane_off, sel);
            const float v = lds_lookup(table, addr);
            acc[i] = scaled_add<GSUB, QO, i, b, NSC>(sc, v, acc[i]);
        });
        // keep the 16 lookups of a unit together: bounds the registers in flight
        __builtin_amdgcn_sched_barrier(0);
    });
}

template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(768) void lut_matvec_kernel(MatvecArgs a)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    __shared__ float table[kTableFloats];
    __shared__ int last_flag;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
    const int waves = blockDim.x >> 6;
    const int ntile = blockIdx.x % a.ntiles;
    const int ks = blockIdx.x / a.ntiles;
    const int nb = ntile * waves + wave;
    const bool active = nb < a.nb;
    const int ts0 = ks * a.blocks_per_split;
    const int ts1 = min(ts0 + a.blocks_per_split, a.ts);

    const u32x4 *signs = reinterpret_cast<const u32x4 *>(a.signs);
    const uint32_t *scales = reinterpret_cast<const uint32_t *>(a.scales);
    const __half *x = reinterpret_cast<const __half *>(a.x);

    float acc[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; i++) acc[i] = 0.f;

    // byte 0 of every lookup address: this lane's column
    const uint32_t lane_off = (uint32_t)lane * 4u;
    // inactive wavefronts (beyond the last batch) stream batch 0 and discard the result
    const size_t tile0 = (size_t)(active ? nb : 0) * a.ts;

    TileRegs<Q, QO, GSUB> cur, nxt;
    load_tile(cur, signs, scales, tile0 + ts0, lane);

    float f[8];
    for (int ts = ts0; ts < ts1 - 1; ts++) {
        load_activations(x, a.x_stride, a.k, ts, lane, f);
        build_tables(table, f, lane, wave, waves);
        load_tile(nxt, signs, scales, tile0 + ts + 1, lane);
        const float chunk_sum = ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]));
        process_tile<Q, OFF, GSUB>(cur, table, lane_off, chunk_sum, acc);
        cur = nxt;
    }
    {
        load_activations(x, a.x_stride, a.k, ts1 - 1, lane, f);
        build_tables(table, f, lane, wave, waves);
        const float chunk_sum = ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]));
        process_tile<Q, OFF, GSUB>(cur, table, lane_off, chunk_sum, acc);
    }

    // Reduce the 64 per-lane partials of each of the 32 outputs.  Halving butterfly over lane
    // bits 5..1 (after the step with mask M, value index bit log2(M)-1 equals the lane's bit
    // log2(M)), then one full exchange over bit 0: lane L ends with the total of output L>>1.
    static_for<5>([&](auto LV) {
        constexpr int half = 16 >> LV;
        constexpr int mask = half * 2;
        const bool upper = (lane & mask) != 0;
        static_for<half>([&](auto I) {
            const float keep = upper ? acc[I + half] : acc[I];
            const float send = upper ? acc[I] : acc[I + half];
            acc[I] = keep + __shfl_xor(send, mask, 64);
        });
    });
    const float total = acc[0] + __shfl_xor(acc[0], 1, 64);

    const int out = nb * kBatch + (lane >> 1);
    __half *y = reinterpret_cast<__half *>(a.y);
    if (a.k_splits == 1) {
        if (active && (lane & 1) == 0 && out < a.n) y[(size_t)out * a.y_stride] = __float2half_rn(total);
        return;
    }

    // split-k: publish this workgroup's partials, the last workgroup of the column tile adds
    // all of them in ascending split order.
    const size_t npad = (size_t)a.nb * kBatch;
    if (active && (lane & 1) == 0) a.partials[(size_t)ks * npad + out] = total;
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned ticket =
            __hip_atomic_fetch_add(a.counters + ntile, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        last_flag = (ticket == (unsigned)(a.k_splits - 1));
    }
    __syncthreads();
    if (!last_flag) return;
    __threadfence();
    for (int o = tid; o < waves * kBatch; o += blockDim.x) {
        const int col = ntile * waves * kBatch + o;
        if (col < a.n) {
            float s = 0.f;
            for (int i = 0; i < a.k_splits; i++)
                s += __builtin_nontemporal_load(a.partials + (size_t)i * npad + col);
            y[(size_t)col * a.y_stride] = __float2half_rn(s);
        }
    }
    if (tid == 0) a.counters[ntile] = 0u;  // ready for the next launch on this stream
}

// ------------------------------------------------------------------------------------------
// Dense fp16 weight from the packed tiles: W[k][n] or W[n][k], offset included.
// One thread per (chunk, output): reads its q sign bytes and scales, writes 8 weights.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void dequantize_kernel(DequantArgs a)
{
    const int qo = a.q + a.has_offset;
    const int subl = 16 / a.gsub;
    const int lh = 2 * a.gsub * qo;
    const size_t chunks = (size_t)a.k / kChunk;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= chunks * (size_t)a.n) return;
    int out, c;
    if (a.transposed) {  // consecutive threads -> consecutive chunks of one output row
        c = (int)(idx % chunks);
        out = (int)(idx / chunks);
    } else {             // consecutive threads -> consecutive outputs of one chunk
        out = (int)(idx % (size_t)a.n);
        c = (int)(idx / (size_t)a.n);
    }
    const int nb = out / kBatch, i = out % kBatch, h = i / 16, p = i % 16;
    const int ts = c / kLanes, lane = c % kLanes;
    const size_t tile = (size_t)nb * a.ts + ts;
    const int r = lane / 16, j = lane % 16, sub = j / subl;
    // lane of the same sub-row that holds this output's scales, and the slot inside it
    const int holder = r * 16 + sub * subl + (i % subl);
    const int slot = i / subl;
    const __half *sc =
        reinterpret_cast<const __half *>(a.scales) + (tile * kLanes + holder) * (size_t)lh + slot * qo;
    float w[8];
    const float off = a.has_offset ? __half2float(sc[a.q]) : 0.f;
#pragma unroll
    for (int t = 0; t < 8; t++) w[t] = off;
    for (int b = 0; b < a.q; b++) {
        const uint8_t byte = a.signs[(tile * (size_t)(2 * a.q) + 2 * b + h) * kUnitBytes + lane * 16 + p];
        const float al = __half2float(sc[b]);
#pragma unroll
        for (int t = 0; t < 8; t++) w[t] += ((byte >> t) & 1) ? al : -al;
    }
    __half *dst = reinterpret_cast<__half *>(a.out);
    if (a.transposed) {
        __half hv[8];
#pragma unroll
        for (int t = 0; t < 8; t++) hv[t] = __float2half_rn(w[t]);
        *reinterpret_cast<uint4 *>(dst + (size_t)out * a.k + (size_t)c * kChunk) =
            *reinterpret_cast<const uint4 *>(hv);
    } else {
#pragma unroll
        for (int t = 0; t < 8; t++) dst[((size_t)c * kChunk + t) * a.n + out] = __float2half_rn(w[t]);
    }
}

template <int Q, bool OFF, int GSUB>
hipError_t launch_one(const MatvecArgs &a, int workgroups, int threads, hipStream_t stream)
{
    hipLaunchKernelGGL((lut_matvec_kernel<Q, OFF, GSUB>), dim3(workgroups), dim3(threads), 0, stream, a);
    return hipGetLastError();
}

template <int Q, bool OFF>
hipError_t launch_gsub(int gsub, const MatvecArgs &a, int wg, int th, hipStream_t s)
{
    switch (gsub) {
        case 1: return launch_one<Q, OFF, 1>(a, wg, th, s);
        case 2: return launch_one<Q, OFF, 2>(a, wg, th, s);
        default: return launch_one<Q, OFF, 4>(a, wg, th, s);
    }
}

template <int Q>
hipError_t launch_off(int has_offset, int gsub, const MatvecArgs &a, int wg, int th, hipStream_t s)
{
    return has_offset ? launch_gsub<Q, true>(gsub, a, wg, th, s) : launch_gsub<Q, false>(gsub, a, wg, th, s);
}

}  // namespace

hipError_t launch_matvec(int q, int has_offset, int gsub, const MatvecArgs &a, int workgroups,
                         int waves, hipStream_t stream)
{
    const int th = waves * kLanes;
    switch (q) {
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 1
        case 1: return launch_off<1>(has_offset, gsub, a, workgroups, th, stream);
#endif
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 2
        case 2: return launch_off<2>(has_offset, gsub, a, workgroups, th, stream);
#endif
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 3
        case 3: return launch_off<3>(has_offset, gsub, a, workgroups, th, stream);
#endif
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 4
        case 4: return launch_off<4>(has_offset, gsub, a, workgroups, th, stream);
#endif
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 5
        case 5: return launch_off<5>(has_offset, gsub, a, workgroups, th, stream);
#endif
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 6
        case 6: return launch_off<6>(has_offset, gsub, a, workgroups, th, stream);
#endif
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 7
        case 7: return launch_off<7>(has_offset, gsub, a, workgroups, th, stream);
#endif
#if !defined(LUTGEMM_DEV_ONLY_Q) || LUTGEMM_DEV_ONLY_Q == 8
        case 8: return launch_off<8>(has_offset, gsub, a, workgroups, th, stream);
#endif
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_dequantize(const DequantArgs &a, hipStream_t stream)
{
    const size_t total = (size_t)(a.k / kChunk) * (size_t)a.n;
    const int threads = 256;
    const size_t blocks = (total + threads - 1) / threads;
    if (blocks > 0x7fffffffu) return hipErrorInvalidValue;
    hipLaunchKernelGGL(dequantize_kernel, dim3((unsigned)blocks), dim3(threads), 0, stream, a);
    return hipGetLastError();
}

}  // namespace lutgemm_kernels
