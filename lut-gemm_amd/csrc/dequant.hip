// gfx950 kernels that expand a packed BCQ weight to dense fp16.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "kernels.h"
#include "layout.h"

namespace lutgemm_kernels {
using namespace lutgemm_layout;

namespace {

// ------------------------------------------------------------------------------------------
// dequantize_kernel: dense fp16 weight W^T [n][k] from the packed tiles, offset included.
// One wavefront per tile (32 outputs x 512 k), lane L on chunk L as in the matvec: 2q coalesced
// 16-byte sign loads and one scale record per lane, scales fetched across lanes with DPP, then
// per weight the fp32 sum  offset +- alpha_0 +- alpha_1 ...  in plane order (the order of
// lutGEMM::dequantize_cpu, lutGEMM/src/nQWeight_fp16.cu:38-59, so offset-free results are
// bit-identical to it), one rounding to fp16, 16-byte stores: 8 consecutive k of one output
// (a wavefront writes 1 KiB runs of a row of W[n][k]).  A workgroup is four wavefronts on four
// neighbouring batches of the same k-block.  (dequantize_rows_kernel below writes W[k][n].)
// ------------------------------------------------------------------------------------------
template <int GSUB, int LANE_IN_SUB>
__device__ __forceinline__ float scale_from_holder(float v)
{
    const unsigned u = __builtin_bit_cast(unsigned, v);
    if constexpr (GSUB == 1) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, u, 0x150 + LANE_IN_SUB, 0xf, 0xf, false));
    } else if constexpr (GSUB == 2) {
        const unsigned lo = __builtin_amdgcn_update_dpp(0u, u, 0x150 + LANE_IN_SUB, 0xf, 0x3, false);
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(lo, u, 0x150 + 8 + LANE_IN_SUB, 0xf, 0xc, false));
    } else {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0u, u, LANE_IN_SUB * 0x55, 0xf, 0xf, false));
    }
}

// The 8 x 8 weights of outputs P0 .. P0+7 of one half of a batch for this lane's chunk:
// sgh[b] = the lane's 16 sign bytes of plane b for that half, sch = the GSUB scale slots of that
// half as held by this lane.  fp32 sum  offset +- alpha_0 +- alpha_1 ...  in plane order.
template <int Q, bool OFF, int GSUB, int P0>
__device__ __forceinline__ void expand_step(const u32x4 (&sgh)[Q], const float (&sch)[GSUB * (Q + (OFF ? 1 : 0))],
                                            float (&w)[8][8])
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    constexpr int SUBL = 16 / GSUB;
    static_for<8>([&](auto OI) {
        constexpr int oi = OI;
        constexpr int ih = P0 + oi;  // output within the half
        float s[QO];
#pragma unroll
        for (int bo = 0; bo < QO; bo++) s[bo] = scale_from_holder<GSUB, ih % SUBL>(sch[(ih / SUBL) * QO + bo]);
        uint32_t byte[Q];
#pragma unroll
        for (int b = 0; b < Q; b++) {
            const uint32_t word = ih / 4 == 0 ? sgh[b].x : ih / 4 == 1 ? sgh[b].y : ih / 4 == 2 ? sgh[b].z : sgh[b].w;
            byte[b] = (word >> ((ih % 4) * 8)) & 0xffu;
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
            float v = 0.f;
            if constexpr (OFF) v = s[QO - 1];
#pragma unroll
            for (int b = 0; b < Q; b++) v += ((byte[b] >> t) & 1u) ? s[b] : -s[b];
            w[oi][t] = v;
        }
    });
}

template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(256) void dequantize_kernel(DequantArgs a)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nbatches = (a.n + kBatch - 1) / kBatch;
    // neighbouring workgroups write neighbouring memory: consecutive k-blocks of the same rows
    const int ts = (int)(blockIdx.x % a.ts);
    const int bg = (int)(blockIdx.x / a.ts);
    const int nb = bg * 4 + wave;
    if (nb >= nbatches) return;
    const size_t tile = (size_t)nb * a.ts + ts;

    const u32x4 *sp = reinterpret_cast<const u32x4 *>(a.signs) + tile * (size_t)(2 * Q * kLanes) + lane;
    const uint32_t *cp = reinterpret_cast<const uint32_t *>(a.scales) + (tile * kLanes + lane) * (size_t)(GSUB * QO);
    u32x4 sg[2 * Q];
#pragma unroll
    for (int u = 0; u < 2 * Q; u++) sg[u] = __builtin_nontemporal_load(sp + u * kLanes);
    float sc[2 * GSUB * QO];  // [slot][plane or offset]
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) {
        const uint32_t rec = __builtin_nontemporal_load(cp + d);
        const __half2 h2 = *reinterpret_cast<const __half2 *>(&rec);
        sc[2 * d] = __low2float(h2);
        sc[2 * d + 1] = __high2float(h2);
    }

    const int kbase = ts * kBlockK + lane * kChunk;
    const bool k_ok = kbase < a.k;  // k is a multiple of 32: a chunk is wholly inside or outside
    __half *dst = reinterpret_cast<__half *>(a.out);

    for (int h = 0; h < 2; h++) {  // the two halves of the batch: sign units (b, h), scale slots of that half
        u32x4 sgh[Q];
#pragma unroll
        for (int b = 0; b < Q; b++) {
            sgh[b].x = h ? sg[2 * b + 1].x : sg[2 * b].x;
            sgh[b].y = h ? sg[2 * b + 1].y : sg[2 * b].y;
            sgh[b].z = h ? sg[2 * b + 1].z : sg[2 * b].z;
            sgh[b].w = h ? sg[2 * b + 1].w : sg[2 * b].w;
        }
        float sch[GSUB * QO];  // the GSUB slots of this half
#pragma unroll
        for (int d = 0; d < GSUB * QO; d++) sch[d] = h ? sc[GSUB * QO + d] : sc[d];
        static_for<2>([&](auto P) {
            constexpr int p0 = P * 8;  // outputs h*16 + p0 .. +7: bytes p0 .. p0+7 of the sign vectors
            float w[8][8];             // [output][k]
            expand_step<Q, OFF, GSUB, p0>(sgh, sch, w);
            const int col0 = nb * kBatch + h * 16 + p0;  // first of the 8 outputs
#pragma unroll
            for (int oi = 0; oi < 8; oi++) {
                if (k_ok && col0 + oi < a.n) {
                    __half2 hh[4];
#pragma unroll
                    for (int t2 = 0; t2 < 4; t2++) hh[t2] = __floats2half2_rn(w[oi][2 * t2], w[oi][2 * t2 + 1]);
                    u32x4 v;
                    v.x = *reinterpret_cast<uint32_t *>(&hh[0]);
                    v.y = *reinterpret_cast<uint32_t *>(&hh[1]);
                    v.z = *reinterpret_cast<uint32_t *>(&hh[2]);
                    v.w = *reinterpret_cast<uint32_t *>(&hh[3]);
                    *reinterpret_cast<u32x4 *>(dst + (size_t)(col0 + oi) * a.k + kbase) = v;
                }
            }
        });
    }
}

// W[k][n], n a multiple of 8.  A row of W[k][n] holds the outputs side by side, while a lane of
// the tile kernel holds 8 k of 8 outputs: written directly, every 16-byte store of a wavefront
// would go to 64 different rows.  Here a workgroup of eight wavefronts expands two neighbouring
// batches of one k-block (wavefront = batch x quarter of its outputs, the quarter's sign bytes are
// one 8-byte load per plane), transposes through LDS and writes whole 128-byte lines: 8 rows x
// 128 bytes per store instruction.  The LDS image is [512 rows][8 pieces of 16 bytes]; a piece
// is stored at position (piece ^ (row/8 & 7)) and every 64 rows are followed by 128 bytes of
// padding, so that 16 consecutive lanes (rows 8 apart) hit 16 different 16-byte bank groups
// when they write, and the read-back of 8 consecutive rows is one contiguous KiB.
constexpr int kRowsPitch = 128;                            // bytes per row: 2 batches x 32 outputs x fp16
constexpr int kRowsLds = kBlockK * kRowsPitch + 8 * 128;   // + padding after every 64 rows

__device__ __forceinline__ int rows_lds_offset(int row, int piece)
{
    return row * kRowsPitch + (row >> 6) * 128 + ((piece ^ ((row >> 3) & 7)) << 4);
}

template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(512) void dequantize_rows_kernel(DequantArgs a)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    __shared__ __attribute__((aligned(16))) unsigned char image[kRowsLds];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nbatches = (a.n + kBatch - 1) / kBatch;
    const int npairs = (nbatches + 1) / 2;
    // neighbouring workgroups write neighbouring lines of the same 512 rows
    const int pair = (int)(blockIdx.x % npairs);
    const int ts = (int)(blockIdx.x / npairs);
    const int bi = wave >> 2, st = wave & 3, h = st >> 1;
    const int nb = pair * 2 + bi;

    if (nb < nbatches) {  // wave-uniform
        const size_t tile = (size_t)nb * a.ts + ts;
        const unsigned char *sp =
            a.signs + (tile * (size_t)(2 * Q) + h) * kUnitBytes + lane * 16 + (st & 1) * 8;
        const uint32_t *cp = reinterpret_cast<const uint32_t *>(a.scales) + (tile * kLanes + lane) * (size_t)(GSUB * QO);
        // Ordinary loads, not streaming ones: the two wavefronts of a half read the two 8-byte halves of the
        // same lines, and the four wavefronts of a batch the same scale words; the later ones should find
        // them in the cache.
        // the 8 sign bytes of this quarter sit in .x/.y (first 8 outputs of the half) or .z/.w
        u32x4 sgh[Q];
#pragma unroll
        for (int b = 0; b < Q; b++) {
            const uint64_t v = *reinterpret_cast<const uint64_t *>(sp + (size_t)(2 * b) * kUnitBytes);
            sgh[b].x = sgh[b].z = (uint32_t)v;
            sgh[b].y = sgh[b].w = (uint32_t)(v >> 32);
        }
        float sc[2 * GSUB * QO];  // [slot][plane or offset]
#pragma unroll
        for (int d = 0; d < GSUB * QO; d++) {
            const uint32_t rec = cp[d];
            const __half2 h2 = *reinterpret_cast<const __half2 *>(&rec);
            sc[2 * d] = __low2float(h2);
            sc[2 * d + 1] = __high2float(h2);
        }
        float sch[GSUB * QO];  // the GSUB slots of this half
#pragma unroll
        for (int d = 0; d < GSUB * QO; d++) sch[d] = h ? sc[GSUB * QO + d] : sc[d];
        float w[8][8];  // [output][k]
        if (st & 1) expand_step<Q, OFF, GSUB, 8>(sgh, sch, w);
        else        expand_step<Q, OFF, GSUB, 0>(sgh, sch, w);
#pragma unroll
        for (int t = 0; t < 8; t++) {
            __half2 hh[4];
#pragma unroll
            for (int o2 = 0; o2 < 4; o2++) hh[o2] = __floats2half2_rn(w[2 * o2][t], w[2 * o2 + 1][t]);
            u32x4 v;
            v.x = *reinterpret_cast<uint32_t *>(&hh[0]);
            v.y = *reinterpret_cast<uint32_t *>(&hh[1]);
            v.z = *reinterpret_cast<uint32_t *>(&hh[2]);
            v.w = *reinterpret_cast<uint32_t *>(&hh[3]);
            *reinterpret_cast<u32x4 *>(image + rows_lds_offset(lane * kChunk + t, wave)) = v;
        }
    }
    __syncthreads();

    // 512 threads x 8 rounds: 64 rows x 8 pieces per round, one piece = 8 outputs of one row
    const int piece = threadIdx.x & 7;
    const int col = pair * 2 * kBatch + piece * 8;
    if (col >= a.n) return;  // n is a multiple of 8: a piece is wholly inside or outside
    __half *dst = reinterpret_cast<__half *>(a.out) + col;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int row = j * 64 + (int)(threadIdx.x >> 3);
        const int kk = ts * kBlockK + row;
        if (kk < a.k) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(image + rows_lds_offset(row, piece));
            *reinterpret_cast<u32x4 *>(dst + (size_t)kk * a.n) = v;
        }
    }
}

// W[k][n] for any n (rows of W are only 2-byte aligned when n is odd): one thread per (chunk,
// output), consecutive threads on consecutive outputs, 2-byte stores that a wavefront coalesces
// into 128-byte runs.  Same arithmetic.
__global__ __launch_bounds__(256) void dequantize_generic_kernel(DequantArgs a)
{
    const int qo = a.q + a.has_offset;
    const int subl = 16 / a.gsub;
    const int lh = 2 * a.gsub * qo;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)(a.k / kChunk) * (size_t)a.n) return;
    const int out = (int)(idx % (size_t)a.n);
    const int c = (int)(idx / (size_t)a.n);
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
#pragma unroll
    for (int t = 0; t < 8; t++) dst[((size_t)c * kChunk + t) * a.n + out] = __float2half_rn(w[t]);
}

}  // namespace

namespace {
template <int Q, bool OFF>
hipError_t launch_dequantize_gsub(const DequantArgs &a, unsigned blocks, hipStream_t stream)
{
    if (a.transposed) {
        switch (a.gsub) {
            case 1: hipLaunchKernelGGL((dequantize_kernel<Q, OFF, 1>), dim3(blocks), dim3(256), 0, stream, a); break;
            case 2: hipLaunchKernelGGL((dequantize_kernel<Q, OFF, 2>), dim3(blocks), dim3(256), 0, stream, a); break;
            default: hipLaunchKernelGGL((dequantize_kernel<Q, OFF, 4>), dim3(blocks), dim3(256), 0, stream, a); break;
        }
    } else {
        switch (a.gsub) {
            case 1: hipLaunchKernelGGL((dequantize_rows_kernel<Q, OFF, 1>), dim3(blocks), dim3(512), 0, stream, a); break;
            case 2: hipLaunchKernelGGL((dequantize_rows_kernel<Q, OFF, 2>), dim3(blocks), dim3(512), 0, stream, a); break;
            default: hipLaunchKernelGGL((dequantize_rows_kernel<Q, OFF, 4>), dim3(blocks), dim3(512), 0, stream, a); break;
        }
    }
    return hipGetLastError();
}
template <int Q>
hipError_t launch_dequantize_q(const DequantArgs &a, unsigned blocks, hipStream_t stream)
{
    return a.has_offset ? launch_dequantize_gsub<Q, true>(a, blocks, stream)
                        : launch_dequantize_gsub<Q, false>(a, blocks, stream);
}
}  // namespace

hipError_t launch_dequantize(const DequantArgs &a, hipStream_t stream)
{
    if (!a.transposed && a.n % 8 != 0) {
        const size_t total = (size_t)(a.k / kChunk) * (size_t)a.n;
        const size_t blocks = (total + 255) / 256;
        if (blocks > 0x7fffffffu) return hipErrorInvalidValue;
        hipLaunchKernelGGL(dequantize_generic_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a);
        return hipGetLastError();
    }
    const size_t nbatches = ((size_t)a.n + kBatch - 1) / kBatch;
    const size_t blocks = (a.transposed ? (nbatches + 3) / 4 : (nbatches + 1) / 2) * (size_t)a.ts;
    if (blocks > 0x7fffffffu) return hipErrorInvalidValue;
    const unsigned nblk = (unsigned)blocks;
    switch (a.q) {
        case 1: return launch_dequantize_q<1>(a, nblk, stream);
        case 2: return launch_dequantize_q<2>(a, nblk, stream);
        case 3: return launch_dequantize_q<3>(a, nblk, stream);
        case 4: return launch_dequantize_q<4>(a, nblk, stream);
        case 5: return launch_dequantize_q<5>(a, nblk, stream);
        case 6: return launch_dequantize_q<6>(a, nblk, stream);
        case 7: return launch_dequantize_q<7>(a, nblk, stream);
        case 8: return launch_dequantize_q<8>(a, nblk, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace lutgemm_kernels
