// gfx950 kernel for small batches: 3..16 activation rows against a packed BCQ weight in ONE pass
// over its tiles.
//
// The reference sends every batch larger than one row through a dense round trip: it dequantises
// the whole weight to fp16 in a scratch buffer and calls a library GEMM
// (lutGEMM/src/kernels.cu:73-79, lutGEMM/src/nQWeight_fp16.cu:93-99).  Here the packed tiles are
// streamed once, exactly as the one-row kernel streams them, and the batch is contracted on the
// matrix cores while the tile is in registers:
//
//  * A sign byte (8 consecutive k of one output, one plane) is the B operand of one lane of a
//    v_mfma_f32_16x16x32_f16: its 8 sign bits become 8 fp16 values +1 / -1 by a 16-byte read from
//    a constant table in LDS (256 patterns, replicated per lane slot so that the reads are
//    bank-conflict free).  MFMA lane (kappa = lane / 16, j = lane % 16) supplies output j and, in
//    MFMA t of a k-block, chunk 4 t + kappa: the four k groups of an MFMA are four neighbouring
//    chunks, so an MFMA never mixes two scale groups and four MFMAs cover one 128-k group.
//  * The tiles arrive "k across lanes" (lane = chunk, 16 bytes = 16 outputs).  Per 16-byte sign
//    vector the wavefront writes its 64 x 16 bytes into a 1 KiB staging area of its own in LDS and
//    reads them back with two transposing reads (ds_read_b64_tr_b8, a gfx950 instruction: 16 lanes
//    exchange the bytes of their 8-byte rows inside the LDS unit): lane (kappa, j) then holds the
//    sign bytes of output j for chunks kappa, kappa + 4, ..., kappa + 60 in MFMA order.  No vector
//    instruction takes part in the transposition.
//  * The A operand is the activation block: lane (kappa, i) holds x[row i][8 k of chunk
//    4 t + kappa], read from an LDS copy that the workgroup shares (rows beyond the batch are zero).
//  * After the four MFMAs of a group, the 16 x 16 result (rows x outputs) is multiplied by the
//    fp16 scale of that (plane, group, output) and added to the fp32 accumulators; the offset
//    term uses the group sums of x, which one more MFMA chain with an all-ones operand provides.
//    Products of fp16 numbers are exact in fp32, so the only roundings are fp32 additions.
//  * At the end every (row, output) goes through the same split-k completion as the one-row kernel.
//
// Scale groups of 128 k and more are applied once per four MFMAs; groups of 64 or 32 k (two or
// four per 128 k) after two or after every MFMA, with the scales re-ordered through LDS first.
//
// This header holds the workgroup body; batch.hip wraps it into the kernel of a single batch,
// batch_multi.hip into the work-list kernel of lutgemm_matvec_many (two translation units, so that
// the many instantiations compile side by side).
#ifndef LUTGEMM_BATCH_BODY_H
#define LUTGEMM_BATCH_BODY_H

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <type_traits>

#include "device_util.h"
#include "kernels.h"
#include "layout.h"
#include "tile_device.h"

#ifndef LUTGEMM_BATCH_AHEAD
#define LUTGEMM_BATCH_AHEAD 1
#endif

namespace lutgemm_kernels {
using namespace lutgemm_layout;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) unsigned char lds_byte;

constexpr int kPatternBytes = 256 * 16 * 16;               // 64 KiB: [pattern][lane slot][16 bytes]
constexpr int kXRowBytes = kBlockK * 2 + 16;               // one activation row of a k-block, padded:
                                                           // 16 rows read at one column hit 64 different banks
constexpr int kXBufBytes = (kBatchRows + 1) * kXRowBytes;  // 17,680: 16 rows and a spare one that is never read
static_assert(batch_lds_bytes(0, 1, 1) == kPatternBytes + 2 * kXBufBytes, "kernels.h states the LDS of this kernel");
constexpr int kStageBytes = 1024;                          // per wavefront: [16 outputs][64 chunk positions]
// The activation block of k-block ts is 16 rows x 64 chunks of 16 bytes.  Wavefront w moves rows w
// and w + waves (a launch has at least 8 wavefronts, so two rows per wavefront cover the 16 of a
// pass), lane = chunk.  The load and the LDS write are separate so that the load of the next block
// is in flight while the current one is processed.  k beyond the weight and rows beyond the batch
// read as zero.  No branches: a
// branch in the loop body costs the register allocator dearly, and with straight-line code the
// wait counts of the loads stay exact.
__device__ __forceinline__ u32x4 load_activation_row(const MatvecArgs &a, int ts, int row, int lane, bool valid)
{
    const __half *x = reinterpret_cast<const __half *>(a.x);
    // A row is kept in LDS ordered [kappa = chunk % 4][t = chunk / 4]: position L holds chunk
    // 4 (L % 16) + L / 16, so that the 16-byte reads of the matrix lanes (kappa, j) at step t fall
    // into bank groups that depend on j and t only (see the read in the kernel).
    const int kpos = ts * kBlockK + (4 * (lane & 15) + (lane >> 4)) * kChunk;
    const uint32_t m = 0u - (uint32_t)(valid && row < a.rows && kpos < a.k);
    const size_t offset = ((size_t)row * (size_t)a.x_row_stride + (size_t)kpos) & (size_t)(0 - (long long)(m & 1u));
    u32x4 v = *reinterpret_cast<const u32x4 *>(x + offset);
    v.x &= m;
    v.y &= m;
    v.z &= m;
    v.w &= m;
    return v;
}

__device__ __forceinline__ void store_activation_row(const u32x4 &v, lds_byte *buf, int row, int lane)
{
    // rows 16 and up (second rows of the wavefronts of a large workgroup) do not exist: their zeros
    // go to a spare row behind the 16, so that the store needs no branch
    const int slot = row < kBatchRows ? row : kBatchRows;
    *reinterpret_cast<__attribute__((address_space(3))) u32x4 *>(buf + slot * kXRowBytes + lane * 16) = v;
}

// LDS reads whose order and wait counts are fixed by hand.  The compiler waits for every LDS read
// right before its first use and schedules that use early, which leaves one read in flight per
// wavefront; the contraction below instead issues the reads of a whole step (one activation
// operand, one expanded sign operand per unit) one or two steps ahead and waits with the exact
// count of younger reads (LDS reads of a wavefront return in order).  The asm statements are
// volatile, so they keep their order among themselves; a result is tied to the wait that covers
// it by passing through that wait's (or a following empty) asm statement.
__device__ __forceinline__ half8 lds_read128(uint32_t addr)
{
    half8 v;
    asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr));
    return v;
}
template <int OFFSET>
__device__ __forceinline__ half8 lds_read128_at(uint32_t addr)
{
    half8 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
template <int OFFSET>
__device__ __forceinline__ uint32_t lds_read32_at(uint32_t addr)
{
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
template <int YOUNGER>
__device__ __forceinline__ void lds_wait(half8 &v)
{
    static_assert(YOUNGER >= 0 && YOUNGER <= 15, "lgkmcnt has four bits");
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(YOUNGER));
}
__device__ __forceinline__ void after_wait(half8 &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void after_wait(uint32_t &v) { asm volatile("" : "+v"(v)); }

// W is the largest number of wavefronts a workgroup may have (it sets the register budget); the
// launch picks a number from eight up to it that divides the column batches of the shape well
// over the compute units.  TWO: the batch has more rows than the workgroup has wavefronts, so
// every wavefront stages a second activation row (a build of its own: the second row's load and
// store cost the batches that do not need them 2.5 %).
template <int Q, bool OFF, int GSUB, int W, bool TWO>
__device__ __forceinline__ void batch_workgroup(const MatvecArgs &a, unsigned block)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    constexpr int SW = GSUB * QO;   // scale words a lane holds per tile
    constexpr int SG = 4 / GSUB;    // matrix instructions per scale group (a k-block has 4 GSUB groups)
    constexpr int SUBL = 16 / GSUB; // lanes of a row that share a scale group
    constexpr int NU = 2 * Q;   // sign vectors (units) of a tile: unit U = plane U / 2, output half U % 2
    // Steps of LDS reads in flight ahead of the matrix instructions (0: the compiler's order), and the
    // sign vectors taken per pass over the k-block.  Up to three planes the reads are placed by hand
    // (three planes in two passes of three vectors: the registers of six do not fit); four planes
    // keep the compiler's order (with reads ahead they spill).
    constexpr int P = Q <= 3 ? LUTGEMM_BATCH_AHEAD : 0;
    constexpr int CH = P > 0 ? (NU <= 4 ? NU : 3) : NU <= 6 ? NU : NU % 6 == 0 ? 6 : NU % 5 == 0 ? 5 : NU % 4 == 0 ? 4 : 2;
    // The kernel's only LDS object, so it starts at LDS address 0: pattern addresses are formed
    // from the sign byte and a lane constant alone.
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_generic[];
    lds_byte *lds = (lds_byte *)lds_generic;
    lds_byte *pattern = lds;
    lds_byte *xbuf = lds + kPatternBytes;

    const int tid = threadIdx.x;
    const int threads = blockDim.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = threads >> 6;
    const int ntile = (int)(block % (unsigned)a.ntiles);
    const int ks = (int)(block / (unsigned)a.ntiles);
    const int nb = ntile * waves + wave;
    const bool active = nb < a.nb;
    const int ts0 = ks * a.blocks_per_split;
    const int ts1 = min(ts0 + a.blocks_per_split, a.ts);
    lds_byte *stage = lds + kPatternBytes + 2 * kXBufBytes + wave * (kStageBytes + batch_scale_area_bytes(GSUB, QO));
    lds_byte *scale_area = stage + kStageBytes;

    const u32x4 *signs = reinterpret_cast<const u32x4 *>(a.signs);
    const uint32_t *scales = reinterpret_cast<const uint32_t *>(a.scales);
    const size_t tile0 = (size_t)(active ? nb : 0) * a.ts;

    // One tile in registers as in the one-row kernel: the sign vectors and this lane's own scale
    // words, both fetched one k-block ahead.  The MFMA lanes need the scales of all four 128-k
    // groups of the k-block for their two outputs (j and 16 + j); group r is held by lane 16 r + j,
    // so every wavefront passes its scale words through a small LDS area of its own, [word][lane].
    u32x4 sign[NU];
    uint32_t scale[SW];
    {
        const NextTile n0 = tile_address_uniform<Q, QO, GSUB>(signs, scales, tile0 + ts0, lane, true);
#pragma unroll
        for (int d = 0; d < SW; d++) scale[d] = __builtin_nontemporal_load(n0.scale + d);
#pragma unroll
        for (int u = 0; u < NU; u++) sign[u] = __builtin_nontemporal_load(n0.sign + u * n0.sign_stride);
    }
    __builtin_amdgcn_sched_barrier(0);
    // Sign patterns: entry e, dword v holds the fp16 pair for bits 2v and 2v+1 of e: +1.0 where
    // the bit is set, -1.0 where it is clear.  All 16 lane slots of an entry hold the same 16 bytes.
    for (int idx = tid; idx < 256 * 16; idx += threads) {
        const uint32_t e = (uint32_t)idx >> 4;
        u32x4 m;
        m.x = (((e >> 0) & 1u) ? 0x3c00u : 0xbc00u) | (((e >> 1) & 1u) ? 0x3c000000u : 0xbc000000u);
        m.y = (((e >> 2) & 1u) ? 0x3c00u : 0xbc00u) | (((e >> 3) & 1u) ? 0x3c000000u : 0xbc000000u);
        m.z = (((e >> 4) & 1u) ? 0x3c00u : 0xbc00u) | (((e >> 5) & 1u) ? 0x3c000000u : 0xbc000000u);
        m.w = (((e >> 6) & 1u) ? 0x3c00u : 0xbc00u) | (((e >> 7) & 1u) ? 0x3c000000u : 0xbc000000u);
        *reinterpret_cast<__attribute__((address_space(3))) u32x4 *>(pattern + idx * 16) = m;
    }
    // both activation buffers start at zero
    for (int idx = tid; idx < 2 * kXBufBytes / 16; idx += threads)
        *reinterpret_cast<__attribute__((address_space(3))) u32x4 *>(xbuf + idx * 16) = u32x4{0u, 0u, 0u, 0u};
    u32x4 xrow = load_activation_row(a, ts0, wave, lane, true);
    u32x4 xrow2 = u32x4{0u, 0u, 0u, 0u};
    if constexpr (TWO) xrow2 = load_activation_row(a, ts0, wave + waves, lane, true);
    __syncthreads();   // the zeros are in place before the first rows go on top of them
    store_activation_row(xrow, xbuf, wave, lane);
    if constexpr (TWO) store_activation_row(xrow2, xbuf, wave + waves, lane);


    // lane roles
    const int kappa = lane >> 4, j = lane & 15;       // MFMA: k group and output column / activation row
    // Staging.  ds_read_b64_tr_b8 works on rows of 16 lanes: every lane passes the address of an
    // 8-byte row, and lane 8 h + b of the 16 receives byte b of the rows addressed by lanes h, h + 2,
    // ..., h + 14, in that order (measured on gfx950 with tagged bytes).  Lane (kappa, s) addresses
    // outputs 8 (s % 2) .. 8 (s % 2) + 7 of chunk kappa + 4 (s / 2); lane (kappa, j) then receives
    // the sign bytes of output j for chunks kappa + 4 t, t = 0..7, and the same read 512 bytes
    // further on delivers t = 8..15: together the 16 bytes the contraction consumes.
    // Lane c (chunk c: kap = c % 4, t = c / 4) writes its 16 bytes to the 16-byte slot
    //     16 (2 (t / 8) + kap / 2) + ((2 (t % 8) + kap % 2) xor 8 (kap / 2)),
    // chosen so that both directions are free of bank conflicts: the 16 lanes the LDS serves together
    // on a 16-byte write fall into 16 different slots modulo 16, and the 32 lanes it serves together
    // on an 8-byte read cover 256 consecutive bytes.
    const int w_kap = lane & 3, w_t = lane >> 2;
    const int w_slot = 16 * (2 * (w_t >> 3) + (w_kap >> 1)) + (((2 * (w_t & 7)) + (w_kap & 1)) ^ (8 * (w_kap >> 1)));
    __attribute__((address_space(3))) u32x4 *stage_w =
        reinterpret_cast<__attribute__((address_space(3))) u32x4 *>(stage + 16 * w_slot);
    const int r_slot = 16 * (kappa >> 1) + (((2 * (j >> 1)) + (kappa & 1)) ^ (8 * (kappa >> 1)));
    typedef int v2i __attribute__((ext_vector_type(2)));
    __attribute__((address_space(3))) v2i *stage_r0 =
        reinterpret_cast<__attribute__((address_space(3))) v2i *>(stage + 16 * r_slot + 8 * (j & 1));
    __attribute__((address_space(3))) v2i *stage_r1 =
        reinterpret_cast<__attribute__((address_space(3))) v2i *>(stage + 16 * r_slot + 8 * (j & 1) + 512);
    // bytes 0, 2 and 3 of a pattern address: lane slot and the LDS address bits above 64 KiB
    const uint32_t pattern_lane = ((uint32_t)j << 4) + (uint32_t)(size_t)pattern;

    // One group per 128 k: the scale words go to LDS as they are, [word][lane]; the matrix lane
    // (kappa, j) finds the pair (output j, output 16 + j) of 128-k group r at lane 16 r + j.
    // Two or four groups per 128 k: lane (row r, sub-row sub, jj) holds, in slot t, the scales of
    // output t SUBL + jj for the group (r, sub); each fp16 number goes to
    // [group r GSUB + sub][plane or offset][output % 16][output / 16], so that the matrix lanes
    // again read one word per (group, plane) with the pair (output j, output 16 + j).
    __attribute__((address_space(3))) uint32_t *scale_w =
        reinterpret_cast<__attribute__((address_space(3))) uint32_t *>(scale_area) + lane;
    // (the halves are read back as 32-bit words: the write type may alias them)
    typedef uint16_t __attribute__((may_alias)) aliasing_u16;
    __attribute__((address_space(3))) aliasing_u16 *scale_wh = reinterpret_cast<__attribute__((address_space(3))) aliasing_u16 *>(
        scale_area + ((((lane >> 4) * GSUB + (lane & 15) / SUBL) * QO) * 16 + (lane & 15) % SUBL) * 4);
    const __attribute__((address_space(3))) uint32_t *scale_r =
        reinterpret_cast<const __attribute__((address_space(3))) uint32_t *>(scale_area) + j;
    // LDS byte offset (from scale_r) of the word of scale group G (0 .. 4 GSUB - 1 of the k-block) that
    // holds fp16 number hb = half * QO + plane-or-offset (GSUB 1) or the pair of plane-or-offset b
    auto scale_word_offset = [](int G, int idx) constexpr {
        return GSUB == 1 ? (idx * kLanes + 16 * G) * 4 : ((G * QO + idx) * 16) * 4;
    };
    // the fp16 number of (plane or offset b, output half h) out of the words of one group
    auto scale_value = [](const uint32_t (&words)[QO], int b, int h) {
        const int hb = h * QO + b;
        const uint32_t w = GSUB == 1 ? words[hb >> 1] : words[b];
        const __half2 h2 = *reinterpret_cast<const __half2 *>(&w);
        return (GSUB == 1 ? (hb & 1) : h) ? __high2float(h2) : __low2float(h2);
    };

    float4v acc[2];
    acc[0] = float4v{0.f, 0.f, 0.f, 0.f};
    acc[1] = float4v{0.f, 0.f, 0.f, 0.f};
    const float4v zero4 = float4v{0.f, 0.f, 0.f, 0.f};
    const u32x4 ones = {0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};

    __syncthreads();
    for (int ts = ts0; ts < ts1; ts++) {
        const int cur = (ts - ts0) & 1;
        const bool more = ts + 1 < ts1;
        const NextTile next = tile_address_uniform<Q, QO, GSUB>(signs, scales, tile0 + ts + 1, lane, more);
        xrow = load_activation_row(a, ts + 1, wave, lane, more);
        if constexpr (TWO) xrow2 = load_activation_row(a, ts + 1, wave + waves, lane, more);

        // this k-block's scale words into the wavefront's LDS area, then the refill of their registers
        if constexpr (GSUB == 1) {
#pragma unroll
            for (int d = 0; d < SW; d++) scale_w[d * kLanes] = scale[d];
        } else {
            static_for<2 * SW>([&](auto F) {
                constexpr int f = F, t = f / QO, bo = f % QO;   // slot t: output t SUBL + jj
                constexpr int dest = (bo * 16 + (t % GSUB) * SUBL) * 2 + t / GSUB;   // in fp16 units from scale_wh
                scale_wh[dest] = (uint16_t)(scale[f >> 1] >> (16 * (f & 1)));
            });
        }
        // the reads of these words further down are asm statements or reads through another pointer
        // type: keep the compiler from moving them above the writes (no instruction is emitted)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int d = 0; d < SW; d++) scale[d] = __builtin_nontemporal_load(next.scale + d);
        // the words of scale group G, read when needed (the paths without hand-placed reads)
        auto scale_of = [&](int G, int b, int h) {
            const int hb = h * QO + b;
            const uint32_t w = scale_r[scale_word_offset(G, GSUB == 1 ? hb >> 1 : b) / 4];
            const __half2 h2 = *reinterpret_cast<const __half2 *>(&w);
            return (GSUB == 1 ? (hb & 1) : h) ? __high2float(h2) : __low2float(h2);
        };

        const lds_byte *xr = xbuf + cur * kXBufBytes + j * kXRowBytes + kappa * 256;
        // The sign vectors are taken CH at a time (all of them up to three planes), so that the
        // registers of a pass stay within the budget for any number of planes.
        static_for<NU / CH>([&](auto C) {
            constexpr int u0 = C * CH;
            // transpose through the staging area (LDS operations of a wavefront execute in order, so
            // the reads see the write before them and the next write comes after them); the registers
            // of a sign vector are refilled right away
            u32x4 R[CH];
            static_for<CH>([&](auto I) {
                constexpr int U = u0 + I;
                *stage_w = sign[U];
                const v2i lo = __builtin_amdgcn_ds_read_tr8_b64_v2i32(stage_r0);
                const v2i hi = __builtin_amdgcn_ds_read_tr8_b64_v2i32(stage_r1);
                R[I] = u32x4{(uint32_t)lo.x, (uint32_t)lo.y, (uint32_t)hi.x, (uint32_t)hi.y};
                sign[U] = __builtin_nontemporal_load(next.sign + U * next.sign_stride);
            });
            if constexpr (P > 0) {
                // Steps g = 0..15 of the k-block (MFMA t = g: scale group g / SG): the LDS reads of step
                // g + P are issued before step g is waited for and contracted.
                half8 xa[P + 1];
                half8 bits[P + 1][CH];
                uint32_t sw[2][QO];   // scale words of a group, read with the last step of the group
                float4v part[CH];
                float4v xsum = zero4;
                const uint32_t xaddr = (uint32_t)(size_t)xr, saddr = (uint32_t)(size_t)scale_r;
                auto issue = [&](auto Gc) {
                    constexpr int g = Gc, slot = g % (P + 1);
                    xa[slot] = lds_read128_at<g * 16>(xaddr);
                    static_for<CH>([&](auto I) {
                        const uint32_t word = g < 4 ? R[I].x : g < 8 ? R[I].y : g < 12 ? R[I].z : R[I].w;
                        constexpr uint32_t sel = 0x03020400u + ((uint32_t)(g & 3) << 8);   // address byte 1 <- sign byte g % 4
                        bits[slot][I] = lds_read128(__builtin_amdgcn_perm(word, pattern_lane, sel));
                    });
                    if constexpr (g % SG == SG - 1)
                        static_for<QO>([&](auto Wd) { sw[(g / SG) & 1][Wd] = lds_read32_at<scale_word_offset(g / SG, Wd)>(saddr); });
                };
                static_for<P>(issue);
                static_for<16>([&](auto Gc) {
                    constexpr int g = Gc, G = g / SG, TT = g % SG, slot = g % (P + 1);
                    if constexpr (g + P < 16) issue(std::integral_constant<int, (g + P < 16 ? g + P : 0)>{});
                    // reads younger than those of step g: the steps g + 1 .. g + P that exist
                    constexpr int last = g + P < 16 ? g + P : 15;
                    // (the scale words of a group are read with its last step: (x + 1) / SG groups end by step x)
                    constexpr int younger = (last - g) * (1 + CH) + QO * ((last + 1) / SG - (g + 1) / SG);
                    lds_wait<younger>(xa[slot]);
                    static_for<CH>([&](auto I) {
                        after_wait(bits[slot][I]);
                        part[I] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[slot], bits[slot][I], TT == 0 ? zero4 : part[I], 0, 0, 0);
                    });
                    if constexpr (OFF && C == 0)   // the offset term once per k-block, with the first pass
                        xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[slot], __builtin_bit_cast(half8, ones),
                                                                      TT == 0 ? zero4 : xsum, 0, 0, 0);
                    if constexpr (TT == SG - 1) {
                        static_for<QO>([&](auto Wd) { after_wait(sw[G & 1][Wd]); });
                        static_for<CH>([&](auto I) {
                            constexpr int U = u0 + I, b = U / 2, h = U % 2;
                            const float sc = scale_value(sw[G & 1], b, h);
                            acc[h][0] += sc * part[I][0];
                            acc[h][1] += sc * part[I][1];
                            acc[h][2] += sc * part[I][2];
                            acc[h][3] += sc * part[I][3];
                        });
                        if constexpr (OFF && C == 0) {
#pragma unroll
                            for (int h = 0; h < 2; h++) {
                                const float z = scale_value(sw[G & 1], Q, h);
                                acc[h][0] += z * xsum[0];
                                acc[h][1] += z * xsum[1];
                                acc[h][2] += z * xsum[2];
                                acc[h][3] += z * xsum[3];
                            }
                        }
                    }
                });
            } else {
            static_for<4 * GSUB>([&](auto G) {   // the scale groups of the k-block
                    constexpr int r = G;
                    float4v part[CH];
                    float4v xsum = zero4;
                    static_for<SG>([&](auto TT) {
                        constexpr int t = SG * r + TT;   // MFMA t: chunks 4 t .. 4 t + 3
                        const half8 xa = *reinterpret_cast<const __attribute__((address_space(3))) half8 *>(xr + t * 16);
                        static_for<CH>([&](auto I) {
                            const uint32_t word = t < 4 ? R[I].x : t < 8 ? R[I].y : t < 12 ? R[I].z : R[I].w;
                            constexpr uint32_t sel = 0x03020400u + ((uint32_t)(t & 3) << 8);   // address byte 1 <- sign byte t % 4
                            const uint32_t addr = __builtin_amdgcn_perm(word, pattern_lane, sel);
                            const half8 bits = *reinterpret_cast<const __attribute__((address_space(3))) half8 *>(addr);
                            part[I] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, bits, TT == 0 ? zero4 : part[I], 0, 0, 0);
                        });
                        if constexpr (OFF && C == 0 && NU <= 6)
                            xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, __builtin_bit_cast(half8, ones), xsum, 0, 0, 0);
                    });
                    static_for<CH>([&](auto I) {
                        constexpr int U = u0 + I, b = U / 2, h = U % 2;
                        const float s = scale_of(r, b, h);
                        acc[h][0] += s * part[I][0];
                        acc[h][1] += s * part[I][1];
                        acc[h][2] += s * part[I][2];
                        acc[h][3] += s * part[I][3];
                    });
                    if constexpr (OFF && C == 0 && NU <= 6) {
#pragma unroll
                        for (int h = 0; h < 2; h++) {
                            const float z = scale_of(r, Q, h);
                            acc[h][0] += z * xsum[0];
                            acc[h][1] += z * xsum[1];
                            acc[h][2] += z * xsum[2];
                            acc[h][3] += z * xsum[3];
                        }
                    }
                    if constexpr (NU > 6) __builtin_amdgcn_sched_barrier(0);   // many planes: keep the groups' registers apart
                });
            }
            __builtin_amdgcn_sched_barrier(0);   // one pass after the other: keeps the registers of a pass apart
        });
        if constexpr (OFF && NU > 6 && P == 0) {   // many planes: the offset term in a pass of its own
            static_for<4 * GSUB>([&](auto G) {
                constexpr int r = G;
                float4v xsum = zero4;
                static_for<SG>([&](auto TT) {
                    constexpr int t = SG * r + TT;
                    const half8 xa = *reinterpret_cast<const __attribute__((address_space(3))) half8 *>(xr + t * 16);
                    xsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa, __builtin_bit_cast(half8, ones), xsum, 0, 0, 0);
                });
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const float z = scale_of(r, Q, h);
                    acc[h][0] += z * xsum[0];
                    acc[h][1] += z * xsum[1];
                    acc[h][2] += z * xsum[2];
                    acc[h][3] += z * xsum[3];
                }
            });
        }
        store_activation_row(xrow, xbuf + (cur ^ 1) * kXBufBytes, wave, lane);
        if constexpr (TWO) store_activation_row(xrow2, xbuf + (cur ^ 1) * kXBufBytes, wave + waves, lane);
        __syncthreads();   // the next activation block is in place; this one is no longer read
    }

    // acc[h][v]: activation row 4 kappa + v, output nb * 32 + 16 h + j.  All eight split-k atomics
    // of a lane are issued before the first answer is looked at.
    __half *y = reinterpret_cast<__half *>(a.y);
    bool valid[2][4];
    unsigned long long *word[2][4];
    __half *yout[2][4];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int row = 4 * kappa + v, out = nb * kBatch + 16 * h + j;
            valid[h][v] = active && row < a.rows && out < a.n;
            word[h][v] = a.accum + (size_t)row * a.accum_row_stride + out;
            yout[h][v] = y + (size_t)row * a.y_row_stride + (size_t)out * a.y_stride;
        }
    if (a.k_splits == 1) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (valid[h][v]) *yout[h][v] = __float2half_rn(acc[h][v]);
        return;
    }
    Arrival arrival[2][4];
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int v = 0; v < 4; v++) arrival[h][v] = arrive_output(acc[h][v], valid[h][v], word[h][v]);
    // Every answer is looked at before the first output is written (see arrived_last): the eight
    // verdicts go through one register that an empty asm statement pins in front of all stores,
    // so the compiler cannot sink the wait for a later answer behind an earlier store.
    unsigned last = 0;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int v = 0; v < 4; v++) last |= (unsigned)arrived_last(arrival[h][v], valid[h][v], a.k_splits) << (4 * h + v);
    asm volatile("" : "+v"(last) : : "memory");
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
        for (int v = 0; v < 4; v++)
            if (last & (1u << (4 * h + v))) finish_last(arrival[h][v], word[h][v], yout[h][v], a.k_splits);
}


// Launches kernel<Q, OFF, GSUB, kBatchWaves, TWO>(args) for the runtime (q, has_offset, gsub, rows
// against wavefronts): the same dispatch for the kernel of one batch and for the work-list kernel.
// Launcher<Q, OFF, GSUB, W, TWO>::run(args, workgroups, waves, stream) is provided by the includer.
template <template <int, bool, int, int, bool> class Launcher, typename Args>
hipError_t dispatch_batch(int q, int has_offset, int gsub, bool two, const Args &args, int workgroups, int waves,
                          hipStream_t stream)
{
    constexpr int W = kBatchWaves;
    if (gsub != 1 && gsub != 2 && gsub != 4) return hipErrorInvalidValue;
    auto by_gsub = [&](auto Qc, auto OFFc) -> hipError_t {
        constexpr int Q = decltype(Qc)::value;
        constexpr bool OFF = decltype(OFFc)::value;
        if (waves < kBatchWavesMin || waves > batch_waves_max(gsub, Q + (OFF ? 1 : 0))) return hipErrorInvalidValue;
        switch (gsub) {
            case 1: return two ? Launcher<Q, OFF, 1, W, true>::run(args, workgroups, waves, stream)
                               : Launcher<Q, OFF, 1, W, false>::run(args, workgroups, waves, stream);
            case 2: return two ? Launcher<Q, OFF, 2, W, true>::run(args, workgroups, waves, stream)
                               : Launcher<Q, OFF, 2, W, false>::run(args, workgroups, waves, stream);
            default: return two ? Launcher<Q, OFF, 4, W, true>::run(args, workgroups, waves, stream)
                                : Launcher<Q, OFF, 4, W, false>::run(args, workgroups, waves, stream);
        }
    };
    auto by_offset = [&](auto Qc) -> hipError_t {
        return has_offset ? by_gsub(Qc, std::true_type{}) : by_gsub(Qc, std::false_type{});
    };
    switch (q) {
        case 1: return by_offset(std::integral_constant<int, 1>{});
        case 2: return by_offset(std::integral_constant<int, 2>{});
        case 3: return by_offset(std::integral_constant<int, 3>{});
        case 4: return by_offset(std::integral_constant<int, 4>{});
        default: return hipErrorInvalidValue;   // more planes than kBatchMaxPlanes
    }
}

// more than 64 KiB of dynamic LDS has to be allowed once per kernel and device
template <int Q, bool OFF, int GSUB, typename Kernel>
hipError_t allow_batch_lds(Kernel kernel, std::atomic<unsigned long long> &allowed)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (!(allowed.load(std::memory_order_relaxed) & bit)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                batch_lds_bytes(batch_waves_max(GSUB, QO), GSUB, QO));
        if (e != hipSuccess) return e;
        allowed.fetch_or(bit, std::memory_order_relaxed);
    }
    return hipSuccess;
}

}  // namespace
}  // namespace lutgemm_kernels
#endif
