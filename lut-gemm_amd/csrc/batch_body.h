// gfx950 kernel for small batches: 3..16 activation rows against a packed BCQ weight in ONE pass
// over its tiles.
//
// The reference sends every batch larger than one row through a dense round trip: it dequantises
// the whole weight to fp16 in a scratch buffer and calls a library GEMM
// (lutGEMM/src/kernels.cu:73-79, lutGEMM/src/nQWeight_fp16.cu:93-99).  Here the packed tiles are
// streamed once, exactly as the one-row kernel streams them, and the batch is contracted on the
// matrix cores while the tile is in registers, without ever writing the signs out as numbers:
//
//  * The contraction is v_smfmac_f32_16x16x64_f16, the matrix instruction for an A operand with
//    2:4 structured sparsity: of every four consecutive K positions of A two are non-zero, and a
//    2-bit index per non-zero says which.  The B operand holds every activation twice, as the
//    pair (-x, +x); the A operand is the constant 1.0; and the SIGN BIT IS THE INDEX: non-zero e
//    of a lane picks -x or +x of its k.  A sign byte never becomes fp16 numbers, neither through a
//    table in LDS nor through vector instructions: for the 32 sign bits of a register,
//        (w & 0x55555555) | 0x88888888      and      ((w >> 1) & 0x55555555) | 0x88888888
//    are the index registers of four matrix instructions (even k and odd k of four chunks; the
//    second index of every pair of non-zeros has its high bit set because it addresses positions
//    2 and 3).  Products 1.0 * (+-x) are exact and the sums are fp32, so the only roundings are
//    fp32 additions, as in the one-row kernel.
//  * Operand layout of the instruction (measured on gfx950 with random operands): A lane
//    (kappa = lane / 16, output = lane % 16) holds non-zeros e = 0..7 for dense positions
//    K = 16 kappa + 4 (e / 2) + index; the low or high 16 bits of the index register are chosen
//    by an immediate.  B lane (kb = lane / 16, row = lane % 16) holds K = 8 kb .. 8 kb + 7 in its
//    first eight halves and K = 32 + 8 kb .. 32 + 8 kb + 7 in the second eight.  C lane
//    (kappa, row): outputs 4 kappa + v, v = 0..3.
//  * The tiles arrive "k across lanes" (lane = chunk of 8 k, 16 bytes = 16 outputs).  Per 16-byte
//    sign vector the wavefront writes its 64 x 16 bytes into a 1 KiB staging area of its own in LDS
//    and reads them back with two transposing reads (ds_read_b64_tr_b8, a gfx950 instruction: 16
//    lanes exchange the bytes of their 8-byte rows inside the LDS unit): lane (kappa, output) then
//    holds the sign bytes of its output for chunks kappa, kappa + 4, ..., kappa + 60; byte b of
//    word w is chunk kappa + 16 w + 4 b.  Step (w, hh, p) of a k-block takes bytes 2 hh and
//    2 hh + 1 of word w and the k of parity p: lane kappa contributes k = 8 c + 2 i + p for
//    c = kappa + 16 w + 8 hh (non-zeros i = 0..3) and c + 4 (non-zeros 4 + i).
//  * The activation block of a k-block lives in LDS in exactly the form the B operand wants: per
//    row and (chunk c, parity p) one 16-byte block [-x, +x] x 4 for k = 8 c + p, + 2, + 4, + 6.  A B
//    lane (kb, row) reads the blocks of chunks base + kb / 2 + 4 (kb % 2) and that + 2.
//  * After the steps of a scale group, the 16 x 16 result (outputs x rows) is multiplied by the
//    fp16 scales of that (plane, group) and added to the fp32 accumulators; the offset term uses
//    the group sums of x, which the same instruction provides with an index that always picks +x.
//  * At the end every (row, output) goes through the same split-k completion as the one-row kernel.
//
// Scale groups of 128 k and more are applied once per four steps, groups of 64 k after two.  With
// groups of 32 k a step spans two groups (its chunks c and c + 4); there the scales themselves are
// the A operand (four times the scale of the first group, four times that of the second) and
// nothing is multiplied afterwards.
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

namespace lutgemm_kernels {
using namespace lutgemm_layout;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half16 __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) unsigned char lds_byte;

// LDS reads whose order and wait counts are fixed by hand.  The compiler waits for every LDS read
// right before its first use and schedules that use early, which leaves one read in flight per
// wavefront; the contraction below instead issues the reads of a whole step (the two halves of
// the B operand, the scales of a group with its last step) ahead of the step before and waits
// with the count of younger reads (LDS reads of a wavefront return in order; a count that leaves
// out other younger LDS operations only waits longer).  The asm statements are volatile, so they
// keep their order among themselves; a result is tied to the wait that covers it by passing
// through that wait's (or a following empty) asm statement.
template <int OFFSET>
__device__ __forceinline__ half8 lds_read128_at(uint32_t addr)
{
    half8 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
template <int OFFSET>
__device__ __forceinline__ u32x4 lds_read128u_at(uint32_t addr)
{
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
template <int YOUNGER>
__device__ __forceinline__ void lds_wait(half8 &v)
{
    static_assert(YOUNGER >= 0 && YOUNGER <= 15, "lgkmcnt has four bits");
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(v) : "n"(YOUNGER));
}
__device__ __forceinline__ void after_wait(half8 &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void after_wait(u32x4 &v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void after_wait(uint32_t &v) { asm volatile("" : "+v"(v)); }
template <int OFFSET>
__device__ __forceinline__ uint32_t lds_read32_at(uint32_t addr)
{
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}

// acc + fp16 half (low or high) of pair * x; written so that the compiler can fold the conversion
// into a mixed-precision multiply-add (an inline asm instruction here would read the result of a
// matrix instruction without the wait states the compiler inserts for its own instructions)
template <bool HIGH>
__device__ __forceinline__ float fma_half(float acc, uint32_t pair, float x)
{
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    const half2v h = __builtin_bit_cast(half2v, pair);
    return __builtin_fmaf((float)(HIGH ? h.y : h.x), x, acc);
}

// One activation row of a k-block in LDS: 64 chunks x 2 parities x 16 bytes, block (c, p) at
// 16 * (16 (c % 8) + 2 (c / 8) + p), and 16 bytes of padding: the B lanes of one read differ in
// row and in c % 8 only, so the 16 lanes the LDS serves together fall into 16 different 16-byte
// slots modulo 256.
constexpr int kXRowBytes = kBlockK * 4 + 16;               // 2064
constexpr int kXBufBytes = (kBatchRows + 1) * kXRowBytes;  // 16 rows and a spare one that is never read
static_assert(batch_lds_bytes(0, 1, 1) == 2 * kXBufBytes, "kernels.h states the LDS of this kernel");
constexpr int kStageBytes = 1024;                          // per wavefront: [16 outputs][64 chunk positions]
// The activation block of k-block ts is 16 rows x 64 chunks.  Wavefront w moves rows w and
// w + waves (a launch has at least 8 wavefronts, so two rows per wavefront cover the 16 of a
// pass); lane L moves chunk 8 (L % 8) + L / 8.  The load and the LDS write are separate so that
// the load of the next block is in flight while the current one is processed.  k beyond the
// weight and rows beyond the batch read as zero.  No branches: a branch in the loop body costs
// the register allocator dearly.
__device__ __forceinline__ u32x4 load_activation_row(const MatvecArgs &a, int ts, int row, int lane, bool valid)
{
    const __half *x = reinterpret_cast<const __half *>(a.x);
    const int kpos = ts * kBlockK + (8 * (lane & 7) + (lane >> 3)) * kChunk;
    const uint32_t m = 0u - (uint32_t)(valid && row < a.rows && kpos < a.k);
    const size_t offset = ((size_t)row * (size_t)a.x_row_stride + (size_t)kpos) & (size_t)(0 - (long long)(m & 1u));
    u32x4 v = *reinterpret_cast<const u32x4 *>(x + offset);
    v.x &= m;
    v.y &= m;
    v.z &= m;
    v.w &= m;
    return v;
}

// word (x[2i], x[2i+1]) -> (-x[2i], +x[2i]) (selector 0x01000100) or (-x[2i+1], +x[2i+1]) (0x03020302)
__device__ __forceinline__ uint32_t minus_plus(uint32_t pair, uint32_t selector)
{
    return __builtin_amdgcn_perm(pair, pair, selector) ^ 0x00008000u;
}

__device__ __forceinline__ void store_activation_row(const u32x4 &v, lds_byte *buf, int row, int lane)
{
    // rows 16 and up (second rows of the wavefronts of a large workgroup) do not exist: their zeros
    // go to a spare row behind the 16, so that the store needs no branch
    const int slot = row < kBatchRows ? row : kBatchRows;
    // Chunk c = 8 (lane % 8) + lane / 8: block (c, p) at 16 (16 (c % 8) + 2 (c / 8) + p).  The first
    // store writes parity (lane / 16) % 2, the second the other one: the 16 lanes the LDS serves
    // together then differ in (c / 8, parity), that is in their 16-byte slot modulo 256.
    const int first = (lane >> 4) & 1;
    lds_byte *at = buf + slot * kXRowBytes + ((lane >> 3) * 16 + (lane & 7) * 2) * 16;
    const uint32_t sel_a = first ? 0x03020302u : 0x01000100u, sel_b = first ? 0x01000100u : 0x03020302u;
    *reinterpret_cast<__attribute__((address_space(3))) u32x4 *>(at + 16 * first) =
        u32x4{minus_plus(v.x, sel_a), minus_plus(v.y, sel_a), minus_plus(v.z, sel_a), minus_plus(v.w, sel_a)};
    *reinterpret_cast<__attribute__((address_space(3))) u32x4 *>(at + 16 * (first ^ 1)) =
        u32x4{minus_plus(v.x, sel_b), minus_plus(v.y, sel_b), minus_plus(v.z, sel_b), minus_plus(v.w, sel_b)};
}

// TWO: every wavefront stages a second activation row (batches of more rows than the workgroup
// has wavefronts).
template <int Q, bool OFF, int GSUB, int W, bool TWO>
__device__ __forceinline__ void batch_workgroup(const MatvecArgs &a, unsigned block)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    constexpr int NU = 2 * Q;            // sign vectors of a tile: plane b, output half h -> 2 b + h
    constexpr int SW = GSUB * QO;        // scale words of a lane per tile
    constexpr int SUBL = 16 / GSUB;      // lanes of a tile row per scale sub-row (scale tiles)
    // the sign vectors taken per pass over the k-block (the registers of more do not fit)
    constexpr int CH = NU <= 4 ? NU : NU % 3 == 0 ? 3 : 2;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_generic[];
    lds_byte *lds = (lds_byte *)lds_generic;
    lds_byte *xbuf = lds;

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
    lds_byte *stage = lds + 2 * kXBufBytes + wave * (kStageBytes + batch_scale_area_bytes(GSUB, QO));
    lds_byte *scale_area = stage + kStageBytes;

    const u32x4 *signs = reinterpret_cast<const u32x4 *>(a.signs);
    const uint32_t *scales = reinterpret_cast<const uint32_t *>(a.scales);
    const size_t tile0 = (size_t)(active ? nb : 0) * a.ts;

    // One tile in registers as in the one-row kernel: the sign vectors and this lane's own scale
    // words, both fetched one k-block ahead.
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
    // Rows that no wavefront stages (beyond the batch, when the workgroup has fewer wavefronts than
    // 16) keep whatever the LDS holds: a row is a column of the B operand, and its garbage stays in
    // the result column of that row, which is never stored.
    u32x4 xrow = load_activation_row(a, ts0, wave, lane, true);
    u32x4 xrow2 = u32x4{0u, 0u, 0u, 0u};
    if constexpr (TWO) xrow2 = load_activation_row(a, ts0, wave + waves, lane, true);
    store_activation_row(xrow, xbuf, wave, lane);
    if constexpr (TWO) store_activation_row(xrow2, xbuf, wave + waves, lane);

    // lane roles in the matrix instruction
    const int kappa = lane >> 4, j = lane & 15;
    // Staging.  ds_read_b64_tr_b8 works on rows of 16 lanes: every lane passes the address of an
    // 8-byte row, and lane 8 h + b of the 16 receives byte b of the rows addressed by lanes h, h + 2,
    // ..., h + 14, in that order (measured on gfx950 with tagged bytes).  Lane (kappa, s) addresses
    // outputs 8 (s % 2) .. 8 (s % 2) + 7 of chunk kappa + 4 (s / 2); lane (kappa, j) then receives
    // the sign bytes of output j for chunks kappa + 4 t, t = 0..7, and the same read 512 bytes
    // further on delivers t = 8..15.
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

    // Scales.  The matrix lane (kappa, row) needs the scales of its outputs 4 kappa .. 4 kappa + 3 (both
    // output halves) for every (group of the k-block, plane or offset); the wavefront passes its scale
    // words through an LDS area of its own so that one 16-byte read delivers them.
    // One group per 128 k: lane (r = lane / 16, jj = lane % 16) holds, as number hb = h QO + b of its
    // words, the scale of (group r, plane or offset b, output 16 h + jj).  The words go to LDS as they
    // are, [word][lane]; the four words d of lanes 16 G + 4 kappa .. + 3 are the numbers 2 d and 2 d + 1
    // of the lane's four outputs in group G.
    // Two or four groups per 128 k: lane (row r, sub-row sub, jj) holds, in slot t, the scales of
    // output t SUBL + jj for the group r GSUB + sub.  Two groups: every fp16 number goes (2-byte
    // writes) to [group][plane or offset][(output % 16) / 4][output half][output % 4].  Four groups:
    // the scales are the matrix operand themselves and take a layout of their own (see the loop).
    // (the halves are read back as wider words: the write type may alias them)
    typedef uint16_t __attribute__((may_alias)) aliasing_u16;
    const int s_jj = (lane & 15) % SUBL;
    __attribute__((address_space(3))) uint32_t *scale_w =
        reinterpret_cast<__attribute__((address_space(3))) uint32_t *>(scale_area) + lane;
    __attribute__((address_space(3))) aliasing_u16 *scale_wh = reinterpret_cast<__attribute__((address_space(3))) aliasing_u16 *>(
        scale_area + (((lane >> 4) * GSUB + (lane & 15) / SUBL) * QO * 32 + (s_jj >> 2) * 8 + (s_jj & 3)) * 2);
    // (four groups per 128 k: lane (r, sub, jj) holds group 4 r + sub = pair 2 r + sub / 2, half sub % 2)
    __attribute__((address_space(3))) aliasing_u16 *scale_w4 = reinterpret_cast<__attribute__((address_space(3))) aliasing_u16 *>(
        scale_area + ((((lane >> 4) * 2 + ((lane >> 3) & 1)) * QO * 32 + (lane & 3)) * 2 + ((lane >> 2) & 1)) * 2);
    const uint32_t saddr = (uint32_t)(size_t)(scale_area + 16 * kappa);
    // LDS byte offset (from saddr) of read number rd (0 .. QO - 1) of group G
    auto scale_read_offset = [](int G, int rd) constexpr { return GSUB == 1 ? rd * 256 + 64 * G : (G * QO + rd) * 64; };
    // acc + scale of (plane or offset B, output half H, output 4 kappa + V) out of the reads of a group * x
    auto scale_fma = [](float acc, const u32x4 (&reads)[QO], auto Bc, auto Hc, auto Vc, float x) {
        constexpr int B = Bc, H = Hc, V = Vc;
        if constexpr (GSUB == 1) {
            constexpr int hb = H * QO + B;
            const u32x4 &w = reads[hb >> 1];
            return fma_half<(hb & 1) != 0>(acc, V == 0 ? w.x : V == 1 ? w.y : V == 2 ? w.z : w.w, x);
        } else {
            const u32x4 &w = reads[B];
            return fma_half<(V & 1) != 0>(acc, H == 0 ? (V < 2 ? w.x : w.y) : (V < 2 ? w.z : w.w), x);
        }
    };

    // B operand: blocks of chunks base + kb / 2 + 4 (kb % 2) (first eight halves) and that + 2
    // (512 bytes further on), base = 16 w + 8 hh: block (base + c8, p) sits at 256 c8 + 16 (4 w + 2 hh + p)
    const int xlane = j * kXRowBytes + ((kappa >> 1) + 4 * (kappa & 1)) * 256;

    float4v acc[2];
    acc[0] = float4v{0.f, 0.f, 0.f, 0.f};
    acc[1] = float4v{0.f, 0.f, 0.f, 0.f};
    // four scale groups per 128 k: an accumulator per output half and unit of a pass, and one per
    // half for the offset term (see the contraction)
    float4v acc2[2][2], acc_off[2];
    acc2[0][0] = acc2[0][1] = acc2[1][0] = acc2[1][1] = acc_off[0] = acc_off[1] = float4v{0.f, 0.f, 0.f, 0.f};
    const float4v zero4 = float4v{0.f, 0.f, 0.f, 0.f};
    const half8 ones = {1, 1, 1, 1, 1, 1, 1, 1};
    constexpr int kAlwaysPlus = (int)0xddddddddu;   // index 1 for the first, 3 for the second non-zero of a pair
    // (kept in registers, so that the mask and the OR are one v_and_or_b32, which takes no literals)
    uint32_t mask55 = 0x55555555u, high88 = 0x88888888u;
    asm("" : "+s"(mask55));
    asm("" : "+v"(high88));

    __syncthreads();
    for (int ts = ts0; ts < ts1; ts++) {
        const int cur = (ts - ts0) & 1;
        const bool more = ts + 1 < ts1;
        const NextTile next = tile_address_uniform<Q, QO, GSUB>(signs, scales, tile0 + ts + 1, lane, more);
        xrow = load_activation_row(a, ts + 1, wave, lane, more);
        if constexpr (TWO) xrow2 = load_activation_row(a, ts + 1, wave + waves, lane, more);

        // this k-block's scales into the wavefront's LDS area, then the refill of their registers
        if constexpr (GSUB == 1) {
#pragma unroll
            for (int d = 0; d < SW; d++) scale_w[d * kLanes] = scale[d];
        } else if constexpr (GSUB == 2) {
            static_for<2 * SW>([&](auto F) {
                constexpr int f = F, t = f / QO, bo = f % QO;   // slot t: output t SUBL + jj
                constexpr int h = t / GSUB, within = (t % GSUB) * SUBL;
                scale_wh[bo * 32 + (within / 4) * 8 + h * 4] = (uint16_t)(scale[f >> 1] >> (16 * (f & 1)));
            });
        } else {
            // four groups per 128 k: the scales of the groups 2 P and 2 P + 1 of (plane or offset, output)
            // side by side in one word, [pair P][plane or offset][output half][output % 16]
            static_for<2 * SW>([&](auto F) {
                constexpr int f = F, t = f / QO, bo = f % QO;   // slot t: output 4 t + jj
                constexpr int h = t / 4;
                scale_w4[((bo * 2 + h) * 16 + (t % 4) * 4) * 2] = (uint16_t)(scale[f >> 1] >> (16 * (f & 1)));
            });
        }
        // the reads of these numbers further down are asm statements: keep the compiler from moving
        // them above the writes (no instruction is emitted)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int d = 0; d < SW; d++) scale[d] = __builtin_nontemporal_load(next.scale + d);

        const lds_byte *xr = xbuf + cur * kXBufBytes + xlane;
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
            // Steps g = 4 w + 2 hh + p of the k-block.  The LDS reads of step g + P are issued before
            // step g is waited for and contracted.
            constexpr int P = 1;
            constexpr bool WITH_OFFSET4 = OFF && C == 0;
            const uint32_t xaddr = (uint32_t)(size_t)xr;
            if constexpr (GSUB == 4) {
                // Four scale groups per 128 k: a step covers 64 k of every output, two groups (the lane's
                // chunks c and c + 4), so the scales go into the A operand instead of 1.0: four times
                // the scale of the first group, four times that of the second.  The instruction then adds
                // scale * (+-x) products (exact in fp32) of both groups into one accumulator, for every
                // plane and group alike, and nothing is left to multiply afterwards.  (With one or two
                // groups per 128 k this form measured slower than 1.0 and a multiply-add per group: matrix
                // instructions run slower the more their operand bits vary.)
                constexpr int NA = CH + (WITH_OFFSET4 ? 2 : 0);   // A operands of a step pair: the units, the offset per half
                half8 xb0[P + 1], xb1[P + 1], av[NA];
                uint32_t aw[2][NA];
                const uint32_t waddr = (uint32_t)(size_t)(scale_area + 4 * j);
                auto issue = [&](auto Gc) {
                    constexpr int g = Gc, slot = g % (P + 1), pair = g / 2;
                    xb0[slot] = lds_read128_at<16 * g>(xaddr);
                    xb1[slot] = lds_read128_at<16 * g + 512>(xaddr);
                    if constexpr (g % 2 == 0)
                        static_for<NA>([&](auto A) {
                            constexpr int U = u0 + A, bo = A < CH ? U / 2 : Q, h = A < CH ? U % 2 : A - CH;
                            aw[pair & 1][A] = lds_read32_at<((pair * QO + bo) * 2 + h) * 64>(waddr);
                        });
                };
                static_for<P>(issue);
                static_for<16>([&](auto Gc) {
                    constexpr int g = Gc, w = g / 4, hh = (g / 2) % 2, p = g % 2, slot = g % (P + 1), pair = g / 2;
                    if constexpr (g + P < 16) issue(std::integral_constant<int, (g + P < 16 ? g + P : 0)>{});
                    constexpr int ahead = g + P < 16 ? g + P : 15;
                    constexpr int younger = 2 * (ahead - g) + NA * ((ahead + 2) / 2 - (g + 2) / 2);
                    lds_wait<(younger < 15 ? younger : 15)>(xb0[slot]);
                    after_wait(xb1[slot]);
                    if constexpr (p == 0)
                        static_for<NA>([&](auto A) {
                            after_wait(aw[pair & 1][A]);
                            const uint32_t word = aw[pair & 1][A];
                            const uint32_t lo = __builtin_amdgcn_perm(word, word, 0x01000100u), hi = __builtin_amdgcn_perm(word, word, 0x03020302u);
                            av[A] = __builtin_bit_cast(half8, u32x4{lo, lo, hi, hi});
                        });
                    const half16 xb = __builtin_shufflevector(xb0[slot], xb1[slot], 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
                    static_for<CH>([&](auto I) {
                        constexpr int U = u0 + I, h = U % 2, nth = I / 2;   // the nth unit of this pass with this output half
                        const uint32_t word = w == 0 ? R[I].x : w == 1 ? R[I].y : w == 2 ? R[I].z : R[I].w;
                        const int index = (int)(((p ? word >> 1 : word) & mask55) | high88);
                        acc2[h][nth] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(av[I], xb, acc2[h][nth], index, 0, hh);
                    });
                    if constexpr (WITH_OFFSET4) {   // the offset term once per k-block, with the first pass
                        acc_off[0] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(av[NA - 2], xb, acc_off[0], kAlwaysPlus, 0, 0);
                        acc_off[1] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(av[NA - 1], xb, acc_off[1], kAlwaysPlus, 0, 0);
                    }
                });
            } else {
            // Steps per scale group: 4 (one group per 128 k) or 2 (two groups).
            constexpr int STEPS = GSUB == 1 ? 4 : 2;
            // which of the QO scale reads of a group this pass uses: those of its planes and, with the
            // first pass, of the offset
            constexpr bool WITH_OFFSET = OFF && C == 0;
            auto needed = [](int rd) constexpr {
                for (int i = 0; i < CH + 2; i++) {
                    const bool offset_term = i >= CH;
                    if (offset_term && !WITH_OFFSET) continue;
                    const int b = offset_term ? Q : (u0 + i) / 2, h = offset_term ? i - CH : (u0 + i) % 2;
                    if ((GSUB == 1 ? (h * QO + b) >> 1 : b) == rd) return true;
                }
                return false;
            };
            constexpr int SR = [&]() constexpr { int c = 0; for (int rd = 0; rd < QO; rd++) c += needed(rd) ? 1 : 0; return c; }();   // scale reads with the last step of a group
            half8 xb0[P + 1], xb1[P + 1];
            u32x4 sw[2][QO];
            float4v part[CH];
            float4v xsum = zero4;
            auto issue = [&](auto Gc) {
                constexpr int g = Gc, slot = g % (P + 1), w = g / 4, hh = (g / 2) % 2;
                constexpr int G = GSUB == 1 ? w : 2 * w + hh;
                xb0[slot] = lds_read128_at<16 * g>(xaddr);
                xb1[slot] = lds_read128_at<16 * g + 512>(xaddr);
                if constexpr (g % STEPS == STEPS - 1)
                    static_for<QO>([&](auto Bo) {
                        if constexpr (needed(Bo)) sw[(g / STEPS) & 1][Bo] = lds_read128u_at<scale_read_offset(G, Bo)>(saddr);
                    });
            };
            static_for<P>(issue);
            static_for<16>([&](auto Gc) {
                constexpr int g = Gc, w = g / 4, hh = (g / 2) % 2, p = g % 2, slot = g % (P + 1);
                constexpr bool first = g % STEPS == 0, last = g % STEPS == STEPS - 1;
                if constexpr (g + P < 16) issue(std::integral_constant<int, (g + P < 16 ? g + P : 0)>{});
                // reads younger than those of step g: the steps g + 1 .. g + P that exist, two each, and
                // the scales of the groups that end with one of them
                constexpr int ahead = g + P < 16 ? g + P : 15;
                constexpr int younger = 2 * (ahead - g) + SR * ((ahead + 1) / STEPS - (g + 1) / STEPS);
                lds_wait<(younger < 15 ? younger : 15)>(xb0[slot]);
                after_wait(xb1[slot]);
                const half16 xb = __builtin_shufflevector(xb0[slot], xb1[slot], 0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
                static_for<CH>([&](auto I) {
                    const uint32_t word = w == 0 ? R[I].x : w == 1 ? R[I].y : w == 2 ? R[I].z : R[I].w;
                    const int index = (int)(((p ? word >> 1 : word) & mask55) | high88);
                    part[I] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(ones, xb, first ? zero4 : part[I], index, 0, hh);
                });
                if constexpr (WITH_OFFSET)   // the offset term once per k-block, with the first pass
                    xsum = __builtin_amdgcn_smfmac_f32_16x16x64_f16(ones, xb, first ? zero4 : xsum, kAlwaysPlus, 0, 0);
                if constexpr (last) {
                    // (the scale reads were issued with this step's operand reads and are older than
                    // everything the wait above left in flight)
                    constexpr int S = (g / STEPS) & 1;
                    static_for<QO>([&](auto Bo) {
                        if constexpr (needed(Bo)) after_wait(sw[S][Bo]);
                    });
                    static_for<CH>([&](auto I) {
                        constexpr int U = u0 + I, b = U / 2, h = U % 2;
                        static_for<4>([&](auto Vc) {
                            constexpr int v = Vc;
                            acc[h][v] = scale_fma(acc[h][v], sw[S], std::integral_constant<int, b>{}, std::integral_constant<int, h>{}, Vc, part[I][v]);
                        });
                    });
                    if constexpr (WITH_OFFSET) {
                        static_for<2>([&](auto Hc) {
                            static_for<4>([&](auto Vc) {
                                constexpr int h = Hc, v = Vc;
                                acc[h][v] = scale_fma(acc[h][v], sw[S], std::integral_constant<int, Q>{}, Hc, Vc, xsum[v]);
                            });
                        });
                    }
                }
            });
            }
            __builtin_amdgcn_sched_barrier(0);   // one pass after the other: keeps the registers of a pass apart
        });
        store_activation_row(xrow, xbuf + (cur ^ 1) * kXBufBytes, wave, lane);
        if constexpr (TWO) store_activation_row(xrow2, xbuf + (cur ^ 1) * kXBufBytes, wave + waves, lane);
        __syncthreads();   // the next activation block is in place; this one is no longer read
    }

    if constexpr (GSUB == 4) {
        acc[0] = (acc2[0][0] + acc2[0][1]) + acc_off[0];
        acc[1] = (acc2[1][0] + acc2[1][1]) + acc_off[1];
    }
    // acc[h][v] is (activation row j, output nb * 32 + 16 h + 4 kappa + v).  The end of the workgroup
    // wants the outputs of a row side by side in the lanes (one cache line per row for its stores
    // and atomics), so each 16 x 16 tile is turned through the wavefront's staging area:
    // afterwards acc[h][v] is (activation row 4 kappa + v, output nb * 32 + 16 h + j).
    {
        __attribute__((address_space(3))) float *turn = reinterpret_cast<__attribute__((address_space(3))) float *>(stage);
#pragma unroll
        for (int h = 0; h < 2; h++) {
            asm volatile("" ::: "memory");   // the reads of the tile before are done with (LDS operations of a wavefront execute in order)
#pragma unroll
            for (int v = 0; v < 4; v++) turn[(4 * kappa + v) * 16 + j] = acc[h][v];
            asm volatile("" ::: "memory");
            acc[h] = *reinterpret_cast<__attribute__((address_space(3))) float4v *>(turn + j * 16 + 4 * kappa);
        }
        asm volatile("" ::: "memory");
    }
    // All eight split-k atomics of a lane are issued before the first answer is looked at.
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


// Launches kernel<Q, OFF, GSUB, W, TWO>(args) for the runtime (q, has_offset, gsub, rows against
// wavefronts): the same dispatch for the kernel of one batch and for the work-list kernel.  W, the
// largest workgroup the kernel is compiled for, is kBatchWaves for up to kBatchWidePlanes planes and
// kBatchWavesMin beyond (one instantiation there, the one that stages two rows per wavefront: it
// serves every batch size).
// Launcher<Q, OFF, GSUB, W, TWO>::run(args, workgroups, waves, stream) is provided by the includer.
template <template <int, bool, int, int, bool> class Launcher, typename Args>
hipError_t dispatch_batch(int q, int has_offset, int gsub, bool two, const Args &args, int workgroups, int waves,
                          hipStream_t stream)
{
    if (gsub != 1 && gsub != 2 && gsub != 4) return hipErrorInvalidValue;
    auto by_gsub = [&](auto Qc, auto OFFc) -> hipError_t {
        constexpr int Q = decltype(Qc)::value;
        constexpr bool OFF = decltype(OFFc)::value;
        constexpr int W = Q > kBatchWidePlanes ? kBatchWavesMin : kBatchWaves;
        if (waves < kBatchWavesMin || waves > batch_waves_max(gsub, Q, Q + (OFF ? 1 : 0))) return hipErrorInvalidValue;
        if constexpr (Q > kBatchWidePlanes) {
            switch (gsub) {
                case 1: return Launcher<Q, OFF, 1, W, true>::run(args, workgroups, waves, stream);
                case 2: return Launcher<Q, OFF, 2, W, true>::run(args, workgroups, waves, stream);
                default: return Launcher<Q, OFF, 4, W, true>::run(args, workgroups, waves, stream);
            }
        } else
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
        case 5: return by_offset(std::integral_constant<int, 5>{});
        case 6: return by_offset(std::integral_constant<int, 6>{});
        case 7: return by_offset(std::integral_constant<int, 7>{});
        case 8: return by_offset(std::integral_constant<int, 8>{});
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
                                batch_lds_bytes(batch_waves_max(GSUB, Q, QO), GSUB, QO));
        if (e != hipSuccess) return e;
        allowed.fetch_or(bit, std::memory_order_relaxed);
    }
    return hipSuccess;
}

}  // namespace
}  // namespace lutgemm_kernels
#endif
