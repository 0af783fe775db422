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
//    add their partials into a per-output fixed-point integer with one 64-bit atomic; the
//    last arrival finishes the output.  Integer sums do not depend on arrival order, so the
//    result is deterministic, and no memset or floating-point atomic on y is needed.
//  * Batches take two activation rows per pass over the weight (lut_matvec2_kernel: table
//    entries hold both rows, one 8-byte LDS read per lookup).
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <type_traits>
#include <utility>

#include "device_util.h"
#include "kernels.h"
#include "layout.h"
#include "tile_device.h"

namespace lutgemm_kernels {
using namespace lutgemm_layout;

namespace {

// Split-k words of the allocation-free entry point.  In host code this name is not a device
// address, only the handle hipGetSymbolAddress takes; kernels get the address it returns.
static __device__ __align__(256) unsigned long long scratch[kStaticSplitKWords];

constexpr int kTableFloats = 256 * kLanes;  // one table set: 64 KiB

// ------------------------------------------------------------------------------------------
// Eight table lookups with their scaled accumulation, written in GCN assembly so that a lookup
// costs two vector ALU instructions and one LDS read:
//     v_perm_b32      address = {LDS bits 31..16, sign byte, lane * 4} = entry * 256 + lane * 4
//     ds_read_b32     value   = table[entry][lane]
//     v_fmac_f32_dpp  acc    += scale (fetched from the lane that holds it) * value
// The compiler does not fold the cross-lane fetch into the multiply-add by itself and keeps
// far more lookups in flight than the register budget allows, hence the hand scheduling: all
// eight reads are issued, then each multiply-add waits only for its own value.
//
// Hazard note: a DPP instruction must not read a VGPR that a vector ALU instruction wrote in the
// two preceding issue slots.  The only DPP-read registers are the scale registers; every block
// puts at least sixteen other instructions (or an s_nop 1) before its first DPP read, so
// nothing the compiler places just before a block can violate this.
//
// Operands: %0-%7 accumulators, %8-%15 scratch, %16/%17 the two sign dwords, %18 lane offset
// (its upper half carries LDS address bits 16 and up), %19-%22 byte selectors, %23 (%24) scales.
// The "memory" clobber keeps the compiler from hoisting the next tiles' global loads above the
// lookups of the current one, which would double the registers a tile in flight costs.
// ------------------------------------------------------------------------------------------
#define LG_ADDR_AND_READ                                                                             \
    "v_perm_b32 %8, %16, %18, %19\n v_perm_b32 %9, %16, %18, %20\n v_perm_b32 %10, %16, %18, %21\n"   \
    "v_perm_b32 %11, %16, %18, %22\n v_perm_b32 %12, %17, %18, %19\n v_perm_b32 %13, %17, %18, %20\n" \
    "v_perm_b32 %14, %17, %18, %21\n v_perm_b32 %15, %17, %18, %22\n"                                 \
    "ds_read_b32 %8, %8\n ds_read_b32 %9, %9\n ds_read_b32 %10, %10\n ds_read_b32 %11, %11\n"         \
    "ds_read_b32 %12, %12\n ds_read_b32 %13, %13\n ds_read_b32 %14, %14\n ds_read_b32 %15, %15\n"
#define LG_OUT(acc, I0, tmp)                                                                          \
    "+v"(acc[I0 + 0]), "+v"(acc[I0 + 1]), "+v"(acc[I0 + 2]), "+v"(acc[I0 + 3]), "+v"(acc[I0 + 4]),      \
        "+v"(acc[I0 + 5]), "+v"(acc[I0 + 6]), "+v"(acc[I0 + 7]), "=&v"(tmp[0]), "=&v"(tmp[1]),          \
        "=&v"(tmp[2]), "=&v"(tmp[3]), "=&v"(tmp[4]), "=&v"(tmp[5]), "=&v"(tmp[6]), "=&v"(tmp[7])
#define LG_IN(w0, w1, lane_off)                                                                        \
    "v"(w0), "v"(w1), "v"(lane_off), "s"(0x03020400u), "s"(0x03020500u), "s"(0x03020600u), "s"(0x03020700u)
#define LG_WAIT(n) "s_waitcnt lgkmcnt(" #n ")\n"
#define LG_ROW(n) " row_newbcast:" #n " row_mask:0xf bank_mask:0xf\n"
#define LG_LOHALF(n) " row_newbcast:" #n " row_mask:0xf bank_mask:0x3\n"
#define LG_HIHALF(n) " row_newbcast:" #n " row_mask:0xf bank_mask:0xc\n"
#define LG_QUAD(n) " quad_perm:[" #n "," #n "," #n "," #n "] row_mask:0xf bank_mask:0xf\n"
// multiply-add k of a block: accumulator %k, scale operand S, value %(8+k)
#define LG_FMA(k, S, v, CTRL) "v_fmac_f32_dpp %" #k ", %" #S ", %" #v CTRL

// Outputs I0..I0+7 of the batch (I0 a multiple of 8), sign bytes in w0 (outputs I0..I0+3) and
// w1 (I0+4..I0+7).  GSUB as in the scale tile layout: the scale of output i sits in
//   GSUB 1: lane i%16 of the row, in sa
//   GSUB 2: lane i%8 of each half row, in sa (two masked multiply-adds per lookup)
//   GSUB 4: lane i%4 of each quad, in sa for I0..I0+3 and sb for I0+4..I0+7
template <int GSUB, int I0>
__device__ __forceinline__ void lookup8(float (&acc)[kBatch], uint32_t w0, uint32_t w1, uint32_t lane_off,
                                        float sa, float sb)
{
    uint32_t tmp[8];
    if constexpr (GSUB == 1 && (I0 % 16) == 0) {
        asm volatile(LG_ADDR_AND_READ
                     LG_WAIT(7) LG_FMA(0, 23, 8, LG_ROW(0)) LG_WAIT(6) LG_FMA(1, 23, 9, LG_ROW(1))
                     LG_WAIT(5) LG_FMA(2, 23, 10, LG_ROW(2)) LG_WAIT(4) LG_FMA(3, 23, 11, LG_ROW(3))
                     LG_WAIT(3) LG_FMA(4, 23, 12, LG_ROW(4)) LG_WAIT(2) LG_FMA(5, 23, 13, LG_ROW(5))
                     LG_WAIT(1) LG_FMA(6, 23, 14, LG_ROW(6)) LG_WAIT(0) LG_FMA(7, 23, 15, LG_ROW(7))
                     : LG_OUT(acc, I0, tmp)
                     : LG_IN(w0, w1, lane_off), "v"(sa)
                     : "memory");
    } else if constexpr (GSUB == 1) {
        asm volatile(LG_ADDR_AND_READ
                     LG_WAIT(7) LG_FMA(0, 23, 8, LG_ROW(8)) LG_WAIT(6) LG_FMA(1, 23, 9, LG_ROW(9))
                     LG_WAIT(5) LG_FMA(2, 23, 10, LG_ROW(10)) LG_WAIT(4) LG_FMA(3, 23, 11, LG_ROW(11))
                     LG_WAIT(3) LG_FMA(4, 23, 12, LG_ROW(12)) LG_WAIT(2) LG_FMA(5, 23, 13, LG_ROW(13))
                     LG_WAIT(1) LG_FMA(6, 23, 14, LG_ROW(14)) LG_WAIT(0) LG_FMA(7, 23, 15, LG_ROW(15))
                     : LG_OUT(acc, I0, tmp)
                     : LG_IN(w0, w1, lane_off), "v"(sa)
                     : "memory");
    } else if constexpr (GSUB == 2) {
        asm volatile(LG_ADDR_AND_READ
                     LG_WAIT(7) LG_FMA(0, 23, 8, LG_LOHALF(0)) LG_FMA(0, 23, 8, LG_HIHALF(8))
                     LG_WAIT(6) LG_FMA(1, 23, 9, LG_LOHALF(1)) LG_FMA(1, 23, 9, LG_HIHALF(9))
                     LG_WAIT(5) LG_FMA(2, 23, 10, LG_LOHALF(2)) LG_FMA(2, 23, 10, LG_HIHALF(10))
                     LG_WAIT(4) LG_FMA(3, 23, 11, LG_LOHALF(3)) LG_FMA(3, 23, 11, LG_HIHALF(11))
                     LG_WAIT(3) LG_FMA(4, 23, 12, LG_LOHALF(4)) LG_FMA(4, 23, 12, LG_HIHALF(12))
                     LG_WAIT(2) LG_FMA(5, 23, 13, LG_LOHALF(5)) LG_FMA(5, 23, 13, LG_HIHALF(13))
                     LG_WAIT(1) LG_FMA(6, 23, 14, LG_LOHALF(6)) LG_FMA(6, 23, 14, LG_HIHALF(14))
                     LG_WAIT(0) LG_FMA(7, 23, 15, LG_LOHALF(7)) LG_FMA(7, 23, 15, LG_HIHALF(15))
                     : LG_OUT(acc, I0, tmp)
                     : LG_IN(w0, w1, lane_off), "v"(sa)
                     : "memory");
    } else {
        asm volatile(LG_ADDR_AND_READ
                     LG_WAIT(7) LG_FMA(0, 23, 8, LG_QUAD(0)) LG_WAIT(6) LG_FMA(1, 23, 9, LG_QUAD(1))
                     LG_WAIT(5) LG_FMA(2, 23, 10, LG_QUAD(2)) LG_WAIT(4) LG_FMA(3, 23, 11, LG_QUAD(3))
                     LG_WAIT(3) LG_FMA(4, 24, 12, LG_QUAD(0)) LG_WAIT(2) LG_FMA(5, 24, 13, LG_QUAD(1))
                     LG_WAIT(1) LG_FMA(6, 24, 14, LG_QUAD(2)) LG_WAIT(0) LG_FMA(7, 24, 15, LG_QUAD(3))
                     : LG_OUT(acc, I0, tmp)
                     : LG_IN(w0, w1, lane_off), "v"(sa), "v"(sb)
                     : "memory");
    }
}

// acc[I0..I0+7] += offset scale (fetched across lanes like any scale) * v, no table involved.
// Operands: %0-%7 accumulators, %8 v, %9 (%10) scale registers.
#define LG_OFMA(k, S, CTRL) "v_fmac_f32_dpp %" #k ", %" #S ", %8" CTRL
#define LG_OOUT(acc, I0)                                                                           \
    "+v"(acc[I0 + 0]), "+v"(acc[I0 + 1]), "+v"(acc[I0 + 2]), "+v"(acc[I0 + 3]), "+v"(acc[I0 + 4]),   \
        "+v"(acc[I0 + 5]), "+v"(acc[I0 + 6]), "+v"(acc[I0 + 7])
template <int GSUB, int I0>
__device__ __forceinline__ void offset8(float (&acc)[kBatch], float v, float sa, float sb)
{
    if constexpr (GSUB == 1 && (I0 % 16) == 0) {
        asm volatile("s_nop 1\n" LG_OFMA(0, 9, LG_ROW(0)) LG_OFMA(1, 9, LG_ROW(1)) LG_OFMA(2, 9, LG_ROW(2))
                     LG_OFMA(3, 9, LG_ROW(3)) LG_OFMA(4, 9, LG_ROW(4)) LG_OFMA(5, 9, LG_ROW(5))
                     LG_OFMA(6, 9, LG_ROW(6)) LG_OFMA(7, 9, LG_ROW(7))
                     : LG_OOUT(acc, I0) : "v"(v), "v"(sa));
    } else if constexpr (GSUB == 1) {
        asm volatile("s_nop 1\n" LG_OFMA(0, 9, LG_ROW(8)) LG_OFMA(1, 9, LG_ROW(9)) LG_OFMA(2, 9, LG_ROW(10))
                     LG_OFMA(3, 9, LG_ROW(11)) LG_OFMA(4, 9, LG_ROW(12)) LG_OFMA(5, 9, LG_ROW(13))
                     LG_OFMA(6, 9, LG_ROW(14)) LG_OFMA(7, 9, LG_ROW(15))
                     : LG_OOUT(acc, I0) : "v"(v), "v"(sa));
    } else if constexpr (GSUB == 2) {
        asm volatile("s_nop 1\n" LG_OFMA(0, 9, LG_LOHALF(0)) LG_OFMA(0, 9, LG_HIHALF(8))
                     LG_OFMA(1, 9, LG_LOHALF(1)) LG_OFMA(1, 9, LG_HIHALF(9))
                     LG_OFMA(2, 9, LG_LOHALF(2)) LG_OFMA(2, 9, LG_HIHALF(10))
                     LG_OFMA(3, 9, LG_LOHALF(3)) LG_OFMA(3, 9, LG_HIHALF(11))
                     LG_OFMA(4, 9, LG_LOHALF(4)) LG_OFMA(4, 9, LG_HIHALF(12))
                     LG_OFMA(5, 9, LG_LOHALF(5)) LG_OFMA(5, 9, LG_HIHALF(13))
                     LG_OFMA(6, 9, LG_LOHALF(6)) LG_OFMA(6, 9, LG_HIHALF(14))
                     LG_OFMA(7, 9, LG_LOHALF(7)) LG_OFMA(7, 9, LG_HIHALF(15))
                     : LG_OOUT(acc, I0) : "v"(v), "v"(sa));
    } else {
        asm volatile("s_nop 1\n" LG_OFMA(0, 9, LG_QUAD(0)) LG_OFMA(1, 9, LG_QUAD(1)) LG_OFMA(2, 9, LG_QUAD(2))
                     LG_OFMA(3, 9, LG_QUAD(3)) LG_OFMA(4, 10, LG_QUAD(0)) LG_OFMA(5, 10, LG_QUAD(1))
                     LG_OFMA(6, 10, LG_QUAD(2)) LG_OFMA(7, 10, LG_QUAD(3))
                     : LG_OOUT(acc, I0) : "v"(v), "v"(sa), "v"(sb));
    }
}

// Build one eighth (entries part*32 .. part*32+31, part wave-uniform) of this lane's 256-entry
// table from its 8 activations f[0..7]:  entry(idx) = sum_j (bit_j(idx) ? +f[j] : -f[j]).
// Split as (bits 5..7 fixed by part) + (bits 3,4) + (bits 0..2) so no entry is more than a few
// fp32 additions away from the inputs.  One code path for all parts: only `top` and the base
// address depend on part.
constexpr int kBuildParts = 8;
__device__ __forceinline__ void build_part(float *col, int part, const float (&f)[8])
{
    float lo[8];
#pragma unroll
    for (int t = 0; t < 8; t++)
        lo[t] = ((t & 1) ? f[0] : -f[0]) + ((t & 2) ? f[1] : -f[1]) + ((t & 4) ? f[2] : -f[2]);
    const float top =
        (((part & 1) ? f[5] : -f[5]) + ((part & 2) ? f[6] : -f[6])) + ((part & 4) ? f[7] : -f[7]);
    float *q = col + part * (32 * kLanes);
#pragma unroll
    for (int h = 0; h < 4; h++) {
        const float hi = top + (((h & 1) ? f[3] : -f[3]) + ((h & 2) ? f[4] : -f[4]));
#pragma unroll
        for (int t = 0; t < 8; t++) q[(h * 8 + t) * kLanes] = hi + lo[t];
        __builtin_amdgcn_sched_barrier(0);  // store each row of 8 before computing the next
    }
}

// ------------------------------------------------------------------------------------------
// Two activation rows per pass.  The table set holds, for every (entry, lane), the partial sums
// of both rows side by side (8 bytes), laid out [lane / 32][entry][lane % 32]: the address is
// still three bytes of lane constant around the sign byte (one v_perm_b32), a lookup is one
// ds_read_b64, and the 16 lanes served per LDS cycle read 16 consecutive 8-byte slots, so the
// reads stay conflict free.  Each weight byte fetched from HBM now serves two rows; per row and
// lookup the cost drops to 1.5 vector ALU instructions and half an LDS read.  Table values,
// their order of accumulation and the reduction are those of the one-row kernel, so each row's
// result is bit-identical to a one-row launch with the same plan.
//
// The 64-bit read results are named in C++ (a register pair cannot be split inside an asm
// template), so the reads and their multiply-adds are separate asm statements and the first
// one waits for all of its reads.
// ------------------------------------------------------------------------------------------
constexpr int kTable2Floats = 2 * kTableFloats;  // 128 KiB

#define LG2_FMA(k, v, CTRL) "v_fmac_f32_dpp %" #k ", %16, %" #v CTRL
#define LG2_OPS(acc0, acc1, I0, t)                                                                       \
    "+v"(acc0[I0 + 0]), "+v"(acc0[I0 + 1]), "+v"(acc0[I0 + 2]), "+v"(acc0[I0 + 3]), "+v"(acc1[I0 + 0]),   \
        "+v"(acc1[I0 + 1]), "+v"(acc1[I0 + 2]), "+v"(acc1[I0 + 3])                                        \
        : "v"((uint32_t)t[0]), "v"((uint32_t)(t[0] >> 32)), "v"((uint32_t)t[1]),                           \
          "v"((uint32_t)(t[1] >> 32)), "v"((uint32_t)t[2]), "v"((uint32_t)(t[2] >> 32)),                   \
          "v"((uint32_t)t[3]), "v"((uint32_t)(t[3] >> 32))

// acc0/acc1[I0..I0+3] += scale * (row 0 / row 1 half of t[0..3]); I0 a multiple of 4, scale
// register s holds the scales of these four outputs (see lookup8 for where in the row).
// Operands: %0-%3 row 0 accumulators, %4-%7 row 1, %8-%15 values, %16 scale, %17.. lane numbers.
template <int GSUB, int I0>
__device__ __forceinline__ void fma4x2(float (&acc0)[kBatch], float (&acc1)[kBatch],
                                       const unsigned long long (&t)[4], float s)
{
    if constexpr (GSUB == 1) {
        constexpr int L = I0 % 16;
#define LG2_CTRL(n) " row_newbcast:%" #n " row_mask:0xf bank_mask:0xf\n"
        asm volatile("s_nop 1\n" LG2_FMA(0, 8, LG2_CTRL(17)) LG2_FMA(4, 9, LG2_CTRL(17))
                     LG2_FMA(1, 10, LG2_CTRL(18)) LG2_FMA(5, 11, LG2_CTRL(18))
                     LG2_FMA(2, 12, LG2_CTRL(19)) LG2_FMA(6, 13, LG2_CTRL(19))
                     LG2_FMA(3, 14, LG2_CTRL(20)) LG2_FMA(7, 15, LG2_CTRL(20))
                     : LG2_OPS(acc0, acc1, I0, t), "v"(s), "n"(L), "n"(L + 1), "n"(L + 2), "n"(L + 3));
#undef LG2_CTRL
    } else if constexpr (GSUB == 2) {
        constexpr int L = I0 % 8;
#define LG2_LO(n) " row_newbcast:%" #n " row_mask:0xf bank_mask:0x3\n"
#define LG2_HI(n) " row_newbcast:%" #n " row_mask:0xf bank_mask:0xc\n"
        asm volatile("s_nop 1\n"
                     LG2_FMA(0, 8, LG2_LO(17)) LG2_FMA(0, 8, LG2_HI(21)) LG2_FMA(4, 9, LG2_LO(17)) LG2_FMA(4, 9, LG2_HI(21))
                     LG2_FMA(1, 10, LG2_LO(18)) LG2_FMA(1, 10, LG2_HI(22)) LG2_FMA(5, 11, LG2_LO(18)) LG2_FMA(5, 11, LG2_HI(22))
                     LG2_FMA(2, 12, LG2_LO(19)) LG2_FMA(2, 12, LG2_HI(23)) LG2_FMA(6, 13, LG2_LO(19)) LG2_FMA(6, 13, LG2_HI(23))
                     LG2_FMA(3, 14, LG2_LO(20)) LG2_FMA(3, 14, LG2_HI(24)) LG2_FMA(7, 15, LG2_LO(20)) LG2_FMA(7, 15, LG2_HI(24))
                     : LG2_OPS(acc0, acc1, I0, t), "v"(s), "n"(L), "n"(L + 1), "n"(L + 2), "n"(L + 3),
                       "n"(L + 8), "n"(L + 9), "n"(L + 10), "n"(L + 11));
#undef LG2_LO
#undef LG2_HI
    } else {
        asm volatile("s_nop 1\n" LG2_FMA(0, 8, LG_QUAD(0)) LG2_FMA(4, 9, LG_QUAD(0))
                     LG2_FMA(1, 10, LG_QUAD(1)) LG2_FMA(5, 11, LG_QUAD(1))
                     LG2_FMA(2, 12, LG_QUAD(2)) LG2_FMA(6, 13, LG_QUAD(2))
                     LG2_FMA(3, 14, LG_QUAD(3)) LG2_FMA(7, 15, LG_QUAD(3))
                     : LG2_OPS(acc0, acc1, I0, t), "v"(s));
    }
}

// Eight two-row lookups: outputs I0..I0+7 (I0 a multiple of 8), sign bytes in w0 and w1.
template <int GSUB, int I0>
__device__ __forceinline__ void lookup8x2(float (&acc0)[kBatch], float (&acc1)[kBatch], uint32_t w0,
                                          uint32_t w1, uint32_t lane_off, float sa, float sb)
{
    unsigned long long ta[4], tb[4];
    uint32_t ad[8];
    asm volatile(
        "v_perm_b32 %8, %16, %18, %19\n v_perm_b32 %9, %16, %18, %20\n v_perm_b32 %10, %16, %18, %21\n"
        "v_perm_b32 %11, %16, %18, %22\n v_perm_b32 %12, %17, %18, %19\n v_perm_b32 %13, %17, %18, %20\n"
        "v_perm_b32 %14, %17, %18, %21\n v_perm_b32 %15, %17, %18, %22\n"
        "ds_read_b64 %0, %8\n ds_read_b64 %1, %9\n ds_read_b64 %2, %10\n ds_read_b64 %3, %11\n"
        "ds_read_b64 %4, %12\n ds_read_b64 %5, %13\n ds_read_b64 %6, %14\n ds_read_b64 %7, %15\n"
        "s_waitcnt lgkmcnt(0)\n"
        : "=&v"(ta[0]), "=&v"(ta[1]), "=&v"(ta[2]), "=&v"(ta[3]), "=&v"(tb[0]), "=&v"(tb[1]), "=&v"(tb[2]),
          "=&v"(tb[3]), "=&v"(ad[0]), "=&v"(ad[1]), "=&v"(ad[2]), "=&v"(ad[3]), "=&v"(ad[4]), "=&v"(ad[5]),
          "=&v"(ad[6]), "=&v"(ad[7])
        : LG_IN(w0, w1, lane_off)
        : "memory");
    fma4x2<GSUB, I0>(acc0, acc1, ta, sa);
    fma4x2<GSUB, I0 + 4>(acc0, acc1, tb, GSUB == 4 ? sb : sa);
}

// build_part for two rows: entries are (row 0, row 1) pairs, 32 pairs per entry row.
__device__ __forceinline__ void build_part2(float2 *col, int part, const float (&f0)[8], const float (&f1)[8])
{
    float lo0[8], lo1[8];
#pragma unroll
    for (int t = 0; t < 8; t++) {
        lo0[t] = ((t & 1) ? f0[0] : -f0[0]) + ((t & 2) ? f0[1] : -f0[1]) + ((t & 4) ? f0[2] : -f0[2]);
        lo1[t] = ((t & 1) ? f1[0] : -f1[0]) + ((t & 2) ? f1[1] : -f1[1]) + ((t & 4) ? f1[2] : -f1[2]);
    }
    const float top0 =
        (((part & 1) ? f0[5] : -f0[5]) + ((part & 2) ? f0[6] : -f0[6])) + ((part & 4) ? f0[7] : -f0[7]);
    const float top1 =
        (((part & 1) ? f1[5] : -f1[5]) + ((part & 2) ? f1[6] : -f1[6])) + ((part & 4) ? f1[7] : -f1[7]);
    float2 *q = col + part * (32 * 32);
#pragma unroll
    for (int h = 0; h < 4; h++) {
        const float hi0 = top0 + (((h & 1) ? f0[3] : -f0[3]) + ((h & 2) ? f0[4] : -f0[4]));
        const float hi1 = top1 + (((h & 1) ? f1[3] : -f1[3]) + ((h & 2) ? f1[4] : -f1[4]));
#pragma unroll
        for (int t = 0; t < 8; t++) q[(h * 8 + t) * 32] = make_float2(hi0 + lo0[t], hi1 + lo1[t]);
        __builtin_amdgcn_sched_barrier(0);
    }
}


// Raw fp16 activations of this lane's chunk in k-block ts (zero beyond k or when !valid).
// Branch free for the same reason.  x is contiguous.
__device__ __forceinline__ u32x4 load_activations(const __half *x, int k, int ts, int lane, bool valid)
{
    const int kpos = (ts * kLanes + lane) * kChunk;
    const uint32_t m = 0u - (uint32_t)(valid && kpos < k);
    const u32x4 raw = *reinterpret_cast<const u32x4 *>(x + (kpos & (int)m));
    u32x4 out = raw;
    out.x &= m;
    out.y &= m;
    out.z &= m;
    out.w &= m;
    return out;
}

__device__ __forceinline__ void unpack_activations(const u32x4 &raw, float (&f)[8])
{
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const __half2 h2 = *reinterpret_cast<const __half2 *>(&w[j]);
        f[2 * j] = __low2float(h2);
        f[2 * j + 1] = __high2float(h2);
    }
    // Pin the conversion here for every wavefront.  Only some wavefronts build table parts; left
    // alone, the compiler sinks the activation load itself into that branch, behind all the tile
    // loads, and then has to wait for every outstanding load before the first build.
#pragma unroll
    for (int j = 0; j < 8; j++) asm volatile("" : "+v"(f[j]));
}

// This wavefront's share of the table set of one k-block: eight parts spread over the
// wavefronts of the workgroup.  No barrier here; the caller synchronises.
__device__ __forceinline__ void build_tables(float *table, const float (&f)[8], int lane, int wave,
                                             int waves)
{
    float *col = table + lane;
    for (int task = wave; task < kBuildParts; task += waves) build_part(col, task, f);
}

// All lookups of one tile (32 outputs x Q planes for this lane's chunk) into acc, and the
// refill of the same registers with the next tile: each 16-byte sign vector is reloaded right
// after its 16 lookups, the scale words right after their conversion.  The loads of a
// wavefront are thereby spread evenly over its compute instead of being issued in a burst
// (vector memory issue blocks the wavefront while the request queue of the CU is full).
// Scale register of output i, plane/offset slot bo: sc[(i / (16/GSUB)) * QO + bo].
template <int Q, bool OFF, int GSUB>
__device__ __forceinline__ void process_tile(TileRegs<Q, Q + (OFF ? 1 : 0), GSUB> &t, uint32_t lane_off,
                                             float chunk_sum, float (&acc)[kBatch], const NextTile &next)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    constexpr int NSC = 2 * GSUB * QO;  // scales held per lane
    constexpr int SUBL = 16 / GSUB;     // outputs per scale slot
    float sc[NSC];
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) {
        const __half2 h2 = *reinterpret_cast<const __half2 *>(&t.scale[d]);
        sc[2 * d] = __low2float(h2);
        sc[2 * d + 1] = __high2float(h2);
    }
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) t.scale[d] = __builtin_nontemporal_load(next.scale + d);
    // scale registers of the 8 outputs starting at I0 (second one only differs for GSUB 4)
    auto sa = [&](auto I0, int bo) { return sc[(I0 / SUBL) * QO + bo]; };
    auto sb = [&](auto I0, int bo) { return sc[((I0 + 4) / SUBL) * QO + bo]; };

    // offset term: q_bias[group][out] * (sum of this lane's 8 activations)
    if constexpr (OFF) {
        static_for<4>([&](auto G) {
            constexpr int I0 = G * 8;
            offset8<GSUB, I0>(acc, chunk_sum, sa(std::integral_constant<int, I0>{}, Q),
                              sb(std::integral_constant<int, I0>{}, Q));
        });
    }

    static_for<2 * Q>([&](auto U) {
        // one unit = 16 lookups = one 16-byte sign vector (plane b, output half h)
        constexpr int b = U / 2, h = U % 2;
        constexpr int I0 = h * 16;
        const u32x4 w4 = t.sign[U];
        lookup8<GSUB, I0>(acc, w4.x, w4.y, lane_off, sa(std::integral_constant<int, I0>{}, b),
                          sb(std::integral_constant<int, I0>{}, b));
        lookup8<GSUB, I0 + 8>(acc, w4.z, w4.w, lane_off, sa(std::integral_constant<int, I0 + 8>{}, b),
                              sb(std::integral_constant<int, I0 + 8>{}, b));
        t.sign[U] = __builtin_nontemporal_load(next.sign + U * next.sign_stride);
    });
}

// Sum of each of the 32 accumulators over the 64 lanes, VALU only, fixed order.
// Halving butterfly: each step pairs accumulators (i, i+half) and leaves in every lane the one
// its lane bit selects, summed with the partner lane's copy.  Lane bit 5 / 4 steps use the
// gfx950 half-wave / row swaps, bits 3 and 2 use masked row shifts, bits 1 and 0 quad
// permutes.  Lane L ends with the total of output L >> 1 (both lanes of a pair hold it).
__device__ __forceinline__ float reduce_across_lanes(float (&acc)[kBatch], int lane)
{
    auto as_u = [](float v) { return __builtin_bit_cast(unsigned, v); };
    auto as_f = [](unsigned v) { return __builtin_bit_cast(float, v); };
    // lane bit 5: swap the upper half of A with the lower half of B, then add
    static_for<16>([&](auto I) {
        const auto r = __builtin_amdgcn_permlane32_swap(as_u(acc[I]), as_u(acc[I + 16]), false, false);
        acc[I] = as_f(r[0]) + as_f(r[1]);
    });
    // lane bit 4: swap the odd rows of A with the even rows of B, then add
    static_for<8>([&](auto I) {
        const auto r = __builtin_amdgcn_permlane16_swap(as_u(acc[I]), as_u(acc[I + 8]), false, false);
        acc[I] = as_f(r[0]) + as_f(r[1]);
    });
    // lane bit 3: banks 0,1 (lanes 0..7 of a row) keep A and fetch A from lane+8,
    //             banks 2,3 keep B and fetch B from lane-8
    static_for<4>([&](auto I) {
        const float a = acc[I], b = acc[I + 4];
        const unsigned got = __builtin_amdgcn_update_dpp(
            __builtin_amdgcn_update_dpp(0u, as_u(a), 0x108 /* row_shl:8 */, 0xf, 0x3, false), as_u(b),
            0x118 /* row_shr:8 */, 0xf, 0xc, false);
        acc[I] = ((lane & 8) ? b : a) + as_f(got);
    });
    // lane bit 2: banks 0,2 keep A (fetch from lane+4), banks 1,3 keep B (fetch from lane-4)
    static_for<2>([&](auto I) {
        const float a = acc[I], b = acc[I + 2];
        const unsigned got = __builtin_amdgcn_update_dpp(
            __builtin_amdgcn_update_dpp(0u, as_u(a), 0x104 /* row_shl:4 */, 0xf, 0x5, false), as_u(b),
            0x114 /* row_shr:4 */, 0xf, 0xa, false);
        acc[I] = ((lane & 4) ? b : a) + as_f(got);
    });
    // lane bit 1: exchange inside quads (lane ^ 2)
    {
        const float a = acc[0], b = acc[1];
        const bool up = (lane & 2) != 0;
        const float send = up ? a : b;
        const unsigned got = __builtin_amdgcn_update_dpp(0u, as_u(send), 0x4e /* quad_perm:[2,3,0,1] */, 0xf,
                                                         0xf, true);
        acc[0] = (up ? b : a) + as_f(got);
    }
    // lane bit 0: both lanes of a pair end with the same total
    const unsigned other =
        __builtin_amdgcn_update_dpp(0u, as_u(acc[0]), 0xb1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, true);
    return acc[0] + as_f(other);
}

// Workgroup `block` of one matvec (the body of lut_matvec_kernel and of lut_matvec_multi_kernel).
template <int Q, bool OFF, int GSUB>
__device__ __forceinline__ void matvec_workgroup(const MatvecArgs &a, int block)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    // Two table sets: while the lookups of k-block t read one, the other is rebuilt for t+1.
    // Dynamic LDS: a workgroup with a single k-block is launched with one set only (64 KiB), so
    // that two such workgroups fit a compute unit.
    extern __shared__ float table[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
    const int waves = blockDim.x >> 6;
    const int ntile = block % a.ntiles;
    const int ks = block / a.ntiles;
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

    // Bytes 0, 2 and 3 of every lookup address: this lane's column plus the LDS address of the
    // table set in use (a multiple of 64 KiB: the tables are the kernel's only LDS object).
    const uint32_t lane_base =
        (uint32_t)lane * 4u + (uint32_t)(size_t)(__attribute__((address_space(3))) float *)table;
    // wavefronts beyond the last batch stream batch 0 and discard the result
    const size_t tile0 = (size_t)(active ? nb : 0) * a.ts;

    // One tile of registers per wavefront, refilled in place while it is consumed; activations
    // are fetched two k-blocks ahead because the table of k-block t+1 is built during t.
    TileRegs<Q, QO, GSUB> tile;
    u32x4 xcur = load_activations(x, a.k, ts0, lane, true);
    u32x4 xnext = load_activations(x, a.k, ts0 + 1, lane, ts0 + 1 < ts1);
    float f[8];
    {
        // The first table set gates every lookup of the workgroup, and a wavefront that has
        // queued a whole tile of loads behind its activations waits for the queue before it
        // gets to build.  So only the scale words and the first sign vectors go out before the
        // build, the rest of the tile right after it (measured: 5 % faster at 8 wavefronts per
        // workgroup, 1 % at 12; same loads, same order, same arithmetic).
        constexpr int kFirst = 2 < 2 * Q ? 2 : 2 * Q;
        const NextTile n0 = tile_address<Q, QO, GSUB>(signs, scales, tile0 + ts0, lane, true);
#pragma unroll
        for (int d = 0; d < GSUB * QO; d++) tile.scale[d] = __builtin_nontemporal_load(n0.scale + d);
#pragma unroll
        for (int u = 0; u < kFirst; u++) tile.sign[u] = __builtin_nontemporal_load(n0.sign + u * n0.sign_stride);
        __builtin_amdgcn_sched_barrier(0);
        unpack_activations(xcur, f);
        build_tables(table, f, lane, wave, waves);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = kFirst; u < 2 * Q; u++) tile.sign[u] = __builtin_nontemporal_load(n0.sign + u * n0.sign_stride);
        __syncthreads();
    }

    for (int ts = ts0; ts < ts1; ts++) {
        const int cur = (ts - ts0) & 1;
        const float chunk_sum = ((f[0] + f[1]) + (f[2] + f[3])) + ((f[4] + f[5]) + (f[6] + f[7]));
        const bool more = ts + 1 < ts1;
        // table set of the next k-block, if there is one
        unpack_activations(xnext, f);
        xnext = load_activations(x, a.k, ts + 2, lane, ts + 2 < ts1);
        if (more) build_tables(table + (cur ^ 1) * kTableFloats, f, lane, wave, waves);
        process_tile<Q, OFF, GSUB>(tile, lane_base + (uint32_t)cur * (kTableFloats * 4u), chunk_sum, acc,
                                   tile_address<Q, QO, GSUB>(signs, scales, tile0 + ts + 1, lane, more));
        // the next table set is complete and every lookup into the current one has finished;
        // after the last k-block each wavefront goes straight to its reduction
        if (more) __syncthreads();
    }

    const float total = reduce_across_lanes(acc, lane);
    finish_output(total, active, nb * kBatch + (lane >> 1), lane, reinterpret_cast<__half *>(a.y), a.accum, a);
}

template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(768) void lut_matvec_kernel(MatvecArgs a)
{
    matvec_workgroup<Q, OFF, GSUB>(a, blockIdx.x);
}

// Several independent one-row matvecs in one launch: the workgroups of entry i follow those of
// entry i-1 in the grid, so a compute unit that has finished its share of one matvec starts on the
// next while other units are still at the end of theirs, and the matvecs pay one launch between
// them instead of one each.  All entries share Q, OFF, GSUB and the wavefronts per workgroup.
template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(768) void lut_matvec_multi_kernel(MultiMatvecArgs m)
{
    int i = 0;
    while (i + 1 < m.count && (int)blockIdx.x >= m.first_block[i + 1]) i++;   // scalar: at most 31 steps
    matvec_workgroup<Q, OFF, GSUB>(m.entry[i], (int)blockIdx.x - m.first_block[i]);
}

// process_tile for two activation rows (tables of lookup8x2).
template <int Q, bool OFF, int GSUB>
__device__ __forceinline__ void process_tile2(TileRegs<Q, Q + (OFF ? 1 : 0), GSUB> &t, uint32_t lane_off,
                                              float chunk_sum0, float chunk_sum1, float (&acc0)[kBatch],
                                              float (&acc1)[kBatch], const NextTile &next)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    constexpr int NSC = 2 * GSUB * QO;
    constexpr int SUBL = 16 / GSUB;
    float sc[NSC];
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) {
        const __half2 h2 = *reinterpret_cast<const __half2 *>(&t.scale[d]);
        sc[2 * d] = __low2float(h2);
        sc[2 * d + 1] = __high2float(h2);
    }
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) t.scale[d] = __builtin_nontemporal_load(next.scale + d);
    auto sa = [&](auto I0, int bo) { return sc[(I0 / SUBL) * QO + bo]; };
    auto sb = [&](auto I0, int bo) { return sc[((I0 + 4) / SUBL) * QO + bo]; };

    if constexpr (OFF) {
        static_for<4>([&](auto G) {
            constexpr int I0 = G * 8;
            offset8<GSUB, I0>(acc0, chunk_sum0, sa(std::integral_constant<int, I0>{}, Q),
                              sb(std::integral_constant<int, I0>{}, Q));
            offset8<GSUB, I0>(acc1, chunk_sum1, sa(std::integral_constant<int, I0>{}, Q),
                              sb(std::integral_constant<int, I0>{}, Q));
        });
    }

    static_for<2 * Q>([&](auto U) {
        constexpr int b = U / 2, h = U % 2;
        constexpr int I0 = h * 16;
        const u32x4 w4 = t.sign[U];
        lookup8x2<GSUB, I0>(acc0, acc1, w4.x, w4.y, lane_off, sa(std::integral_constant<int, I0>{}, b),
                            sb(std::integral_constant<int, I0>{}, b));
        lookup8x2<GSUB, I0 + 8>(acc0, acc1, w4.z, w4.w, lane_off, sa(std::integral_constant<int, I0 + 8>{}, b),
                                sb(std::integral_constant<int, I0 + 8>{}, b));
        t.sign[U] = __builtin_nontemporal_load(next.sign + U * next.sign_stride);
    });
}

// Two activation rows (a.x and a.x + a.x_row_stride) against the same weight in one pass over
// its tiles.  One 128 KiB table set: it is rebuilt between two barriers at the start of every
// k-block, while the tile loads of that block (issued one block earlier) are in flight.
template <int Q, bool OFF, int GSUB>
__device__ __forceinline__ void matvec2_workgroup(const MatvecArgs &a, int block)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    __shared__ float2 table[kTable2Floats / 2];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = blockDim.x >> 6;
    const int ntile = block % a.ntiles;
    const int ks = block / a.ntiles;
    const int nb = ntile * waves + wave;
    const bool active = nb < a.nb;
    const int ts0 = ks * a.blocks_per_split;
    const int ts1 = min(ts0 + a.blocks_per_split, a.ts);

    const u32x4 *signs = reinterpret_cast<const u32x4 *>(a.signs);
    const uint32_t *scales = reinterpret_cast<const uint32_t *>(a.scales);
    const __half *x0 = reinterpret_cast<const __half *>(a.x);
    const __half *x1 = x0 + a.x_row_stride;

    float acc0[kBatch], acc1[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; i++) acc0[i] = acc1[i] = 0.f;

    // bytes 0, 2 and 3 of every lookup address: (lane % 32) * 8 + (lane / 32) * 64 KiB + LDS base
    const uint32_t lane_base = (uint32_t)(lane & 31) * 8u + ((uint32_t)(lane >> 5) << 16) +
                               (uint32_t)(size_t)(__attribute__((address_space(3))) float2 *)table;
    float2 *col = table + (lane >> 5) * (256 * 32) + (lane & 31);
    const size_t tile0 = (size_t)(active ? nb : 0) * a.ts;

    TileRegs<Q, QO, GSUB> tile;
    u32x4 xa = load_activations(x0, a.k, ts0, lane, true);
    u32x4 xb = load_activations(x1, a.k, ts0, lane, true);
    float f0[8], f1[8];
    {
        // as in the one-row kernel: the first table set goes ahead of most of the first tile
        constexpr int kFirst = 2 < 2 * Q ? 2 : 2 * Q;
        const NextTile n0 = tile_address<Q, QO, GSUB>(signs, scales, tile0 + ts0, lane, true);
#pragma unroll
        for (int d = 0; d < GSUB * QO; d++) tile.scale[d] = __builtin_nontemporal_load(n0.scale + d);
#pragma unroll
        for (int u = 0; u < kFirst; u++) tile.sign[u] = __builtin_nontemporal_load(n0.sign + u * n0.sign_stride);
        __builtin_amdgcn_sched_barrier(0);
        unpack_activations(xa, f0);
        unpack_activations(xb, f1);
        for (int task = wave; task < kBuildParts; task += waves) build_part2(col, task, f0, f1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = kFirst; u < 2 * Q; u++) tile.sign[u] = __builtin_nontemporal_load(n0.sign + u * n0.sign_stride);
    }

    for (int ts = ts0; ts < ts1; ts++) {
        const float chunk_sum0 = ((f0[0] + f0[1]) + (f0[2] + f0[3])) + ((f0[4] + f0[5]) + (f0[6] + f0[7]));
        const float chunk_sum1 = ((f1[0] + f1[1]) + (f1[2] + f1[3])) + ((f1[4] + f1[5]) + (f1[6] + f1[7]));
        const bool more = ts + 1 < ts1;
        xa = load_activations(x0, a.k, ts + 1, lane, more);
        xb = load_activations(x1, a.k, ts + 1, lane, more);
        __syncthreads();  // the table set of this k-block is complete
        process_tile2<Q, OFF, GSUB>(tile, lane_base, chunk_sum0, chunk_sum1, acc0, acc1,
                                    tile_address<Q, QO, GSUB>(signs, scales, tile0 + ts + 1, lane, more));
        if (more) {  // workgroup-uniform
            unpack_activations(xa, f0);
            unpack_activations(xb, f1);
            __syncthreads();  // every lookup into the current table set has finished
            for (int task = wave; task < kBuildParts; task += waves) build_part2(col, task, f0, f1);
        }
    }

    const int out = nb * kBatch + (lane >> 1);
    __half *y = reinterpret_cast<__half *>(a.y);
    const float total0 = reduce_across_lanes(acc0, lane);
    const float total1 = reduce_across_lanes(acc1, lane);
    const bool valid0 = active && (lane & 1) == 0 && out < a.n, valid1 = valid0 && a.rows > 1;
    __half *y0 = y + (size_t)out * a.y_stride, *y1 = y0 + a.y_row_stride;
    if (a.k_splits == 1) {
        if (valid0) *y0 = __float2half_rn(total0);
        if (valid1) *y1 = __float2half_rn(total1);
        return;
    }
    // both atomics go out before the first answer is looked at
    unsigned long long *w0 = a.accum + out, *w1 = w0 + a.accum_row_stride;
    const Arrival r0 = arrive_output(total0, valid0, w0);
    const Arrival r1 = arrive_output(total1, valid1, w1);
    // both answers are looked at before the first output is written (pinned by the empty asm statement)
    unsigned last = (unsigned)arrived_last(r0, valid0, a.k_splits) | ((unsigned)arrived_last(r1, valid1, a.k_splits) << 1);
    asm volatile("" : "+v"(last) : : "memory");
    if (last & 1u) finish_last(r0, w0, y0, a.k_splits);
    if (last & 2u) finish_last(r1, w1, y1, a.k_splits);
}

template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(768) void lut_matvec2_kernel(MatvecArgs a)
{
    matvec2_workgroup<Q, OFF, GSUB>(a, blockIdx.x);
}

// Several independent two-row passes in one launch, laid out like the one-row work list.
template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(768) void lut_matvec2_multi_kernel(MultiMatvecArgs m)
{
    int i = 0;
    while (i + 1 < m.count && (int)blockIdx.x >= m.first_block[i + 1]) i++;   // scalar: at most 31 steps
    matvec2_workgroup<Q, OFF, GSUB>(m.entry[i], (int)blockIdx.x - m.first_block[i]);
}

// The matvec without its arithmetic: same grid, same tile registers, the same loads in the same
// order refilled at the same points (scale words, then one 16-byte sign vector after the other),
// the loaded data only xor-ed into a value that is never stored.  No activations, no tables.
// Its time is the device's pure-read time for the matvec's bytes in the matvec's order.
template <int Q, bool OFF, int GSUB>
__global__ __launch_bounds__(768) void read_probe_kernel(MatvecArgs a)
{
    constexpr int QO = Q + (OFF ? 1 : 0);
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int ntile = blockIdx.x % a.ntiles;
    const int ks = blockIdx.x / a.ntiles;
    const int nb = ntile * waves + wave;
    const int ts0 = ks * a.blocks_per_split;
    const int ts1 = min(ts0 + a.blocks_per_split, a.ts);
    const u32x4 *signs = reinterpret_cast<const u32x4 *>(a.signs);
    const uint32_t *scales = reinterpret_cast<const uint32_t *>(a.scales);
    const size_t tile0 = (size_t)(nb < a.nb ? nb : 0) * a.ts;

    TileRegs<Q, QO, GSUB> tile;
    load_tile(tile, tile_address<Q, QO, GSUB>(signs, scales, tile0 + ts0, lane, true));
    unsigned acc = 0;
    for (int ts = ts0; ts < ts1; ts++) {
        const NextTile next = tile_address<Q, QO, GSUB>(signs, scales, tile0 + ts + 1, lane, ts + 1 < ts1);
#pragma unroll
        for (int d = 0; d < GSUB * QO; d++) acc ^= tile.scale[d];
#pragma unroll
        for (int d = 0; d < GSUB * QO; d++) tile.scale[d] = __builtin_nontemporal_load(next.scale + d);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 2 * Q; u++) {
            // keep each refill right behind the use of its register, as in the matvec
            acc ^= tile.sign[u].x ^ tile.sign[u].y ^ tile.sign[u].z ^ tile.sign[u].w;
            tile.sign[u] = __builtin_nontemporal_load(next.sign + u * next.sign_stride);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int u = 0; u < 2 * Q; u++) acc ^= tile.sign[u].x;  // the dummy loads of the last refill
    if (a.y && acc == 0x12345678u) *static_cast<unsigned *>(a.y) = acc;
}

// x [k][m] (m vectors stored as columns) -> rows [m][k], so that the matvec kernel can read
// each vector with 16-byte loads.
__global__ __launch_bounds__(256) void gather_columns_kernel(const uint16_t *cols, uint16_t *rows, int k, int m)
{
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= (size_t)k * m) return;
    const int r = (int)(idx / k), i = (int)(idx % k);
    rows[idx] = cols[(size_t)i * m + r];
}

__global__ __launch_bounds__(256) void fill_zero_kernel(unsigned long long *words, size_t count)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x)
        words[i] = 0ull;
}

// more than 64 KiB of dynamic LDS has to be allowed once per kernel and device
template <typename Kernel>
hipError_t allow_two_table_sets(Kernel kernel, std::atomic<unsigned long long> &allowed)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (!(allowed.load(std::memory_order_relaxed) & bit)) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                2 * kTableFloats * (int)sizeof(float));
        if (e != hipSuccess) return e;
        allowed.fetch_or(bit, std::memory_order_relaxed);
    }
    return hipSuccess;
}

template <int Q, bool OFF, int GSUB>
hipError_t launch_one(const MatvecArgs &a, int workgroups, int threads, hipStream_t stream)
{
    if (a.rows == 0)  // read probe
        hipLaunchKernelGGL((read_probe_kernel<Q, OFF, GSUB>), dim3(workgroups), dim3(threads), 0, stream, a);
    else if (a.rows > 1)
        hipLaunchKernelGGL((lut_matvec2_kernel<Q, OFF, GSUB>), dim3(workgroups), dim3(threads), 0, stream, a);
    else
    {
        static std::atomic<unsigned long long> allowed{0};
        const hipError_t e = allow_two_table_sets(&lut_matvec_kernel<Q, OFF, GSUB>, allowed);
        if (e != hipSuccess) return e;
        const size_t lds = (size_t)(a.blocks_per_split == 1 ? 1 : 2) * kTableFloats * sizeof(float);
        hipLaunchKernelGGL((lut_matvec_kernel<Q, OFF, GSUB>), dim3(workgroups), dim3(threads), lds, stream, a);
    }
    return hipGetLastError();
}

template <int Q, bool OFF, int GSUB>
hipError_t launch_multi_one(const MultiMatvecArgs &m, int workgroups, int threads, hipStream_t stream)
{
    if (m.entry[0].rows > 1) {  // two-row passes (static LDS)
        hipLaunchKernelGGL((lut_matvec2_multi_kernel<Q, OFF, GSUB>), dim3(workgroups), dim3(threads), 0, stream, m);
        return hipGetLastError();
    }
    static std::atomic<unsigned long long> allowed{0};
    const hipError_t e = allow_two_table_sets(&lut_matvec_multi_kernel<Q, OFF, GSUB>, allowed);
    if (e != hipSuccess) return e;
    bool one_block = true;
    for (int i = 0; i < m.count; i++) one_block = one_block && m.entry[i].blocks_per_split == 1;
    const size_t lds = (size_t)(one_block ? 1 : 2) * kTableFloats * sizeof(float);
    hipLaunchKernelGGL((lut_matvec_multi_kernel<Q, OFF, GSUB>), dim3(workgroups), dim3(threads), lds, stream, m);
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
        case 1: return launch_off<1>(has_offset, gsub, a, workgroups, th, stream);
        case 2: return launch_off<2>(has_offset, gsub, a, workgroups, th, stream);
        case 3: return launch_off<3>(has_offset, gsub, a, workgroups, th, stream);
        case 4: return launch_off<4>(has_offset, gsub, a, workgroups, th, stream);
        case 5: return launch_off<5>(has_offset, gsub, a, workgroups, th, stream);
        case 6: return launch_off<6>(has_offset, gsub, a, workgroups, th, stream);
        case 7: return launch_off<7>(has_offset, gsub, a, workgroups, th, stream);
        case 8: return launch_off<8>(has_offset, gsub, a, workgroups, th, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t static_split_k_words(int device, unsigned long long **words)
{
    static std::mutex mutex;
    static unsigned long long *address[kMaxDevices];  // each device holds its own copy of the array
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(mutex);
    if (!address[device]) {
        unsigned long long *p = nullptr;
        const hipError_t e = hipGetSymbolAddress((void **)&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        address[device] = p;
    }
    *words = address[device];
    return hipSuccess;
}

namespace {
template <int Q>
hipError_t launch_multi_q(int has_offset, int gsub, const MultiMatvecArgs &m, int wg, int th, hipStream_t s)
{
    if (has_offset) {
        switch (gsub) {
            case 1: return launch_multi_one<Q, true, 1>(m, wg, th, s);
            case 2: return launch_multi_one<Q, true, 2>(m, wg, th, s);
            default: return launch_multi_one<Q, true, 4>(m, wg, th, s);
        }
    }
    switch (gsub) {
        case 1: return launch_multi_one<Q, false, 1>(m, wg, th, s);
        case 2: return launch_multi_one<Q, false, 2>(m, wg, th, s);
        default: return launch_multi_one<Q, false, 4>(m, wg, th, s);
    }
}
}  // namespace

hipError_t launch_matvec_multi(int q, int has_offset, int gsub, const MultiMatvecArgs &m, int workgroups, int waves,
                               hipStream_t stream)
{
    const int th = waves * kLanes;
    switch (q) {
        case 1: return launch_multi_q<1>(has_offset, gsub, m, workgroups, th, stream);
        case 2: return launch_multi_q<2>(has_offset, gsub, m, workgroups, th, stream);
        case 3: return launch_multi_q<3>(has_offset, gsub, m, workgroups, th, stream);
        case 4: return launch_multi_q<4>(has_offset, gsub, m, workgroups, th, stream);
        case 5: return launch_multi_q<5>(has_offset, gsub, m, workgroups, th, stream);
        case 6: return launch_multi_q<6>(has_offset, gsub, m, workgroups, th, stream);
        case 7: return launch_multi_q<7>(has_offset, gsub, m, workgroups, th, stream);
        case 8: return launch_multi_q<8>(has_offset, gsub, m, workgroups, th, stream);
        default: return hipErrorInvalidValue;
    }
}

hipError_t launch_fill_zero(unsigned long long *words, size_t count, hipStream_t stream)
{
    if (count == 0) return hipSuccess;
    const size_t blocks = (count + 255) / 256;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((unsigned)(blocks < 1024 ? blocks : 1024)), dim3(256), 0, stream, words,
                       count);
    return hipGetLastError();
}

hipError_t launch_gather_columns(const void *cols, void *rows, int k, int m, hipStream_t stream)
{
    const size_t total = (size_t)k * m;
    const int threads = 256;
    hipLaunchKernelGGL(gather_columns_kernel, dim3((unsigned)((total + threads - 1) / threads)), dim3(threads),
                       0, stream, static_cast<const uint16_t *>(cols), static_cast<uint16_t *>(rows), k, m);
    return hipGetLastError();
}

hipError_t launch_read_probe(int q, int has_offset, int gsub, const MatvecArgs &a, int workgroups, int waves,
                             hipStream_t stream)
{
    MatvecArgs probe = a;
    probe.rows = 0;
    probe.y = nullptr;
    return launch_matvec(q, has_offset, gsub, probe, workgroups, waves, stream);
}

}  // namespace lutgemm_kernels
