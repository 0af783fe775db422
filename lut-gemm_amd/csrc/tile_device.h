// Device-side pieces shared by the matvec kernels (kernels.hip) and the batch kernel (batch.hip):
// the registers of one weight tile with their loads, and the split-k completion of an output.
#ifndef LUTGEMM_TILE_DEVICE_H
#define LUTGEMM_TILE_DEVICE_H

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "kernels.h"
#include "layout.h"

namespace lutgemm_kernels {
using namespace lutgemm_layout;

template <int Q, int QO, int GSUB>
struct TileRegs {
    u32x4 sign[2 * Q];
    uint32_t scale[GSUB * QO];
};

// Where the next tile's loads of a wavefront come from (all lanes the same dummy line when the
// workgroup has no next k-block, see tile_address).
struct NextTile {
    const u32x4 *sign;    // this lane's first sign vector
    size_t sign_stride;   // in u32x4 units between units
    const uint32_t *scale;
};

// Addresses of tile `tile` for this lane.  `real` is wave-uniform; when false every lane reads
// the first bytes of the arrays instead (one cached line).  Written with masks rather than
// conditionals so that no branch appears: with straight-line code the compiler's wait counts
// for the loads stay exact.
template <int Q, int QO, int GSUB>
__device__ __forceinline__ NextTile tile_address(const u32x4 *signs, const uint32_t *scales, size_t tile,
                                                 int lane, bool real)
{
    const size_t m = (size_t)0 - (size_t)real;  // all ones or zero
    NextTile n;
    n.scale = scales + (((tile * kLanes + lane) * (size_t)(GSUB * QO)) & m);
    n.sign = signs + ((tile * (size_t)(2 * Q * kLanes) + lane) & m);
    n.sign_stride = (size_t)kLanes & m;
    return n;
}

// The same for a kernel that can afford a whole tile of loads past the end of its range: the tile
// number becomes 0 there (tile 0 stays in the cache: every workgroup ends on it).  `tile` and
// `real` are wave-uniform, so an address is a uniform base plus a lane constant plus an immediate
// and the address arithmetic stays on the scalar unit.
template <int Q, int QO, int GSUB>
__device__ __forceinline__ NextTile tile_address_uniform(const u32x4 *signs, const uint32_t *scales, size_t tile,
                                                         int lane, bool real)
{
    const size_t t = real ? tile : (size_t)0;
    NextTile n;
    n.scale = scales + t * (size_t)(kLanes * GSUB * QO) + lane * (GSUB * QO);
    n.sign = signs + t * (size_t)(2 * Q * kLanes) + lane;
    n.sign_stride = (size_t)kLanes;
    return n;
}

template <int Q, int QO, int GSUB>
__device__ __forceinline__ void load_tile(TileRegs<Q, QO, GSUB> &r, const NextTile &n)
{
#pragma unroll
    for (int d = 0; d < GSUB * QO; d++) r.scale[d] = __builtin_nontemporal_load(n.scale + d);
#pragma unroll
    for (int u = 0; u < 2 * Q; u++) r.sign[u] = __builtin_nontemporal_load(n.sign + u * n.sign_stride);
}

// Lane pair (2j, 2j+1) of a wavefront holds the k-range total of output `out`; the even lane
// delivers it.  With one k-split it is the result.  Otherwise: one 64-bit atomic add per output,
// no barrier, no second pass.  The word holds an arrival count in its top 8 bits and the running
// sum below it, as a biased fixed-point integer (2^-24 units, bias 2^46 per addend so every
// addend is positive; at most 128 addends below 2^47 keep the sum below 2^54 and out of the
// flags and the count).  Integer addition is associative, so the total does not depend on the
// order in which the workgroups arrive: the result is deterministic.  The workgroup whose add
// returns count == k_splits-1 is the last one for that output: it holds the complete sum, writes
// y and puts the word back to zero for the next launch.
// A partial sum that is not finite cannot be expressed in fixed point.  Its workgroup first sets
// a flag in the same word (bit 54: +infinity seen, bit 55: -infinity seen, both: NaN) and then
// adds a zero contribution; the finishing workgroup turns the flags into the value IEEE
// arithmetic gives the sum: +-infinity, or NaN for a NaN or for infinities of both signs.  The
// flag store and the add are atomics of one thread on one address, so they take effect in
// program order.
constexpr unsigned long long kPosInfFlag = 1ull << 54, kNegInfFlag = 1ull << 55;
// The two halves of the completion, so that a wavefront that finishes several values per lane can
// issue all its atomics before it waits for the first answer.
struct Arrival {
    unsigned long long old, addend;
};

// First half: the split-k atomic (only with more than one k-split).  `valid` selects the lanes
// that deliver a value.
__device__ __forceinline__ Arrival arrive_output(float total, bool valid, unsigned long long *word)
{
    Arrival r{0ull, 0ull};
    if (!valid) return r;
    float scaled = total * 16777216.f;
    if (!(fabsf(scaled) < 7.0e13f)) {  // beyond 2^46 in fixed point, infinite or NaN
        const unsigned long long flags =
            total != total ? (kPosInfFlag | kNegInfFlag) : total > 0.f ? kPosInfFlag : kNegInfFlag;
        __hip_atomic_fetch_or(word, flags, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        scaled = 0.f;
    }
    r.addend = (unsigned long long)(__float2ll_rn(scaled) + (1ll << 46)) + (1ull << 56);
    r.old = __hip_atomic_fetch_add(word, r.addend, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return r;
}

// Second half: the lane whose add arrived last writes the output and clears the word.
// arrived_last only looks at the answer of the atomic; a wavefront that finishes several values per
// lane evaluates it for all of them before the first finish_last, so that no wait for an answer
// comes behind a store (the wait would then also wait for that store's round trip).
__device__ __forceinline__ bool arrived_last(const Arrival &r, bool valid, int k_splits)
{
    return valid && (r.old >> 56) == (unsigned long long)(k_splits - 1);
}

__device__ __forceinline__ void finish_last(const Arrival &r, unsigned long long *word, __half *yout, int k_splits)
{
    const unsigned long long all = r.old + r.addend;
    const long long value = (long long)(all & (kPosInfFlag - 1)) - (long long)k_splits * (1ll << 46);
    float result = __ll2float_rn(value) * (1.f / 16777216.f);
    const unsigned long long flags = all & (kPosInfFlag | kNegInfFlag);
    if (flags)
        result = flags == kPosInfFlag ? __builtin_inff() : flags == kNegInfFlag ? -__builtin_inff() : __builtin_nanf("");
    *yout = __float2half_rn(result);
    __hip_atomic_store(word, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void complete_output(const Arrival &r, bool valid, unsigned long long *word, __half *yout,
                                                int k_splits)
{
    if (arrived_last(r, valid, k_splits)) finish_last(r, word, yout, k_splits);
}

__device__ __forceinline__ void finish_output(float total, bool active, int out, int lane, __half *y,
                                              unsigned long long *accum, const MatvecArgs &a)
{
    const bool valid = active && (lane & 1) == 0 && out < a.n;
    if (a.k_splits == 1) {
        if (valid) y[(size_t)out * a.y_stride] = __float2half_rn(total);
        return;
    }
    const Arrival r = arrive_output(total, valid, accum + out);
    complete_output(r, valid, accum + out, y + (size_t)out * a.y_stride, a.k_splits);
}

}  // namespace lutgemm_kernels
#endif
