// Host-side weight packer: re-tiles the reference's input layout
//   bW uint32 [k/32][q][n], alpha fp16 [G][q][n], q_bias fp16 [G][n]
// (the layout nQWeight_fp16::parsing receives, lutGEMM/src/nQWeight_fp16.cu:60-91, with the
// bit convention of tests/opt/fp16/int3_col_wise_matmul_fp16.cu:200-215) into the wave64
// tiles described in layout.h, and back.  Pure host code, no HIP calls.
#include "packer.h"

#include <algorithm>
#include <cstring>
#include <thread>
#include <vector>

namespace lutgemm_packer {
using namespace lutgemm_layout;

namespace {

template <typename F>
void parallel_for(int count, F body)
{
    unsigned hw = std::thread::hardware_concurrency();
    int workers = (int)std::min<unsigned>(hw ? hw : 1u, 16u);
    workers = std::min(workers, count);
    if (workers <= 1) {
        for (int i = 0; i < count; i++) body(i);
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(workers);
    for (int w = 0; w < workers; w++)
        pool.emplace_back([=]() {
            for (int i = w; i < count; i += workers) body(i);
        });
    for (auto &t : pool) t.join();
}

// scale group of lane `lane` in k-block `ts`, or -1 when the lane's k range is padding
inline int lane_group(const Shape &s, int ts, int lane)
{
    int r = lane / 16, j = lane % 16;
    int subl = 16 / s.gsub;
    int kpos = ts * kBlockK + r * 128 + (j / subl) * (128 / s.gsub);
    return kpos < s.k ? kpos / s.group_size : -1;
}

}  // namespace

void pack(const Shape &s, const uint32_t *bW, const uint16_t *alpha, const uint16_t *q_bias,
          uint8_t *signs, uint16_t *scales)
{
    const size_t n = (size_t)s.n;
    const int chunks = s.k / kChunk;
    const int subl = 16 / s.gsub, nt = 2 * s.gsub, lh = scale_lane_halves(s);
    parallel_for(s.nb, [&](int nb) {
        for (int ts = 0; ts < s.ts; ts++) {
            uint8_t *tile = signs + ((size_t)nb * s.ts + ts) * sign_tile_bytes(s);
            for (int b = 0; b < s.q; b++)
                for (int h = 0; h < 2; h++) {
                    uint8_t *unit = tile + (size_t)(2 * b + h) * kUnitBytes;
                    int n0 = nb * kBatch + h * 16;
                    int valid = std::max(0, std::min(16, s.n - n0));
                    for (int lane = 0; lane < kLanes; lane++) {
                        uint8_t *dst = unit + lane * 16;
                        int c = ts * kLanes + lane;
                        if (c >= chunks || valid == 0) {
                            std::memset(dst, 0, 16);
                            continue;
                        }
                        const uint32_t *src = bW + ((size_t)(c / 4) * s.q + b) * n + n0;
                        int sh = 8 * (c % 4);
                        for (int p = 0; p < valid; p++) dst[p] = (uint8_t)(src[p] >> sh);
                        for (int p = valid; p < 16; p++) dst[p] = 0;
                    }
                }
            uint16_t *st = scales + ((size_t)nb * s.ts + ts) * (size_t)kLanes * lh;
            for (int lane = 0; lane < kLanes; lane++) {
                int g = lane_group(s, ts, lane);
                int jj = (lane % 16) % subl;
                for (int t = 0; t < nt; t++) {
                    int out = nb * kBatch + t * subl + jj;
                    for (int bo = 0; bo < s.qo; bo++) {
                        uint16_t v = 0;
                        if (g >= 0 && out < s.n) {
                            if (bo < s.q)
                                v = alpha[((size_t)g * s.q + bo) * n + out];
                            else
                                v = q_bias[(size_t)g * n + out];
                        }
                        st[(size_t)lane * lh + t * s.qo + bo] = v;
                    }
                }
            }
        }
    });
}

void unpack(const Shape &s, const uint8_t *signs, const uint16_t *scales, uint32_t *bW,
            uint16_t *alpha, uint16_t *q_bias)
{
    const size_t n = (size_t)s.n;
    const int chunks = s.k / kChunk;
    const int subl = 16 / s.gsub, nt = 2 * s.gsub, lh = scale_lane_halves(s);
    if (bW) std::memset(bW, 0, sizeof(uint32_t) * (size_t)(s.k / 32) * s.q * n);
    // Different batches touch disjoint output columns, so the loop is race free.
    parallel_for(s.nb, [&](int nb) {
        for (int ts = 0; ts < s.ts; ts++) {
            if (bW) {
                const uint8_t *tile = signs + ((size_t)nb * s.ts + ts) * sign_tile_bytes(s);
                for (int b = 0; b < s.q; b++)
                    for (int h = 0; h < 2; h++) {
                        const uint8_t *unit = tile + (size_t)(2 * b + h) * kUnitBytes;
                        int n0 = nb * kBatch + h * 16;
                        int valid = std::max(0, std::min(16, s.n - n0));
                        for (int lane = 0; lane < kLanes; lane++) {
                            int c = ts * kLanes + lane;
                            if (c >= chunks) continue;
                            uint32_t *dst = bW + ((size_t)(c / 4) * s.q + b) * n + n0;
                            int sh = 8 * (c % 4);
                            for (int p = 0; p < valid; p++)
                                dst[p] |= (uint32_t)unit[lane * 16 + p] << sh;
                        }
                    }
            }
            if (alpha || q_bias) {
                const uint16_t *st = scales + ((size_t)nb * s.ts + ts) * (size_t)kLanes * lh;
                for (int lane = 0; lane < kLanes; lane++) {
                    int g = lane_group(s, ts, lane);
                    if (g < 0) continue;
                    int jj = (lane % 16) % subl;
                    for (int t = 0; t < nt; t++) {
                        int out = nb * kBatch + t * subl + jj;
                        if (out >= s.n) continue;
                        for (int bo = 0; bo < s.qo; bo++) {
                            uint16_t v = st[(size_t)lane * lh + t * s.qo + bo];
                            if (bo < s.q) {
                                if (alpha) alpha[((size_t)g * s.q + bo) * n + out] = v;
                            } else if (q_bias) {
                                q_bias[(size_t)g * n + out] = v;
                            }
                        }
                    }
                }
            }
        }
    });
}

// IEEE binary32 -> binary16, round to nearest even (what __float2half does in the reference's
// ingest loop, lutGEMM/src/nQWeight_fp16.cu:81,85).
uint16_t float_to_half(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    x &= 0x7fffffffu;
    if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (x < 0x38800000u) {
        if (x < 0x33000000u) return sign;
        uint32_t shift = 126u - (x >> 23);
        uint32_t m = (x & 0x7fffffu) | 0x800000u;
        uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t h = (((x >> 23) - 112u) << 10) | ((x & 0x7fffffu) >> 13);
    uint32_t rem = x & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

void floats_to_halves(const float *src, uint16_t *dst, size_t count)
{
    const size_t block = 1 << 16;
    int blocks = (int)((count + block - 1) / block);
    parallel_for(blocks, [&](int bi) {
        size_t lo = (size_t)bi * block, hi = std::min(count, lo + block);
        for (size_t i = lo; i < hi; i++) dst[i] = float_to_half(src[i]);
    });
}

}  // namespace lutgemm_packer
