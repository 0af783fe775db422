// Host packer interface (see packer.cpp and layout.h).
#ifndef LUTGEMM_PACKER_H
#define LUTGEMM_PACKER_H

#include "layout.h"

namespace lutgemm_packer {

// Re-tile host input arrays into sign tiles (sign_bytes(s) bytes) and scale tiles
// (scale_bytes(s) bytes).  q_bias may be null iff s.has_offset == 0.
void pack(const lutgemm_layout::Shape &s, const uint32_t *bW, const uint16_t *alpha,
          const uint16_t *q_bias, uint8_t *signs, uint16_t *scales);

// Exact inverse of pack(); any output may be null.
void unpack(const lutgemm_layout::Shape &s, const uint8_t *signs, const uint16_t *scales,
            uint32_t *bW, uint16_t *alpha, uint16_t *q_bias);

uint16_t float_to_half(float f);
void floats_to_halves(const float *src, uint16_t *dst, size_t count);

}  // namespace lutgemm_packer
#endif
