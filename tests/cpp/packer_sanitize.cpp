// Host-only memory-safety check of the packer (lut-gemm_amd/csrc/packer.cpp): built with
// -fsanitize=address,undefined by tests/test_sanitizers.py.  For ragged shapes (k that ends inside a
// k-block, n that ends inside a batch, one to eight planes, one, two and four scale groups per
// 128 k, with and without offset) it packs random input arrays into buffers of exactly the sizes
// layout.h states, unpacks them again and compares bit for bit; any access outside a buffer, any
// misaligned or overflowing index computation aborts the run.  The input layout is the one
// nQWeight_fp16::parsing receives (lutGEMM/src/nQWeight_fp16.cu:60-91).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>

#include "../../lut-gemm_amd/csrc/packer.h"

using namespace lutgemm_layout;

static uint64_t state = 0x9e3779b97f4a7c15ull;
static uint32_t rnd()
{
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    return (uint32_t)(state >> 16);
}

int main()
{
    struct Case { int k, n, q, groups, off; };
    const Case cases[] = {
        {32, 1, 1, 1, 0},     {64, 8, 3, 2, 1},      {96, 33, 4, 1, 1},    {512, 32, 2, 4, 0},   {544, 31, 8, 17, 1},
        {1024, 100, 5, 8, 0}, {1536, 65, 7, 48, 1},  {2048, 40, 3, 1, 1},  {640, 70, 6, 5, 0},   {4096, 97, 2, 64, 1},
        {1152, 513, 1, 6, 1}, {7168, 224, 3, 56, 0}, {12288, 64, 4, 384, 1},
    };
    int checked = 0;
    for (const Case &c : cases) {
        Shape s;
        if (!make_shape(c.k, c.n, c.q, c.groups, c.off, &s)) {
            std::fprintf(stderr, "shape k=%d n=%d q=%d groups=%d refused\n", c.k, c.n, c.q, c.groups);
            return 1;
        }
        const size_t words = (size_t)(c.k / 32) * c.q * c.n, na = (size_t)c.groups * c.q * c.n, nz = (size_t)c.groups * c.n;
        // heap arrays of exactly the stated sizes: the sanitizer's red zones sit right behind them
        std::unique_ptr<uint32_t[]> bW(new uint32_t[words]), bW2(new uint32_t[words]);
        std::unique_ptr<uint16_t[]> alpha(new uint16_t[na]), alpha2(new uint16_t[na]);
        std::unique_ptr<uint16_t[]> z(new uint16_t[nz]), z2(new uint16_t[nz]);
        for (size_t i = 0; i < words; i++) bW[i] = rnd();
        for (size_t i = 0; i < na; i++) alpha[i] = (uint16_t)rnd();
        for (size_t i = 0; i < nz; i++) z[i] = (uint16_t)rnd();
        std::unique_ptr<uint8_t[]> signs(new uint8_t[sign_bytes(s)]);
        std::unique_ptr<uint16_t[]> scales(new uint16_t[scale_bytes(s) / 2]);
        lutgemm_packer::pack(s, bW.get(), alpha.get(), c.off ? z.get() : nullptr, signs.get(), scales.get());
        lutgemm_packer::unpack(s, signs.get(), scales.get(), bW2.get(), alpha2.get(), c.off ? z2.get() : nullptr);
        if (std::memcmp(bW.get(), bW2.get(), words * 4) != 0 || std::memcmp(alpha.get(), alpha2.get(), na * 2) != 0 ||
            (c.off && std::memcmp(z.get(), z2.get(), nz * 2) != 0)) {
            std::fprintf(stderr, "round trip differs for k=%d n=%d q=%d groups=%d off=%d\n", c.k, c.n, c.q, c.groups, c.off);
            return 1;
        }
        // partial outputs are allowed
        lutgemm_packer::unpack(s, signs.get(), scales.get(), nullptr, alpha2.get(), nullptr);
        lutgemm_packer::unpack(s, signs.get(), scales.get(), bW2.get(), nullptr, nullptr);
        checked++;
    }
    // the ingest conversion: every float bit pattern class, array form against the scalar form
    const float specials[] = {0.f, -0.f, 1.f, 65504.f, 65520.f, 1e-8f, 5.96e-8f, 6.1e-5f, -3.14159f, 1e30f, -1e30f};
    uint16_t out[sizeof(specials) / sizeof(specials[0])];
    lutgemm_packer::floats_to_halves(specials, out, sizeof(specials) / sizeof(specials[0]));
    for (size_t i = 0; i < sizeof(specials) / sizeof(specials[0]); i++)
        if (out[i] != lutgemm_packer::float_to_half(specials[i])) {
            std::fprintf(stderr, "floats_to_halves differs from float_to_half at %zu\n", i);
            return 1;
        }
    std::printf("packer under sanitizers: %d shapes ok\n", checked);
    return 0;
}
