// rng.h -- the deterministic host generator that seeds every synthetic input.
// Replaces the cuRAND XORWOW fills of the reference (curandGenerateUniform with
// seed 1337, src/ori_kernel/stencil_kernel.cu:155-159, lbm_kernel.cu:206-210,
// src/include/dnn.h:737-741): splitmix64 expands the seed into a xoshiro256**
// state; floats are the top 24 bits, so [0,1) with 2^-24 spacing.
#pragma once
#include <cstdint>

namespace tk {

class Rng {
public:
    explicit Rng(uint64_t seed = 1337ULL)
    {
        uint64_t z = seed;
        for (int i = 0; i < 4; ++i) {
            z += 0x9e3779b97f4a7c15ULL;
            uint64_t x = z;
            x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ULL;
            x = (x ^ (x >> 27)) * 0x94d049bb133111ebULL;
            s_[i] = x ^ (x >> 31);
        }
    }
    uint64_t next()
    {
        const uint64_t result = rotl(s_[1] * 5, 7) * 9;
        const uint64_t t = s_[1] << 17;
        s_[2] ^= s_[0];
        s_[3] ^= s_[1];
        s_[1] ^= s_[2];
        s_[0] ^= s_[3];
        s_[2] ^= t;
        s_[3] = rotl(s_[3], 45);
        return result;
    }
    // uniform in [0,1)
    float uniform() { return (float)(next() >> 40) * (1.0f / 16777216.0f); }
    float uniform(float lo, float hi) { return lo + (hi - lo) * uniform(); }

private:
    static uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
    uint64_t s_[4];
};

// round-to-nearest-even float -> IEEE half bits (host side; inputs are finite)
inline uint16_t float_to_half_bits(float f)
{
    uint32_t x;
    __builtin_memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x47800000u) return (uint16_t)(sign | (x > 0x7f800000u ? 0x7e00u : 0x7c00u));
    if (x < 0x38800000u) {   // subnormal half or zero
        if (x < 0x33000000u) return (uint16_t)sign;
        const int shift = 113 - (int)(x >> 23);
        uint32_t man = (x & 0x7fffffu) | 0x800000u;
        const uint32_t round_bit = 1u << (shift + 12);
        uint32_t h = man >> (shift + 13);
        const uint32_t rem = man & ((round_bit << 1) - 1);
        if (rem > round_bit || (rem == round_bit && (h & 1))) h++;
        return (uint16_t)(sign | h);
    }
    uint32_t h = ((x - 0x38000000u) >> 13);
    const uint32_t rem = x & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1))) h++;
    return (uint16_t)(sign | h);
}

}  // namespace tk
