// Host-side helpers of the C ABI: bf16 conversion and the seeded input
// generators.  Counter-based (element i depends only on (seed, i)), integer
// exact and libm-free, so the same seed gives the same bits on any machine.
#include <cstring>

#include "maize_hip.h"

namespace {

inline uint64_t splitmix64(uint64_t x) {
    x ^= x >> 30; x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27; x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    return x;
}
inline uint64_t hash_at(uint64_t seed, uint64_t i) { return splitmix64(seed + i * 0x9E3779B97F4A7C15ull); }

// Round-to-nearest-even on the raw bits of a finite double whose magnitude is
// in bf16's normal range or zero (all the generators produce).
inline uint16_t bf16_from_f64_bits(double x) {
    // Via float is NOT allowed here (double rounding); do it on the f64 bits.
    uint64_t u;
    std::memcpy(&u, &x, sizeof u);
    const uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    const uint64_t mag = u & 0x7FFFFFFFFFFFFFFFull;
    if (mag == 0) return sign;
    const int e = (int)(mag >> 52) - 1023;            // unbiased exponent
    uint64_t frac = (mag & 0xFFFFFFFFFFFFFull) | (1ull << 52);  // 53-bit significand
    int shift = 52 - 7;                               // keep 8 significant bits
    int be = e + 127;                                 // biased bf16 exponent
    if (be <= 0) {                                    // subnormal in bf16
        shift += 1 - be;
        be = 0;
        if (shift > 62) return sign;                  // far below half the smallest subnormal
    }
    const uint64_t keep = frac >> shift;
    const uint64_t rem = frac & ((1ull << shift) - 1);
    const uint64_t half = 1ull << (shift - 1);
    uint64_t r = keep;
    if (rem > half || (rem == half && (keep & 1))) r += 1;
    // r carries the implicit bit for normals (bit 7); adding the exponent
    // field with carry handles both mantissa overflow and subnormal->normal.
    uint32_t bits = be == 0 ? (uint32_t)r : (uint32_t)(((uint32_t)(be - 1) << 7) + r);
    if (bits >= 0x7F80u) bits = 0x7F80u;              // overflow -> inf
    return (uint16_t)(sign | bits);
}

}  // namespace

extern "C" {

uint16_t maize_bf16_from_f32(float x) {
    uint32_t u;
    std::memcpy(&u, &x, sizeof u);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float maize_bf16_to_f32(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, sizeof f);
    return f;
}

// uniform on [-1, 1): v = (top 24 bits of the hash - 2^23) * 2^-23, exact in
// fp32, rounded once to bf16; an encoding of +1.0 is clamped to 0x3F7F.
void maize_fill_uniform_bf16(uint16_t* dst, size_t n, uint64_t seed, size_t first_index) {
    if (!dst) return;
    for (size_t i = 0; i < n; ++i) {
        const uint64_t h = hash_at(seed, (uint64_t)(first_index + i));
        const int32_t t = (int32_t)(h >> 40) - (1 << 23);
        const float v = (float)t * (1.0f / 8388608.0f);
        uint16_t e = maize_bf16_from_f32(v);
        if (e == 0x3F80u) e = 0x3F7Fu;
        dst[i] = e;
    }
}

// normal(0, sigma) by Irwin-Hall: twelve 16-bit uniforms (three hashes x four
// lanes) summed as integers, centred, scaled by sigma in fp64, one rounding.
void maize_fill_normal_bf16(uint16_t* dst, size_t n, uint64_t seed, double sigma, size_t first_index) {
    if (!dst) return;
    for (size_t i = 0; i < n; ++i) {
        const uint64_t idx = (uint64_t)(first_index + i);
        int64_t s = 0;
        for (uint64_t j = 0; j < 3; ++j) {
            const uint64_t h = hash_at(seed, idx * 3 + j);
            s += (int64_t)(h & 0xFFFF) + (int64_t)((h >> 16) & 0xFFFF) + (int64_t)((h >> 32) & 0xFFFF) +
                 (int64_t)((h >> 48) & 0xFFFF);
        }
        // sum of 12 U[0,1) minus 6, in units of 2^-16: exact in fp64.
        const double z = (double)(s - 6 * 65536) * (1.0 / 65536.0);
        dst[i] = bf16_from_f64_bits(z * sigma);
    }
}

}  // extern "C"
