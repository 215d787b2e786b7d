// zyx's host-side random number generator (zyx/src/rng.rs) and the tensor initialisers built on it
// (Tensor::rand / uniform / randn / randint, zyx/src/tensor/mod.rs:516-660), so that callers of this backend can
// produce the same seeded inputs the reference produces. Pure host code: no device, no context.
#include "../../include/zyx_hip.h"

#include <cmath>
#include <vector>

#define ZHIP_EXPORT extern "C" __attribute__((visibility("default")))

namespace {

inline uint64_t rotl(uint64_t v, unsigned k) { return (v << k) | (v >> (64u - k)); }

// xoshiro256++ step (rng.rs:65-80)
inline uint64_t step(uint64_t (&s)[4]) {
    const uint64_t out = rotl(s[0] + s[3], 23) + s[0];
    const uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl(s[3], 45);
    return out;
}

// next_f32 (rng.rs:98-110): one LCG step on the low 32 bits of a draw, reduced modulo 2^32 - 1 and divided by
// (f32)(2^32 - 1), which is 2^32 after rounding -- the quotient rounds to exactly 1.0 for the top 128 values.
inline float unit_f32(uint64_t (&s)[4]) {
    const uint32_t lo = (uint32_t)step(s);
    const uint32_t v = (lo * 1664525u + 1013904223u) % 4294967295u;
    return (float)v / 4294967296.0f;
}

} // namespace

ZHIP_EXPORT void zhip_rng_seed(zhip_rng *rng, uint64_t seed) {
    // four rounds of splitmix64 (rng.rs:15-57)
    for (uint64_t &word : rng->s) {
        seed += 0x9e3779b97f4a7c15ull;
        uint64_t z = seed;
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        word = z ^ (z >> 31);
    }
}

ZHIP_EXPORT uint64_t zhip_rng_next_u64(zhip_rng *rng) { return step(rng->s); }

ZHIP_EXPORT int32_t zhip_rng_fill(zhip_rng *rng, int32_t kind, int32_t dtype, void *out, uint64_t n, double lo, double hi) {
    if (!rng || (!out && n)) return ZHIP_INCORRECT_KERNEL_ARG;
    uint64_t(&s)[4] = rng->s;
    switch (kind) {
    case ZHIP_RNG_RAND: // Rng::rand<T> (rng.rs:127-141): every element consumes one 64-bit draw, integers keep its low bytes
        switch (dtype) {
        case ZHIP_F32: for (uint64_t i = 0; i < n; i++) ((float *)out)[i] = unit_f32(s); return ZHIP_OK;
        case ZHIP_U8: case ZHIP_I8: for (uint64_t i = 0; i < n; i++) ((uint8_t *)out)[i] = (uint8_t)step(s); return ZHIP_OK;
        case ZHIP_U16: case ZHIP_I16: for (uint64_t i = 0; i < n; i++) ((uint16_t *)out)[i] = (uint16_t)step(s); return ZHIP_OK;
        case ZHIP_U32: case ZHIP_I32: for (uint64_t i = 0; i < n; i++) ((uint32_t *)out)[i] = (uint32_t)step(s); return ZHIP_OK;
        case ZHIP_U64: case ZHIP_I64: for (uint64_t i = 0; i < n; i++) ((uint64_t *)out)[i] = step(s); return ZHIP_OK;
        default: return ZHIP_INCORRECT_KERNEL_ARG;
        }
    case ZHIP_RNG_UNIFORM: { // Tensor::uniform (tensor/mod.rs:637-648): rand * (high - low) + low in f32
        if (dtype != ZHIP_F32) return ZHIP_INCORRECT_KERNEL_ARG;
        const float low = (float)lo, span = (float)hi - (float)lo;
        for (uint64_t i = 0; i < n; i++) {
            const float p = unit_f32(s) * span; // two roundings, as two tensor ops give
            ((float *)out)[i] = p + low;
        }
        return ZHIP_OK;
    }
    case ZHIP_RNG_RANDN: { // Tensor::randn (tensor/mod.rs:603-613): Box-Muller over one rand([2, n]) draw, times `hi`
        if (dtype != ZHIP_F32) return ZHIP_INCORRECT_KERNEL_ARG;
        std::vector<float> first(n);
        for (uint64_t i = 0; i < n; i++) first[i] = unit_f32(s);
        const float two_pi = 2.0f * 3.14159265358979323846f, scale = hi == 0.0 ? 1.0f : (float)hi;
        for (uint64_t i = 0; i < n; i++) {
            float u = unit_f32(s);
            if (u >= 1.0f) u = 0.99999994f; // ln(1 - 1) would be -inf: the draw that rounds to 1 becomes the float below it
            const float c = cosf(first[i] * two_pi);
            const float r = sqrtf(logf(1.0f - u) * -2.0f);
            ((float *)out)[i] = c * r * scale;
        }
        return ZHIP_OK;
    }
    case ZHIP_RNG_RANDINT: { // Rng::range for signed integers (rng.rs:186-208): next_u64 % (high - low) + low, [low, high)
        int64_t a = (int64_t)lo, b = (int64_t)hi;
        if (b < a) { int64_t t = a; a = b; b = t; }
        const uint64_t width = (uint64_t)(b - a);
        if (dtype != ZHIP_I32 && dtype != ZHIP_I64) return ZHIP_INCORRECT_KERNEL_ARG;
        for (uint64_t i = 0; i < n; i++) {
            const int64_t v = width ? (int64_t)(step(s) % width) + a : a; // an empty range draws nothing
            if (dtype == ZHIP_I32) ((int32_t *)out)[i] = (int32_t)v;
            else ((int64_t *)out)[i] = v;
        }
        return ZHIP_OK;
    }
    default: return ZHIP_INCORRECT_KERNEL_ARG;
    }
}
