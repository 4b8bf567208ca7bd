/* The input generator of the test hosts, in C so that the C++ program and (restated line for line in
 * tests/splitmix64.py) the Python tests draw the same values from the same seed: SplitMix64, a uniform float as
 * lo + (hi - lo) * (top 24 bits) / 2^24 evaluated in single precision in exactly this order, an integer of a closed
 * range as lo + value mod span.  FNV-1a (64 bit) is the checksum both hosts print to compare what they generated and
 * what the device gave back. */
#ifndef ASCQ_TESTS_SPLITMIX64_H
#define ASCQ_TESTS_SPLITMIX64_H

#include <stddef.h>
#include <stdint.h>

typedef struct splitmix64 {
    uint64_t s;
} splitmix64;

static inline uint64_t splitmix64_next(splitmix64* r)
{
    uint64_t z = (r->s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

static inline float splitmix64_uniform(splitmix64* r, float lo, float hi)
{
    const float u = (float)(splitmix64_next(r) >> 40);
    const float span = hi - lo;
    const float scaled = span * u;
    const float frac = scaled / 16777216.0f;
    return lo + frac;
}

static inline int splitmix64_integer(splitmix64* r, int lo, int hi)
{
    return lo + (int)(splitmix64_next(r) % (uint64_t)(hi - lo + 1));
}

static inline uint64_t fnv1a64(const void* data, size_t bytes)
{
    const unsigned char* p = (const unsigned char*)data;
    uint64_t h = 0xCBF29CE484222325ull;
    for (size_t i = 0; i < bytes; ++i) {
        h = (h ^ p[i]) * 0x100000001B3ull;
    }
    return h;
}

#endif
