// Device-side numeric primitives for gfx950.  Every operation rounds exactly once in the stated format; the
// translation units are compiled with -ffp-contract=off so that a multiply and an add are never fused.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/ascq.h"

namespace ascq {

typedef _Float16 half_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x2_t __attribute__((ext_vector_type(2)));
typedef int32_t i32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// fp32 -> bfloat16 bits, round to nearest even (v_cvt_pk_bf16_f32 on gfx950; NaN stays NaN).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f)
{
    return __builtin_bit_cast(unsigned short, static_cast<__bf16>(f));
}

__device__ __forceinline__ float half_bits_to_f32(uint32_t h)
{
    union {
        uint16_t u;
        half_t h;
    } c;
    c.u = static_cast<uint16_t>(h);
    return static_cast<float>(c.h);
}

__device__ __forceinline__ uint32_t f32_to_half_bits(float f)
{
    union {
        uint16_t u;
        half_t h;
    } c;
    // The empty asm makes `f` opaque: without it the compiler folds a preceding fp32 multiply into one
    // mixed-precision instruction that rounds the exact product once to fp16, whereas the operators round to fp32
    // first and to fp16 second.
    asm volatile("" : "+v"(f));
    c.h = static_cast<half_t>(f);  // v_cvt_f16_f32: round to nearest even, overflow to infinity
    return c.u;
}

// fp32 -> fp16 bits with the fixpipe's saturation to +-65504 (NaN passes through).
__device__ __forceinline__ uint32_t f32_to_half_bits_sat(float f)
{
    float c = fminf(fmaxf(f, -65504.0f), 65504.0f);
    return f32_to_half_bits((f != f) ? f : c);
}

// fp32 -> hifloat8, RoundMode::CAST_ROUND (nearest on the grid of the value's own exponent, ties away from zero; a
// mantissa that rounds up past all-ones carries into the exponent), saturating: NaN -> 0, magnitudes from 1.25 * 2^15
// on (infinity included) -> the largest finite code 0x6E, below 1.5 * 2^-23 -> 0 without sign.  Mantissa bits: 3 for
// |e| <= 3, 2 for |e| <= 7, 1 up to 15, none for the powers of two 2^-22 .. 2^-16 (codes 1..7).
__device__ __forceinline__ uint32_t f32_to_hif8_sat(float f)
{
    const uint32_t u = __float_as_uint(f), au = u & 0x7FFFFFFFu, sign = (u >> 24) & 0x80u;
    if (au > 0x7F800000u) {
        return 0u;
    }
    if (au >= 0x47200000u) {  // 1.25 * 2^15
        return sign | 0x6Eu;
    }
    int e = static_cast<int>(au >> 23) - 127;
    if (e < -23) {
        return 0u;
    }
    const int ae0 = e < 0 ? -e : e;
    const int mbits = e < -15 ? 0 : ae0 <= 3 ? 3 : ae0 <= 7 ? 2 : 1;
    const uint32_t tmp = (au & 0x7FFFFFu) >> (22 - mbits);  // the mantissa and one more bit
    uint32_t mant = (tmp + 1u) >> 1;
    if (tmp == (2u << mbits) - 1u) {
        mant = 0u;
        e += 1;
    }
    if (e < -22) {
        return 0u;
    }
    const uint32_t ae = static_cast<uint32_t>(e < 0 ? -e : e), neg = e < 0 ? 1u : 0u;
    uint32_t code;
    if (e < -15) {
        code = static_cast<uint32_t>(e + 23);
    } else if (ae == 0u) {
        code = 0x08u | mant;
    } else if (ae == 1u) {
        code = 0x10u | (neg << 3) | mant;
    } else if (ae <= 3u) {
        code = 0x20u | (neg << 4) | ((ae - 2u) << 3) | mant;
    } else if (ae <= 7u) {
        // a carry from exponent 3 (three mantissa bits) arrives with mant = 0, as does one from -8
        code = 0x40u | (neg << 4) | ((ae - 4u) << 2) | mant;
    } else {
        code = 0x60u | (neg << 4) | ((ae - 8u) << 1) | mant;
    }
    return sign | code;
}

// hifloat8 -> fp32 (exact): 0x80 is NaN, 0x6F / 0xEF the infinities.
__device__ __forceinline__ float hif8_to_f32(uint32_t code)
{
    const uint32_t c = code & 0x7Fu;
    if (c == 0u) {
        return (code & 0x80u) ? __uint_as_float(0x7FC00000u) : 0.0f;
    }
    int e;
    uint32_t mant23;  // the mantissa, left-aligned in the 23 fraction bits of a float
    if (c < 8u) {
        e = static_cast<int>(c) - 23, mant23 = 0u;
    } else if (c < 16u) {
        e = 0, mant23 = (c & 7u) << 20;
    } else if (c < 32u) {
        e = (c & 8u) ? -1 : 1, mant23 = (c & 7u) << 20;
    } else if (c < 64u) {
        const int f = static_cast<int>((c >> 3) & 3u);
        e = f >= 2 ? -f : f + 2, mant23 = (c & 7u) << 20;
    } else if (c < 96u) {
        const int f = static_cast<int>((c >> 2) & 7u);
        e = f >= 4 ? -f : f + 4, mant23 = (c & 3u) << 21;
    } else {
        const int f = static_cast<int>((c >> 1) & 15u);
        e = f >= 8 ? -f : f + 8, mant23 = (c & 1u) << 22;
    }
    uint32_t bits = (static_cast<uint32_t>(e + 127) << 23) | mant23;
    if (c == 0x6Fu) {
        bits = 0x7F800000u;
    }
    return __uint_as_float(bits | ((code & 0x80u) << 24));
}

// Round a value (already exact in fp32) to an integer with the given mode and saturate to int8.
template <bool kRint>
__device__ __forceinline__ int round_sat8(float v, int round_mode)
{
    float r;
    if (kRint) {
        r = __builtin_rintf(v);
    } else {
        switch (round_mode) {
            case ASCQ_CAST_FLOOR: r = __builtin_floorf(v); break;
            case ASCQ_CAST_CEIL: r = __builtin_ceilf(v); break;
            case ASCQ_CAST_ROUND: r = __builtin_roundf(v); break;
            case ASCQ_CAST_TRUNC: r = __builtin_truncf(v); break;
            default: r = __builtin_rintf(v); break;
        }
    }
    r = fminf(fmaxf(r, -128.0f), 127.0f);
    return (v != v) ? 0 : static_cast<int>(r);
}

// ---- arithmetic in a given compute format on values carried as fp32 (each op rounds once in the format) ----
template <int kFmt>
struct Fmt;

template <>
struct Fmt<ASCQ_F32> {
    static __device__ __forceinline__ float cvt(float x) { return x; }
    static __device__ __forceinline__ float mul(float a, float b) { return a * b; }
    static __device__ __forceinline__ float add(float a, float b) { return a + b; }
};
template <>
struct Fmt<ASCQ_F16> {
    static __device__ __forceinline__ float cvt(float x) { return static_cast<float>(static_cast<half_t>(x)); }
    static __device__ __forceinline__ float mul(float a, float b)
    {
        return static_cast<float>(static_cast<half_t>(a) * static_cast<half_t>(b));
    }
    static __device__ __forceinline__ float add(float a, float b)
    {
        return static_cast<float>(static_cast<half_t>(a) + static_cast<half_t>(b));
    }
};
template <>
struct Fmt<ASCQ_BF16> {
    static __device__ __forceinline__ float cvt(float x) { return bf16_bits_to_f32(f32_to_bf16_bits(x)); }
    // 8-bit significands: the fp32 product is exact, the fp32 sum is rounded to 24 >= 2*8+2 bits, so rounding
    // the fp32 result to bfloat16 equals rounding the exact result once.
    static __device__ __forceinline__ float mul(float a, float b) { return cvt(a * b); }
    static __device__ __forceinline__ float add(float a, float b) { return cvt(a + b); }
};

// ---- typed element access (values widened to fp32, which is exact for every source type) ----
template <int kDt>
struct Elem;
template <>
struct Elem<ASCQ_F16> {
    typedef uint16_t type;
    static __device__ __forceinline__ float to_f32(uint16_t v) { return half_bits_to_f32(v); }
};
template <>
struct Elem<ASCQ_BF16> {
    typedef uint16_t type;
    static __device__ __forceinline__ float to_f32(uint16_t v) { return bf16_bits_to_f32(v); }
};
template <>
struct Elem<ASCQ_F32> {
    typedef float type;
    static __device__ __forceinline__ float to_f32(float v) { return v; }
};
template <>
struct Elem<ASCQ_U64> {
    typedef uint64_t type;
    static __device__ __forceinline__ float to_f32(uint64_t v) { return __uint_as_float(static_cast<uint32_t>(v)); }
};
template <>
struct Elem<ASCQ_I32> {
    typedef int32_t type;
    static __device__ __forceinline__ float to_f32(int32_t v) { return static_cast<float>(v); }  // RNE
};

// 16-byte load / store with or without the non-temporal cache policy (data that is touched once per call).
template <bool kNT>
__device__ __forceinline__ u32x4 ld16(const void* p)
{
    if constexpr (kNT) {
        return __builtin_nontemporal_load(static_cast<const u32x4*>(p));
    } else {
        return *static_cast<const u32x4*>(p);
    }
}
template <bool kNT, class V>
__device__ __forceinline__ void st16(void* p, V v)
{
    if constexpr (kNT) {
        __builtin_nontemporal_store(v, static_cast<V*>(p));
    } else {
        *static_cast<V*>(p) = v;
    }
}

// Load 8 consecutive elements (16-byte aligned group for 2-byte types) widened to fp32.
template <int kDt, bool kNT = false>
__device__ __forceinline__ void load8(const void* base, size_t idx, float (&out)[8])
{
    typedef typename Elem<kDt>::type T;
    const T* p = static_cast<const T*>(base) + idx;
    if constexpr (sizeof(T) == 2) {
        u32x4 v = ld16<kNT>(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            out[2 * i] = Elem<kDt>::to_f32(static_cast<uint16_t>(v[i] & 0xFFFFu));
            out[2 * i + 1] = Elem<kDt>::to_f32(static_cast<uint16_t>(v[i] >> 16));
        }
    } else if constexpr (sizeof(T) == 4) {
        u32x4 a = ld16<kNT>(reinterpret_cast<const u32x4*>(p));
        u32x4 b = ld16<kNT>(reinterpret_cast<const u32x4*>(p) + 1);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t ua = a[i], ub = b[i];
            T ta, tb;
            __builtin_memcpy(&ta, &ua, 4);
            __builtin_memcpy(&tb, &ub, 4);
            out[i] = Elem<kDt>::to_f32(ta);
            out[4 + i] = Elem<kDt>::to_f32(tb);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x4 v = reinterpret_cast<const u32x4*>(p)[i];
            out[2 * i] = __uint_as_float(v[0]);
            out[2 * i + 1] = __uint_as_float(v[2]);
        }
    }
}

template <int kDt>
__device__ __forceinline__ float load1(const void* base, size_t idx)
{
    typedef typename Elem<kDt>::type T;
    return Elem<kDt>::to_f32(static_cast<const T*>(base)[idx]);
}

// Store 8 fp32 values as the destination type (rounded once).
template <int kDt, bool kNT = false>
__device__ __forceinline__ void store8(void* base, size_t idx, const float (&v)[8])
{
    if constexpr (kDt == ASCQ_F32) {
        f32x4* p = reinterpret_cast<f32x4*>(static_cast<float*>(base) + idx);
        st16<kNT>(p, f32x4{v[0], v[1], v[2], v[3]});
        st16<kNT>(p + 1, f32x4{v[4], v[5], v[6], v[7]});
    } else {
        u32x4 o;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint32_t lo, hi;
            if constexpr (kDt == ASCQ_BF16) {
                lo = f32_to_bf16_bits(v[2 * i]);
                hi = f32_to_bf16_bits(v[2 * i + 1]);
            } else {
                lo = f32_to_half_bits(v[2 * i]);
                hi = f32_to_half_bits(v[2 * i + 1]);
            }
            o[i] = lo | (hi << 16);
        }
        st16<kNT>(static_cast<uint16_t*>(base) + idx, o);
    }
}

template <int kDt>
__device__ __forceinline__ void store1(void* base, size_t idx, float v)
{
    if constexpr (kDt == ASCQ_F32) {
        static_cast<float*>(base)[idx] = v;
    } else if constexpr (kDt == ASCQ_BF16) {
        static_cast<uint16_t*>(base)[idx] = static_cast<uint16_t>(f32_to_bf16_bits(v));
    } else {
        static_cast<uint16_t*>(base)[idx] = static_cast<uint16_t>(f32_to_half_bits(v));
    }
}

// fp32 -> OCP 8-bit floats, round-half-even, saturating to the largest finite value; NaN -> +0.
// kE5M2 false: e4m3fn (bias 7, max 448 = 0x7E); true: e5m2 (bias 15, max 57344 = 0x7B).
template <bool kE5M2>
__device__ __forceinline__ int f32_to_fp8_sat(float f)
{
    constexpr int kMant = kE5M2 ? 2 : 3;
    constexpr int kBias = kE5M2 ? 15 : 7;
    constexpr int kShift = 23 - kMant;
    constexpr uint32_t kMaxBits = kE5M2 ? 0x47600000u : 0x43E00000u;      // 57344.0f / 448.0f
    constexpr uint32_t kMinNormalBits = static_cast<uint32_t>(127 - kBias + 1) << 23;
    uint32_t u;
    __builtin_memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 24) & 0x80u;
    const uint32_t a = u & 0x7FFFFFFFu;
    uint32_t code;
    if (a > 0x7F800000u) {
        return 0;  // NaN -> +0: what the reference's saturating casts give
    } else if (a >= kMaxBits) {
        code = kE5M2 ? 0x7Bu : 0x7Eu;  // everything from the largest finite value up, infinity included
    } else if (a >= kMinNormalBits) {
        const uint32_t r = a + ((1u << (kShift - 1)) - 1u) + ((a >> kShift) & 1u);  // ties to even
        code = (r >> kShift) - (static_cast<uint32_t>(127 - kBias) << kMant);
    } else {
        // subnormal range: a multiple of the smallest subnormal, 2^(1 - bias - mant); 2^mant is the smallest normal
        float mag;
        __builtin_memcpy(&mag, &a, 4);
        code = static_cast<uint32_t>(__builtin_rintf(mag * (kE5M2 ? 65536.0f : 512.0f)));
    }
    return static_cast<int>(sign | code);
}

// A value already rounded to bfloat16 -> 4-bit float code (sign, then e2m1 or e1m2, both bias 1), rounded with the
// given mode, saturating to the largest magnitude (6 / 1.75); NaN -> +0.  The grid is uniform inside each of the
// ranges used below, so the value is scaled to integers, rounded as a signed number (which makes FLOOR and CEIL right
// for negative inputs, and half-even on the scaled integer is half-even on the code), and scaled back.
template <bool kE1M2>
__device__ __forceinline__ uint32_t f32_to_fp4_sat(float v, int round_mode)
{
    if (v != v) {
        return 0u;
    }
    const uint32_t sign = (__float_as_uint(v) >> 28) & 8u;
    const float a = fminf(fabsf(v), 8.0f);  // everything from 8 up saturates like 8 (and infinity becomes finite)
    float unit;                             // spacing of the grid around |v|
    if (kE1M2) {
        unit = 0.25f;
    } else {
        unit = a < 2.0f ? 0.5f : (a < 4.0f ? 1.0f : 2.0f);
    }
    const float t = (sign ? -a : a) / unit;  // exact: a power-of-two divisor
    float r;
    switch (round_mode) {
        case ASCQ_CAST_FLOOR: r = __builtin_floorf(t); break;
        case ASCQ_CAST_CEIL: r = __builtin_ceilf(t); break;
        case ASCQ_CAST_ROUND: r = __builtin_roundf(t); break;
        case ASCQ_CAST_TRUNC: r = __builtin_truncf(t); break;
        default: r = __builtin_rintf(t); break;
    }
    const float q = fminf(fabsf(r) * unit, kE1M2 ? 1.75f : 6.0f);
    uint32_t code;
    if (kE1M2) {
        code = static_cast<uint32_t>(q * 4.0f);
    } else {
        code = q < 2.0f ? static_cast<uint32_t>(q * 2.0f)
                        : (q < 4.0f ? static_cast<uint32_t>(q) + 2u : static_cast<uint32_t>(q * 0.5f) + 4u);
    }
    return sign | code;
}

__device__ __forceinline__ uint32_t pack4_i8(int a, int b, int c, int d)
{
    return (static_cast<uint32_t>(a) & 0xFFu) | ((static_cast<uint32_t>(b) & 0xFFu) << 8) |
           ((static_cast<uint32_t>(c) & 0xFFu) << 16) | ((static_cast<uint32_t>(d) & 0xFFu) << 24);
}

// Maps a linear workgroup id to a tile id such that each XCD (id mod 8) gets a contiguous range of tiles.
__device__ __forceinline__ uint32_t xcd_remap(uint32_t pid, uint32_t total)
{
    const uint32_t per = (total + 7u) / 8u;
    uint32_t tall = total % 8u;
    if (tall == 0) {
        tall = 8;
    }
    const uint32_t xcd = pid & 7u, local = pid >> 3;
    if (xcd < tall) {
        return local < per ? xcd * per + local : 0xFFFFFFFFu;  // a launch may be larger than `total`
    }
    if (local + 1u >= per) {
        return 0xFFFFFFFFu;  // the short XCDs own one tile less: this workgroup has nothing to do
    }
    return tall * per + (xcd - tall) * (per - 1u) + local;
}

// Tile t of a tiles_m x tiles_n grid in the order the tile kernels run them: bands of 8 row tiles, inside a band column
// by column with the row tiles of a column adjacent (up to 8 row tiles that is the plain column-by-column order).
// With xcd_remap an XCD's share is then a block of a few columns by 8 rows, whose rows of A and columns of B the
// workgroups that run side by side share in that XCD's L2, however many rows the matrix has.
__device__ __forceinline__ void band_order(uint32_t t, uint32_t tiles_m, uint32_t tiles_n, uint32_t& tm, uint32_t& tn)
{
    constexpr uint32_t kBand = 8;
    const uint32_t per_band = kBand * tiles_n, full = tiles_m / kBand;
    if (tiles_m <= kBand) {
        tm = t % tiles_m;
        tn = t / tiles_m;
    } else if (t < full * per_band) {
        const uint32_t r = t % per_band;
        tm = (t / per_band) * kBand + r % kBand;
        tn = r / kBand;
    } else {
        const uint32_t r = t - full * per_band, rows_last = tiles_m - full * kBand;
        tm = full * kBand + r % rows_last;
        tn = r / rows_last;
    }
}

}  // namespace ascq
