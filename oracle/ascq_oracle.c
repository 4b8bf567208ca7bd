/*
 * ascq_oracle.c - CPU restatement of the asc-devkit quantized-inference operators.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP kernels are
 * compared with; nothing in the shipped library links, loads or calls it, and
 * it must never be used as a fallback for a missing GPU path.  It is also the
 * program timed as the "CPU baseline" (kind "port": the reference's own CPU
 * build needs the closed CANN `tikicpulib` model, which is not available).
 *
 * All floating-point formats narrower than fp32 are implemented in software
 * (integer bit manipulation), so the oracle shares no arithmetic with the
 * device code, which uses the hardware's fp16 / bf16 instructions.
 *
 * Each operator cites the reference file it restates (paths relative to the
 * asc-devkit tree).  Pinning status of every function is listed in
 * oracle/README.md.
 *
 * Parity unpinned (no reference vector, document table or independent
 * implementation fixes these; the choice made is stated at the function):
 *   - the fixpipe int32 -> bf16 modes (defined by analogy with DEQF16);
 *   - NaN / Inf inputs of the int8 and half paths, and fp16 overflow inside the half chains;
 *   - fixpipe rounding for |acc| > 2^24, REQ8 offset signedness;
 *   - NaN -> fp8_e4m3fn (the reference's boundary table leaves that cell empty; +0 here, as for every other
 *     saturating cast in that table);
 *   - the nibble order of the fp4x2 types (the reference states one packing rule for int4x2 and both fp4x2 types;
 *     its int4 data scripts fix "even element in the low nibble", no fp4 vector exists).
 */
#include "ascq_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* --------------------------------------------------------------- threads */
static int g_threads = 1;
void orc_set_threads(int n)
{
    g_threads = n > 0 ? n : 1;
#ifdef _OPENMP
    omp_set_num_threads(g_threads);
#endif
}
int orc_get_threads(void) { return g_threads; }

/* ------------------------------------------------------- scalar numerics */
static inline uint32_t f32_bits(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}
static inline float bits_f32(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint64_t f64_bits(double d)
{
    uint64_t u;
    memcpy(&u, &d, 8);
    return u;
}

/* binary16 <- binary64, round to nearest even, IEEE overflow to infinity.
 * Pins: docs/zh/api/SIMD-API/基础API/数据结构/precision_conversion.md:520-534 (float -> half examples). */
uint16_t orc_f64_to_f16(double d)
{
    uint64_t u = f64_bits(d);
    uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
    int exp = (int)((u >> 52) & 0x7FF);
    uint64_t mant = u & 0xFFFFFFFFFFFFFull;
    if (exp == 0x7FF) {
        return (uint16_t)(sign | (mant ? 0x7E00u : 0x7C00u));
    }
    if (exp == 0) {
        return sign; /* zero or a binary64 subnormal, far below half the smallest binary16 subnormal */
    }
    int e = exp - 1023;
    if (e > 15) {
        return (uint16_t)(sign | 0x7C00u);
    }
    if (e >= -14) {
        uint64_t m = mant >> 42;
        uint64_t rem = mant & ((1ull << 42) - 1);
        uint64_t half = 1ull << 41;
        uint32_t r = (uint32_t)(((uint32_t)(e + 15) << 10) + m);
        if (rem > half || (rem == half && (m & 1))) {
            r += 1; /* a carry out of the mantissa increments the exponent, which is the right result */
        }
        if (r >= 0x7C00u) {
            r = 0x7C00u;
        }
        return (uint16_t)(sign | r);
    }
    /* subnormal result: value / 2^-24 rounded to an integer */
    int shift = 28 - e; /* (1.mant * 2^52) >> shift == value * 2^24 */
    if (shift > 63) {
        return sign;
    }
    uint64_t full = (1ull << 52) | mant;
    uint64_t m = full >> shift;
    uint64_t rem = full & ((1ull << shift) - 1);
    uint64_t half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (m & 1))) {
        m += 1;
    }
    return (uint16_t)(sign | (uint16_t)m);
}

uint16_t orc_f32_to_f16(float f) { return orc_f64_to_f16((double)f); }

float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1F;
    uint32_t mant = h & 0x3FFu;
    if (exp == 0x1F) {
        return bits_f32(sign | 0x7F800000u | (mant << 13));
    }
    if (exp == 0) {
        if (mant == 0) {
            return bits_f32(sign);
        }
        float v = (float)mant * 5.9604644775390625e-08f; /* 2^-24 */
        return sign ? -v : v;
    }
    return bits_f32(sign | ((exp + 112u) << 23) | (mant << 13));
}

/* bfloat16 <- binary32, round to nearest even.
 * ref: impl/basic_api/kernel_type_conversion_utils.h:48-60 (IsBf16NeedRound truth table),
 *      precision_conversion.md:541-553. */
uint16_t orc_f32_to_bf16(float f)
{
    uint32_t u = f32_bits(f);
    if ((u & 0x7F800000u) == 0x7F800000u) {
        if (u & 0x007FFFFFu) {
            return (uint16_t)((u >> 16) | 0x0040u);
        }
        return (uint16_t)(u >> 16);
    }
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

float orc_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

/* One IEEE operation in binary16: the exact result rounded once. */
uint16_t orc_f16_mul(uint16_t a, uint16_t b)
{
    /* 11-bit x 11-bit significands: the binary64 product is exact */
    return orc_f64_to_f16((double)orc_f16_to_f32(a) * (double)orc_f16_to_f32(b));
}
uint16_t orc_f16_add(uint16_t a, uint16_t b)
{
    /* exponents span 2^-24 .. 2^15: the binary64 sum is exact */
    return orc_f64_to_f16((double)orc_f16_to_f32(a) + (double)orc_f16_to_f32(b));
}
/* One operation in bfloat16 (8-bit significands: the binary32-range product is exact in binary64). */
uint16_t orc_bf16_mul(uint16_t a, uint16_t b)
{
    double p = (double)orc_bf16_to_f32(a) * (double)orc_bf16_to_f32(b);
    return orc_f32_to_bf16((float)p);
}
uint16_t orc_bf16_add(uint16_t a, uint16_t b)
{
    double s = (double)orc_bf16_to_f32(a) + (double)orc_bf16_to_f32(b);
    return orc_f32_to_bf16((float)s);
}

/* float -> int8 with a round mode and saturation.
 * ref: impl/basic_api/utils/kernel_utils_mode.h:94-109; precision_conversion.md:242-252 (half -> int8, saturating);
 *      impl/adv_api/detail/quantization/quant/ascend_quant_3510_impl.h:969-990 (f32 -> s16 -> f16 -> s8 chain,
 *      which equals a direct saturating conversion because every step saturates and s16 -> f16 is monotone). */
int8_t orc_round_sat8(double v, int round_mode)
{
    double r;
    if (v != v) {
        return 0; /* NaN: outside the pinned domain */
    }
    switch (round_mode) {
        case ASCQ_CAST_FLOOR: r = floor(v); break;
        case ASCQ_CAST_CEIL: r = ceil(v); break;
        case ASCQ_CAST_ROUND: r = round(v); break;
        case ASCQ_CAST_TRUNC: r = trunc(v); break;
        default: r = nearbyint(v); break; /* NONE / RINT: ties to even (default rounding direction) */
    }
    if (r > 127.0) {
        return 127;
    }
    if (r < -128.0) {
        return -128;
    }
    return (int8_t)r;
}

/* The value of an OCP 8-bit float code (sign handled by the caller): e4m3fn has bias 7, 3 mantissa bits and no
 * infinity (0x7F is NaN, 0x7E = 448 the largest finite); e5m2 has bias 15, 2 mantissa bits, 0x7B = 57344 the largest
 * finite.  ref: docs/zh/api/SIMD-API/基础API/数据结构/内置数据类型.md table 5. */
static double fp8_code_value(int code, int e5m2)
{
    int mant_bits = e5m2 ? 2 : 3, bias = e5m2 ? 15 : 7;
    int e = code >> mant_bits, m = code & ((1 << mant_bits) - 1);
    if (e == 0) {
        return ldexp((double)m, 1 - bias - mant_bits);
    }
    return ldexp((double)((1 << mant_bits) + m), e - bias - mant_bits);
}

/* fp32 -> 8-bit float by search: the nearest representable magnitude, ties to the even code, everything beyond the
 * largest finite value (infinity included) saturates to it (SatMode::SAT of the reference's cast trait,
 * ref: impl/adv_api/detail/quantization/quant/ascend_quant_per_group_3510_impl.h:41-42); NaN -> +0, the saturating
 * cast's answer (ref: docs/zh/api/附录/Reg矢量计算接口边界值汇总.md, rows float/fp8_e5m2_t; the e4m3 NaN cell of that
 * table is empty and is given the same answer here). */
uint8_t orc_f32_to_fp8(float f, int e5m2)
{
    int max_code = e5m2 ? 0x7B : 0x7E;
    uint8_t sign = signbit(f) ? 0x80 : 0;
    double a = fabs((double)f);
    if (f != f) {
        return 0;
    }
    if (a >= fp8_code_value(max_code, e5m2)) {
        return (uint8_t)(sign | max_code);
    }
    int lo = 0; /* largest code whose value is <= a */
    for (int c = 1; c <= max_code; ++c) {
        if (fp8_code_value(c, e5m2) <= a) {
            lo = c;
        }
    }
    double below = fp8_code_value(lo, e5m2), above = fp8_code_value(lo + 1, e5m2);
    int pick;
    if (a - below < above - a) {
        pick = lo;
    } else if (a - below > above - a) {
        pick = lo + 1;
    } else {
        pick = (lo & 1) ? lo + 1 : lo;
    }
    return (uint8_t)(sign | pick);
}

/* The 8 magnitudes of the 4-bit floats, code 0..7 (sign in bit 3).  e2m1: exponent bias 1, one mantissa bit, code 0/1
 * subnormal; e1m2: bias 1, two mantissa bits, codes 0..3 subnormal.  Largest values 6 and 1.75 as the reference's
 * boundary table has them (docs/zh/api/附录/Reg矢量计算接口边界值汇总.md, rows bfloat16_t/fp4x2_e2m1_t, .../e1m2_t). */
static const double kFp4E2M1[8] = {0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0};
static const double kFp4E1M2[8] = {0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75};

float orc_fp4_to_f32(uint8_t code, int e1m2)
{
    double v = (e1m2 ? kFp4E1M2 : kFp4E2M1)[code & 7];
    return (float)((code & 8) ? -v : v);
}

/* A (bfloat16) value -> 4-bit float by search over the 15 signed grid points: the two neighbours of the value, then
 * the rounding mode picks one; beyond the largest magnitude (infinity included) the result saturates; NaN -> +0; a
 * zero result keeps the sign of the input.  RINT ties go to the even code, ROUND ties away from zero.
 * ref: impl/adv_api/detail/quantization/quant/ascend_quant_3510_impl.h:994-1032 (Cast<fp4, bfloat16_t, castTrait>,
 * SatMode::SAT), boundary table named above. */
uint8_t orc_f32_to_fp4(float f, int e1m2, int round_mode)
{
    const double* grid = e1m2 ? kFp4E1M2 : kFp4E2M1;
    if (f != f) {
        return 0;
    }
    uint8_t sign = signbit(f) ? 8 : 0;
    double a = fabs((double)f);
    if (a >= grid[7]) {
        return (uint8_t)(sign | 7);
    }
    int lo = 0; /* largest code whose magnitude is <= a; lo + 1 exists because a < grid[7] */
    for (int c = 1; c < 8; ++c) {
        if (grid[c] <= a) {
            lo = c;
        }
    }
    if (grid[lo] == a) {
        return (uint8_t)(sign | lo);
    }
    int pick;
    double below = a - grid[lo], above = grid[lo + 1] - a;
    switch (round_mode) {
        case ASCQ_CAST_TRUNC: pick = lo; break;
        case ASCQ_CAST_FLOOR: pick = sign ? lo + 1 : lo; break; /* towards minus infinity */
        case ASCQ_CAST_CEIL: pick = sign ? lo : lo + 1; break;
        case ASCQ_CAST_ROUND: pick = below < above ? lo : lo + 1; break;
        default: pick = below < above ? lo : (below > above ? lo + 1 : ((lo & 1) ? lo + 1 : lo)); break;
    }
    return (uint8_t)(sign | pick);
}

float orc_fp8_to_f32(uint8_t code, int e5m2)
{
    int mag = code & 0x7F;
    if ((!e5m2 && mag == 0x7F) || (e5m2 && mag > 0x7C)) {
        return NAN;
    }
    if (e5m2 && mag == 0x7C) {
        return (code & 0x80) ? -INFINITY : INFINITY;
    }
    double v = fp8_code_value(mag, e5m2);
    return (float)((code & 0x80) ? -v : v);
}

/* ---- hifloat8: sign, a prefix-coded "dot" field that says how many exponent bits follow (0-4), a sign-magnitude
 * exponent and 3 / 3 / 3 / 2 / 1 mantissa bits for |exponent| 0 / 1 / 2-3 / 4-7 / 8-15; codes 1..7 are the powers of two
 * 2^-22 .. 2^-16 without mantissa; 0 is zero, 0x80 NaN, 0x6F / 0xEF the infinities; the largest finite value is
 * 2^15 (0x6E).  ref: examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_fp8/scripts/hif8.py:387-468
 * (cvt_hifuint8_to_float, over_mode True). */
float orc_hif8_to_f32(uint8_t code)
{
    int c = code & 0x7F, e;
    double m;
    if (c == 0) {
        return code == 0x80 ? NAN : 0.0f;
    }
    if (c == 0x6F) {
        return (code & 0x80) ? -INFINITY : INFINITY;
    }
    if (c < 8) {
        e = c - 23, m = 1.0;
    } else if (c < 16) {
        e = 0, m = 1.0 + (c & 7) / 8.0;
    } else if (c < 32) {
        e = (c & 8) ? -1 : 1, m = 1.0 + (c & 7) / 8.0;
    } else if (c < 64) {
        int f = (c >> 3) & 3;
        e = f >= 2 ? -f : f + 2, m = 1.0 + (c & 7) / 8.0;
    } else if (c < 96) {
        int f = (c >> 2) & 7;
        e = f >= 4 ? -f : f + 4, m = 1.0 + (c & 3) / 4.0;
    } else {
        int f = (c >> 1) & 15;
        e = f >= 8 ? -f : f + 8, m = 1.0 + (c & 1) / 2.0;
    }
    double v = ldexp(m, e);
    return (float)((code & 0x80) ? -v : v);
}

/* fp32 (or any narrower float, widened exactly) -> hifloat8 with RoundMode::CAST_ROUND, the cast's "round to nearest,
 * ties away from zero" (hif8.py:104-118 keeps one bit more than the mantissa and rounds an odd value up), written
 * here as a search over the code values rather than on the bits.  Between 2^-23 and 2^-22 the script rounds on the
 * grid of powers of two and then flushes 2^-23 to zero (:353-361), so the tie point of the smallest code is
 * 1.5 * 2^-23.  Saturating (SatMode::SAT, the trait every quantisation operator passes,
 * ascend_quant_per_group_3510_impl.h:100-101): magnitudes from 1.25 * 2^15 on, infinities included, give the largest
 * finite code, NaN gives 0 (hif8.py:198-214,318-331 with over_mode False); zero and everything that rounds to it
 * lose their sign. */
uint8_t orc_f32_to_hif8(float f)
{
    if (f != f) {
        return 0;
    }
    uint8_t sign = signbit(f) ? 0x80 : 0;
    double a = fabs((double)f);
    if (a >= 1.25 * 32768.0) {
        return (uint8_t)(sign | 0x6E);
    }
    if (a < ldexp(1.5, -23)) {
        return 0;
    }
    int best = 1;
    double best_d = fabs(a - (double)orc_hif8_to_f32(1));
    for (int c = 2; c <= 0x7F; ++c) {
        if (c == 0x6F) {
            continue; /* infinity */
        }
        double v = (double)orc_hif8_to_f32((uint8_t)c), dd = fabs(a - v);
        double bv = (double)orc_hif8_to_f32((uint8_t)best);
        if (dd < best_d || (dd == best_d && v > bv)) {
            best = c, best_d = dd;
        }
    }
    return (uint8_t)(sign | best);
}

static inline float load_as_f32(const void* p, size_t i, int dtype)
{
    switch (dtype) {
        case ASCQ_F16: return orc_f16_to_f32(((const uint16_t*)p)[i]);
        case ASCQ_BF16: return orc_bf16_to_f32(((const uint16_t*)p)[i]);
        case ASCQ_F32: return ((const float*)p)[i];
        case ASCQ_U64: return bits_f32((uint32_t)(((const uint64_t*)p)[i] & 0xFFFFFFFFull));
        default: return 0.0f;
    }
}

static inline void store_from_f32(void* p, size_t i, int dtype, float v)
{
    switch (dtype) {
        case ASCQ_F16: ((uint16_t*)p)[i] = orc_f32_to_f16(v); break;
        case ASCQ_BF16: ((uint16_t*)p)[i] = orc_f32_to_bf16(v); break;
        case ASCQ_F32: ((float*)p)[i] = v; break;
        default: break;
    }
}

/* int4 element i of a packed buffer: element 2j in the low nibble of byte j.
 * ref: impl/utils/common_types.h:57-111; examples/.../matmul_int4/scripts/gen_data.py:32-42. */
static inline int load_i4(const uint8_t* p, size_t i)
{
    uint8_t b = p[i >> 1];
    int v = (i & 1) ? (b >> 4) : (b & 0xF);
    return v >= 8 ? v - 16 : v;
}

/* ------------------------------------------------------------ AscendQuant */
/* index of the scale / offset element that applies to (row i, col j) */
static inline size_t quant_param_index(const ascq_quant_desc* d, size_t i, size_t j)
{
    switch (d->policy) {
        case ASCQ_PER_CHANNEL: return j;
        case ASCQ_PER_TOKEN: return i;
        case ASCQ_PER_GROUP:
            if (d->k_dim == 1) {
                size_t per_row = (d->n + d->group_size - 1) / d->group_size;
                return i * per_row + j / d->group_size;
            }
            return (i / d->group_size) * (size_t)d->n + j;
        default: return 0;
    }
}

/*
 * COMPUTE_F16   ref: impl/adv_api/detail/quantization/quant/ascend_quant_pre_impl.h:101-164 (per channel),
 *               :320-397 (per tensor), :439-483 (float scale/offset are cast to half first);
 *               bf16 source is first cast to half: ascend_quant_3510_impl.h:51-54.
 * COMPUTE_SCALE_T ref: .../quant/ascend_quant_per_group_3510_impl.h:142-178,498-538,1000-1044.
 * COMPUTE_F32   ref: impl/adv_api/detail/quantization/quantize/quantize_impl.h:641-695,737-792,832-872.
 */
int orc_quant(const ascq_quant_desc* d, int8_t* dst, const void* src, const void* scale, const void* offset)
{
    size_t total = d->cal_count;
    size_t n = (d->policy == ASCQ_PER_TENSOR) ? total : d->n;
    if (n == 0) {
        return 0;
    }
    size_t rows = total / n;
    int comp = d->compute;
    int ctype = (comp == ASCQ_COMPUTE_F16) ? ASCQ_F16 : (comp == ASCQ_COMPUTE_F32 ? ASCQ_F32 : d->scale_dtype);
    if (d->dst_format != ASCQ_QDST_I8 && d->dst_format != ASCQ_QDST_HIF8) {
        ctype = ASCQ_F32; /* the fp8 paths widen everything to fp32 (hifloat8 is computed like int8, in the scale type:
                             ascend_quant_per_group_3510_impl.h:93-127, ascend_quant_3510_impl.h:82-111):
                             ascend_quant_per_group_3510_impl.h:54-74, quantize_impl.h:64-73 */
    }
    int rmode = (comp == ASCQ_COMPUTE_F16) ? ASCQ_CAST_RINT : d->round_mode;
    const int fp4 = d->dst_format == ASCQ_QDST_FP4_E2M1 || d->dst_format == ASCQ_QDST_FP4_E1M2;
    if (fp4) {
        ctype = d->scale_dtype; /* the fp4 path multiplies in the scale type ...
                                   ascend_quant_per_group_3510_impl.h:346-379 */
    }
    /* ... and is not given the offset ("fp4 doesn't count offset", :1384) */
    const int offset_kind = fp4 ? (int)ASCQ_OFFSET_NONE : d->offset_kind;

#pragma omp parallel for schedule(static) if (rows * n > 65536)
    for (size_t i = 0; i < rows; ++i) {
        for (size_t j = 0; j < n; ++j) {
            size_t e = i * n + j;
            float s, o = 0.0f;
            if (d->policy == ASCQ_PER_TENSOR) {
                s = d->scale;
            } else {
                s = load_as_f32(scale, quant_param_index(d, i, j), d->scale_dtype);
            }
            if (offset_kind == ASCQ_OFFSET_SCALAR) {
                o = d->offset;
            } else if (offset_kind == ASCQ_OFFSET_TENSOR) {
                o = load_as_f32(offset, quant_param_index(d, i, j), d->scale_dtype);
            }
            float x = load_as_f32(src, e, d->src_dtype);
            double v;
            if (ctype == ASCQ_F16) {
                uint16_t xh = orc_f32_to_f16(x); /* exact for a half source */
                uint16_t t = orc_f16_mul(xh, orc_f32_to_f16(s));
                if (comp == ASCQ_COMPUTE_F16 || offset_kind != ASCQ_OFFSET_NONE) {
                    t = orc_f16_add(t, orc_f32_to_f16(o)); /* the legacy op always executes Adds/Add */
                }
                v = (double)orc_f16_to_f32(t);
            } else if (ctype == ASCQ_BF16) {
                uint16_t t = orc_bf16_mul(orc_f32_to_bf16(x), orc_f32_to_bf16(s));
                if (offset_kind != ASCQ_OFFSET_NONE) {
                    t = orc_bf16_add(t, orc_f32_to_bf16(o));
                }
                v = (double)orc_bf16_to_f32(t);
            } else {
                volatile float t = x * s; /* one fp32 rounding, never fused with the add */
                if (offset_kind != ASCQ_OFFSET_NONE) {
                    volatile float t2 = t + o;
                    t = t2;
                }
                v = (double)t;
            }
            if (d->dst_format == ASCQ_QDST_I8) {
                dst[e] = orc_round_sat8(v, rmode);
            } else if (d->dst_format == ASCQ_QDST_HIF8) {
                dst[e] = (int8_t)orc_f32_to_hif8((float)v); /* every round mode but HYBRID means CAST_ROUND here:
                                                               ascend_quant_3510_impl.h:900-933 */
            } else if (fp4) {
                /* to bfloat16 first (half-even), then to the 4-bit float with the requested rounding; two codes per
                 * byte, the even element in the low nibble.  Rows are whole bytes (n is even). */
                float b = orc_bf16_to_f32(orc_f32_to_bf16((float)v));
                uint8_t code = orc_f32_to_fp4(b, d->dst_format == ASCQ_QDST_FP4_E1M2, rmode);
                uint8_t* byte = (uint8_t*)dst + e / 2;
                *byte = (e & 1) ? (uint8_t)((*byte & 0x0F) | (code << 4)) : code;
            } else {
                dst[e] = (int8_t)orc_f32_to_fp8((float)v, d->dst_format == ASCQ_QDST_FP8_E5M2);
            }
        }
    }
    return 0;
}

/* Dynamic per-token quantisation: the composition ReduceMax(|x|) -> AscendQuant PER_TOKEN (scaleT = float)
 * ref: impl/adv_api/detail/quantization/quant/ascend_quant_per_group_3510_impl.h:142-178. */
int orc_dynamic_quant_per_token(int src_dtype, uint32_t m, uint32_t n, int8_t* q, float* tok_scale, const void* x)
{
#pragma omp parallel for schedule(static) if ((size_t)m * n > 65536)
    for (size_t i = 0; i < m; ++i) {
        float amax = 0.0f;
        for (size_t j = 0; j < n; ++j) {
            float a = fabsf(load_as_f32(x, i * n + j, src_dtype));
            if (a > amax) {
                amax = a;
            }
        }
        if (amax == 0.0f) {
            tok_scale[i] = 1.0f;
            memset(q + i * n, 0, n);
            continue;
        }
        volatile float inv = 127.0f / amax;
        tok_scale[i] = amax / 127.0f;
        for (size_t j = 0; j < n; ++j) {
            volatile float t = load_as_f32(x, i * n + j, src_dtype) * inv;
            q[i * n + j] = orc_round_sat8((double)t, ASCQ_CAST_RINT);
        }
    }
    return 0;
}

/* ---------------------------------------------------------- AscendDequant */
uint32_t orc_dequant_dst_stride(int dst_dtype, uint32_t n)
{
    uint32_t per_blk = (dst_dtype == ASCQ_F32) ? 8u : 16u; /* 32 bytes of dstT */
    return (n + per_blk - 1) / per_blk * per_blk;
}

/*
 * ref: impl/adv_api/detail/quantization/dequant/ascend_dequant_common_impl.h:207-223 (single-row reshape),
 *      :229-255 (scale -> fp32, uint64 keeps the low word), :260-267 (int32 -> fp32), :273-325 (Mul over the first
 *      calCount columns only), :328-362 (cast out), :368-431 (dst row stride padded to 32 bytes);
 *      per token / per group: .../dequant/ascend_dequant_3510_impl.h:227-307,337-380,449-537;
 *      worked example docs/zh/api/SIMD-API/高阶API/量化操作/AscendDequant.md:385-401.
 */
int orc_dequant(const ascq_dequant_desc* d, void* dst, const void* src, const void* scale)
{
    uint32_t m = d->m, n = d->n, cal = d->cal_count;
    if (d->policy >= ASCQ_PER_TOKEN) {
        /* the policy form counts elements: the first calCount / n rows are processed, every column of them scaled
         * (ref: impl/adv_api/detail/quantization/dequant/ascend_dequant_3510_impl.h:230, 272, 341, 397, 533) */
        m = n ? cal / n : 0;
        cal = n;
    }
    if (d->mode == ASCQ_DEQUANT_WITH_SINGLE_ROW && d->policy <= ASCQ_PER_CHANNEL) {
        uint32_t per_blk = (d->dst_dtype == ASCQ_F32) ? 8u : 16u;
        if (m == 1 && cal != 0 && cal % per_blk == 0 && n % cal == 0) {
            m = n / cal;
            n = cal;
        }
    }
    uint32_t stride = orc_dequant_dst_stride(d->dst_dtype, n);
#pragma omp parallel for schedule(static) if ((size_t)m * n > 65536)
    for (size_t i = 0; i < m; ++i) {
        for (size_t j = 0; j < n; ++j) {
            float x = (d->src_dtype == ASCQ_F32) ? ((const float*)src)[i * n + j]
                                                  : (float)((const int32_t*)src)[i * n + j]; /* RNE */
            float v = x;
            if (j < cal) {
                float s;
                switch (d->policy) {
                    case ASCQ_PER_TENSOR: s = d->scale; break;
                    case ASCQ_PER_CHANNEL: s = load_as_f32(scale, j, d->scale_dtype); break;
                    case ASCQ_PER_TOKEN: s = load_as_f32(scale, i, d->scale_dtype); break;
                    default:
                        if (d->k_dim == 1) {
                            size_t per_row = (n + d->group_size - 1) / d->group_size;
                            s = load_as_f32(scale, i * per_row + j / d->group_size, d->scale_dtype);
                        } else {
                            s = load_as_f32(scale, (i / d->group_size) * (size_t)n + j, d->scale_dtype);
                        }
                        break;
                }
                volatile float t = x * s;
                v = t;
            }
            store_from_f32(dst, i * stride + j, d->dst_dtype, v);
        }
    }
    return 0;
}

/* -------------------------------------------------------- AscendAntiQuant */
/*
 * ref: docs/zh/api/SIMD-API/高阶API/量化操作/AscendAntiQuant.md:36-50 (the contract),
 *      impl/adv_api/detail/quantization/antiquant/ascend_antiquant_impl.h:47-135 (cast, add offset, mul scale in
 *      half), .../ascend_antiquant_c220_impl.h:46-101 (bf16 output: fp32 add / mul, one rounding to bf16),
 *      examples/.../03_quantization/antiquant/scripts/gen_data.py:27-49.
 */
int orc_antiquant(const ascq_antiquant_desc* d, void* dst, const void* src, const void* offset, const void* scale)
{
    size_t K = d->k, N = d->n;
    size_t rows = d->is_transpose ? N : K;
    size_t cols = d->is_transpose ? K : N;
    uint32_t G;
    if (d->is_transpose) {
        G = d->scale_width ? d->scale_width : 1;
    } else {
        G = d->scale_height ? d->scale_height : 1;
    }
    size_t gs = K / G;
    int pt = d->dst_dtype; /* parameter dtype == dst dtype */
#pragma omp parallel for schedule(static) if (rows * cols > 65536)
    for (size_t i = 0; i < rows; ++i) {
        for (size_t j = 0; j < cols; ++j) {
            size_t e = i * cols + j;
            int w = (d->src_dtype == ASCQ_I4) ? load_i4((const uint8_t*)src, e) : ((const int8_t*)src)[e];
            float s, o = 0.0f;
            if (d->per_tensor) {
                /* scalars arrive as dstT values */
                s = (pt == ASCQ_F16) ? orc_f16_to_f32(orc_f32_to_f16(d->scale))
                                     : orc_bf16_to_f32(orc_f32_to_bf16(d->scale));
                o = (pt == ASCQ_F16) ? orc_f16_to_f32(orc_f32_to_f16(d->offset))
                                     : orc_bf16_to_f32(orc_f32_to_bf16(d->offset));
            } else {
                size_t pi = d->is_transpose ? (i * G + j / gs) : ((i / gs) * N + j);
                s = load_as_f32(scale, pi, pt);
                if (d->has_offset) {
                    o = load_as_f32(offset, pi, pt);
                }
            }
            if (d->dst_dtype == ASCQ_F16) {
                uint16_t h = orc_f32_to_f16((float)w); /* exact */
                if (d->has_offset) {
                    h = orc_f16_add(h, orc_f32_to_f16(o));
                }
                ((uint16_t*)dst)[e] = orc_f16_mul(orc_f32_to_f16(s), h);
            } else {
                volatile float t = (float)w;
                if (d->has_offset) {
                    volatile float t2 = t + o;
                    t = t2;
                }
                volatile float r = t * s;
                ((uint16_t*)dst)[e] = orc_f32_to_bf16(r);
            }
        }
    }
    return 0;
}

/* ------------------------------------------------- Matmul int8 quant path */
/* ref: examples/01_simd_cpp_api/05_best_practices/03_fusion_compute/quant_group_matmul_high_performance/scripts/
 *      gen_data.py:19-23 (FastGelu closed form), evaluated in fp32 with libm expf. */
float orc_faster_gelu(float x)
{
    float ax = fabsf(x);
    float x2 = expf(0.851f * (x - ax));
    float x3 = 1.0f + expf(-1.702f * ax);
    return x * x2 / x3;
}

/* The fp32 scale a quant parameter word carries.
 * ref: examples/01_simd_cpp_api/03_basic_api/03_matrix_compute/fixpipe_l0c2gm/scripts/gen_data_s322f16.py:37-66
 *      (bits [31:13] = sign, 8 exponent, 10 mantissa bits); matmul_quant/scripts/gen_data.py:36-40 (& 0xFFFFE000). */
float orc_quant_word_scale(uint64_t w, int scale_format)
{
    uint32_t lo = (uint32_t)(w & 0xFFFFFFFFull);
    if (scale_format == ASCQ_MM_SCALE_U64) {
        lo &= 0xFFFFE000u;
    }
    return bits_f32(lo);
}

/* The accumulator as the fixpipe hands it to the multiplier.  With the mode-control bit 36 of the word set it is first
 * shifted right arithmetically by bits [35:32] and saturated: for half outputs to the half range, rounded to half
 * (ref: fixpipe_l0c2gm/scripts/gen_data_s322f16.py:48-58 the fields, :84-90 the shift and `saturation(..., float16)`);
 * for 8-bit outputs to the int16 range (gen_data_s322s8.py:84-86).  No reference script covers the other output
 * types: there the shifted value is used as it is (parity unpinned for bfloat16 / float outputs with bit 36 set). */
float orc_prescaled_accumulator(int32_t acc, uint64_t qword, int scale_format, int out_dtype)
{
    if (scale_format != ASCQ_MM_SCALE_U64 || ((qword >> 36) & 1u) == 0) {
        return (float)acc;
    }
    int n = (int)((qword >> 32) & 0xF);
    /* arithmetic shift written out: floor division by 2^n */
    int64_t q = (int64_t)acc;
    int64_t sh = q >= 0 ? q / ((int64_t)1 << n) : -((-q + ((int64_t)1 << n) - 1) / ((int64_t)1 << n));
    if (out_dtype == ASCQ_F16) {
        double c = (double)sh;
        if (c > 65504.0) c = 65504.0;
        if (c < -65504.0) c = -65504.0;
        return orc_f16_to_f32(orc_f64_to_f16(c));
    }
    if (out_dtype == ASCQ_I8) {
        if (sh > 32767) sh = 32767;
        if (sh < -32768) sh = -32768;
    }
    return (float)sh;
}

/* Epilogue applied to one int32 accumulator.
 * ref: impl/adv_api/detail/matmul/stage/copy_cube_out/quant/quant_processor_fixpipe.h:89-117,197-222 (mode selection),
 *      fixpipe_l0c2gm/scripts/gen_data_s322f16.py:76-102 (deqf16: fp32 multiply, saturate to the fp16 range),
 *      gen_data_s322s8.py:76-97 (req8: round, saturate to 9 bits, add offset, saturate to 8 bits),
 *      quant_group_matmul_custom.asc:433-452 (channel scale, then token scale, then activation). */
/* v of one accumulator: channel scale, token scale, post-dequant bias, each one fp32 rounding (no activation yet). */
static inline float mm_value(const ascq_matmul_desc* d, int32_t acc, uint64_t qword, const float* tok_scale, size_t row,
                             const void* bias, size_t bias_idx)
{
    float s = orc_quant_word_scale(qword, d->scale_format);
    volatile float v = orc_prescaled_accumulator(acc, qword, d->scale_format, d->out_dtype) * s;
    if (d->has_tok_scale) {
        volatile float t = v * tok_scale[row];
        v = t;
    }
    if (d->bias_kind == ASCQ_MM_BIAS_F32_POST) {
        volatile float t = v + ((const float*)bias)[bias_idx];
        v = t;
    } else if (d->bias_kind == ASCQ_MM_BIAS_BF16_POST) {
        volatile float t = v + orc_bf16_to_f32(((const uint16_t*)bias)[bias_idx]);
        v = t;
    }
    return v;
}

/* SwiGLU in fp32, step by step as the reference's vector instructions round:
 * ref: impl/adv_api/detail/activation/swiglu/swiglu_common_impl.h:154-190 (Muls by -beta, Exp, Adds 1, Div, Mul). */
float orc_swiglu(float src0, float src1, float beta)
{
    volatile float nb = -1.0f * beta;
    volatile float t = src1 * nb;
    volatile float e = expf(t);
    volatile float dd = e + 1.0f;
    volatile float sw = src1 / dd;
    volatile float r = src0 * sw;
    return r;
}

/* Output conversion of one value (everything after the activation). */
static inline void mm_store(const ascq_matmul_desc* d, void* c, size_t idx, float r, uint64_t qword)
{
    switch (d->out_dtype) {
        case ASCQ_F16: {
            if (r > 65504.0f) r = 65504.0f;
            if (r < -65504.0f) r = -65504.0f;
            uint16_t h = orc_f32_to_f16(r);
            if ((h & 0x7FFFu) == 0x7C00u) {
                h = (uint16_t)((h & 0x8000u) | 0x7BFFu);
            }
            ((uint16_t*)c)[idx] = h;
            break;
        }
        case ASCQ_BF16: ((uint16_t*)c)[idx] = orc_f32_to_bf16(r); break;
        case ASCQ_F32: ((float*)c)[idx] = r; break;
        case ASCQ_I8: {
            double q = nearbyint((double)r);
            if (q > 255.0) q = 255.0;
            if (q < -256.0) q = -256.0;
            int off = (int)((qword >> 37) & 0x1FF); /* the spec script adds the 9 bits as an unsigned value */
            int t = (int)q + off;
            if ((qword >> 46) & 1) {
                if (t > 127) t = 127;
                if (t < -128) t = -128;
            } else {
                if (t > 255) t = 255;
                if (t < 0) t = 0;
            }
            ((int8_t*)c)[idx] = (int8_t)t;
            break;
        }
        default: break;
    }
}

static inline void mm_epilogue(const ascq_matmul_desc* d, void* c, size_t idx, int32_t acc, uint64_t qword,
                               const float* tok_scale, size_t row, const void* bias, size_t bias_idx)
{
    if (d->quant_mode == ASCQ_MM_QUANT_NONE) {
        ((int32_t*)c)[idx] = acc;
        return;
    }
    float v = mm_value(d, acc, qword, tok_scale, row, bias, bias_idx);
    if (d->activation == ASCQ_MM_ACT_FASTER_GELU) {
        v = orc_faster_gelu(v);
    }
    mm_store(d, c, idx, v, qword);
}

/* Exact int32 accumulation of rows [r0, r1) of A [.., k] with B [k, n] (or [n, k] when trans_b). */
static void mm_rows(const ascq_matmul_desc* d, void* c, const int8_t* a, const int8_t* b, const void* bias,
                    size_t bias_row_off, const uint64_t* qv, const float* qvf, const float* tok_scale, size_t r0,
                    size_t r1)
{
    size_t n = d->n, k = d->k, lda = d->trans_a ? d->m : d->k;
#pragma omp parallel
    {
        int32_t* acc = (int32_t*)malloc(n * sizeof(int32_t));
#pragma omp for schedule(dynamic, 4)
        for (size_t i = r0; i < r1; ++i) {
            for (size_t j = 0; j < n; ++j) {
                acc[j] = (d->bias_kind == ASCQ_MM_BIAS_I32_PRE) ? ((const int32_t*)bias)[bias_row_off + j] : 0;
            }
            if (!d->trans_b) {
                for (size_t kk = 0; kk < k; ++kk) {
                    int32_t av = d->trans_a ? a[kk * lda + i] : a[i * lda + kk];
                    const int8_t* brow = b + kk * n;
                    for (size_t j = 0; j < n; ++j) {
                        acc[j] += av * (int32_t)brow[j];
                    }
                }
            } else {
                for (size_t j = 0; j < n; ++j) {
                    const int8_t* bcol = b + j * k;
                    int32_t s = 0;
                    for (size_t kk = 0; kk < k; ++kk) {
                        int32_t av = d->trans_a ? a[kk * lda + i] : a[i * lda + kk];
                        s += av * (int32_t)bcol[kk];
                    }
                    acc[j] += s;
                }
            }
#define ORC_QWORD(j)                                                                                              \
    ((d->quant_mode == ASCQ_MM_QUANT_VECTOR)                                                                      \
         ? ((d->scale_format == ASCQ_MM_SCALE_U64) ? qv[bias_row_off + (j)] : (uint64_t)f32_bits(qvf[bias_row_off + (j)])) \
         : d->quant_scalar)
            if (d->quant_mode != ASCQ_MM_QUANT_NONE && d->activation == ASCQ_MM_ACT_SWIGLU) {
                /* columns 2j (src0) and 2j + 1 (src1) -> output column j of a row of n / 2 */
                for (size_t j = 0; j + 1 < n; j += 2) {
                    float v0 = mm_value(d, acc[j], ORC_QWORD(j), tok_scale, i, bias, bias_row_off + j);
                    float v1 = mm_value(d, acc[j + 1], ORC_QWORD(j + 1), tok_scale, i, bias, bias_row_off + j + 1);
                    mm_store(d, c, i * (n / 2) + j / 2, orc_swiglu(v0, v1, d->act_beta), 0);
                }
            } else {
                for (size_t j = 0; j < n; ++j) {
                    mm_epilogue(d, c, i * n + j, acc[j], ORC_QWORD(j), tok_scale, i, bias, bias_row_off + j);
                }
            }
#undef ORC_QWORD
        }
        free(acc);
    }
}

/* ref: include/adv_api/matmul/matmul.h:175-185; impl/adv_api/detail/matmul/matmul_impl_base.h:355-378;
 *      stage/compute/mmad_compute.h:40-82 (an int32 bias is the accumulator's initial value);
 *      examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_quant/scripts/gen_data.py:20-51. */
int orc_matmul_w8a8(const ascq_matmul_desc* d, void* c, const int8_t* a, const int8_t* b, const void* bias,
                    const void* quant_vector, const float* tok_scale)
{
    mm_rows(d, c, a, b, bias, 0, (const uint64_t*)quant_vector, (const float*)quant_vector, tok_scale, 0, d->m);
    return 0;
}

/* Same, restricted to rows [r0, r1): lets a benchmark time a bounded sample of a large problem. */
int orc_matmul_w8a8_rows(const ascq_matmul_desc* d, void* c, const int8_t* a, const int8_t* b, const void* bias,
                         const void* quant_vector, const float* tok_scale, uint32_t r0, uint32_t r1)
{
    mm_rows(d, c, a, b, bias, 0, (const uint64_t*)quant_vector, (const float*)quant_vector, tok_scale, r0, r1);
    return 0;
}

/* ref: examples/.../quant_group_matmul_high_performance/quant_group_matmul_custom.asc:255-289 (group walk, groups
 *      with a non-positive count are skipped), :425-454 (epilogue order); scripts/gen_data.py:31-57 (cumsum split). */
int orc_group_matmul_w8a8(const ascq_group_matmul_desc* g, void* y, const int8_t* x, const int8_t* w,
                          const void* bias, const float* scale, const float* tok_scale, const int64_t* group_list)
{
    const ascq_matmul_desc* d = &g->mm;
    size_t n = d->n, k = d->k;
    int64_t off = 0;
    for (uint32_t gi = 0; gi < g->groups; ++gi) {
        int64_t cnt;
        if (g->group_list_kind == ASCQ_GROUP_LIST_PREFIX_SUM) {
            cnt = group_list[gi] - off;
        } else {
            cnt = group_list[gi];
        }
        if (cnt <= 0) {
            continue;
        }
        int64_t end = off + cnt;
        if (end > (int64_t)d->m) {
            end = d->m;
        }
        if (end > off) {
            mm_rows(d, y, x, w + (size_t)gi * k * n, bias, (size_t)gi * n, NULL, scale, tok_scale, (size_t)off,
                    (size_t)end);
        }
        off += cnt;
    }
    return 0;
}

/* ------------------------------------------------------------------- W4A16 */
/* Weight de-quantisation = AscendAntiQuant<int4b_t, half>, half math
 * (ref: impl/adv_api/detail/quantization/antiquant/ascend_antiquant_impl.h:47-135), followed by an fp32-accumulated
 * dot product in increasing k order and one rounding to half. */
int orc_matmul_w4a16(const ascq_w4a16_desc* d, uint16_t* y, const uint16_t* x, const uint8_t* w,
                     const uint16_t* scale, const uint16_t* offset)
{
    return orc_matmul_w4a16_cols(d, y, x, w, scale, offset, 0, d->n);
}

/* Output columns [j0, j1) only: lets a benchmark time a bounded sample of a large problem. */
int orc_matmul_w4a16_cols(const ascq_w4a16_desc* d, uint16_t* y, const uint16_t* x, const uint8_t* w,
                          const uint16_t* scale, const uint16_t* offset, uint32_t j0, uint32_t j1)
{
    size_t M = d->m, N = d->n, K = d->k, gs = d->group_size;
    const size_t blk = 64; /* columns per task: each weight is de-quantised once and used for all m rows */
    size_t nblk = (j1 - j0 + blk - 1) / blk;
    float* xf = (float*)malloc(M * K * sizeof(float));
    for (size_t i = 0; i < M * K; ++i) {
        xf[i] = orc_f16_to_f32(x[i]);
    }
#pragma omp parallel
    {
        double* acc = (double*)malloc(M * blk * sizeof(double));
#pragma omp for schedule(dynamic, 1)
        for (size_t b = 0; b < nblk; ++b) {
            size_t c0 = j0 + b * blk, c1 = c0 + blk < j1 ? c0 + blk : j1;
            for (size_t t = 0; t < M * blk; ++t) {
                acc[t] = 0.0;
            }
            for (size_t kk = 0; kk < K; ++kk) {
                size_t g = kk / gs;
                for (size_t j = c0; j < c1; ++j) {
                    uint16_t h = orc_f32_to_f16((float)load_i4(w, kk * N + j));
                    if (d->has_offset) {
                        h = orc_f16_add(h, offset[g * N + j]);
                    }
                    double wd = (double)orc_f16_to_f32(orc_f16_mul(scale[g * N + j], h));
                    for (size_t i = 0; i < M; ++i) {
                        acc[i * blk + (j - c0)] += (double)xf[i * K + kk] * wd;
                    }
                }
            }
            for (size_t i = 0; i < M; ++i) {
                for (size_t j = c0; j < c1; ++j) {
                    y[i * N + j] = orc_f64_to_f16(acc[i * blk + (j - c0)]);
                }
            }
        }
        free(acc);
    }
    free(xf);
    return 0;
}

/* ------------------------------------- AscendAntiQuant PER_TOKEN / PER_GROUP */
/* One-byte sources (int8, fp8_e4m3fn, fp8_e5m2): the source is converted to the compute type (exact for every source
 * value), the offset is added and the scale multiplied in that type, one rounding each; an fp32 result going to a
 * 16-bit destination is rounded half-even and saturates (LayoutZMrgZRndRSatS): beyond the largest finite value, and
 * infinity, give that value, NaN gives +0 (ref: docs/zh/api/附录/Reg矢量计算接口边界值汇总.md, saturation-mode column
 * of the rows float/half and float/bfloat16_t).
 * ref: impl/adv_api/detail/quantization/antiquant/ascend_antiquant_3510_impl.h:1386-1403 (ConvertSrc),
 *      :1458-1495 (per token), :2176-2222 (group axis = kDim XOR isTranspose); fp32 arithmetic for AntiQuantize. */
static uint16_t f32_to_f16_sat(float v)
{
    if (v != v) {
        return 0;
    }
    if (v == v && v > 65504.0f) {
        v = 65504.0f;
    }
    if (v == v && v < -65504.0f) {
        v = -65504.0f;
    }
    return orc_f32_to_f16(v);
}

static uint16_t f32_to_bf16_sat(float v)
{
    const float top = 3.3895313892515355e38f; /* largest finite bfloat16 */
    if (v != v) {
        return 0;
    }
    if (v == v && v > top) {
        v = top;
    }
    if (v == v && v < -top) {
        v = -top;
    }
    return orc_f32_to_bf16(v);
}

/* fp4 sources, fp8_e8m0 scales (PER_GROUP): scale = 2^(code - 127) held as a bfloat16 (code 0: bits 0x0040 = 2^-127,
 * code 255: NaN), dst = bf16(src) * scale as a bfloat16 product, then the saturating cast when dst is half.
 * ref: impl/adv_api/detail/quantization/antiquant/ascend_antiquant_3510_impl.h:49-57, 69-74, 1727-1779. */
static void antiquant_fp4(const ascq_antiquant_policy_desc* d, uint16_t* dst, const uint8_t* src, const uint8_t* scale)
{
    size_t n = d->n, rows = n ? d->cal_count / n : 0;
    int along_n = (d->k_dim == 1) != (d->is_transpose != 0);
    size_t ppr = (n + d->group_size - 1) / d->group_size;
    for (size_t i = 0; i < rows; ++i) {
        for (size_t j = 0; j < n; ++j) {
            size_t e = i * n + j;
            size_t pi = along_n ? i * ppr + j / d->group_size : (i / d->group_size) * n + j;
            uint8_t code = (e & 1) ? (uint8_t)(src[e / 2] >> 4) : (uint8_t)(src[e / 2] & 15);
            uint16_t xb = orc_f32_to_bf16(orc_fp4_to_f32(code, d->src_format == ASCQ_QDST_FP4_E1M2)); /* exact */
            uint8_t c = scale[pi];
            uint16_t sb = c == 0 ? 0x0040 : (c == 255 ? 0x7FFF : (uint16_t)(c << 7));
            uint16_t prod = orc_bf16_mul(xb, sb);
            dst[e] = d->dst_dtype == ASCQ_BF16 ? prod : f32_to_f16_sat(orc_bf16_to_f32(prod));
        }
    }
}

int orc_antiquant_policy(const ascq_antiquant_policy_desc* d, void* dst, const uint8_t* src, const void* scale,
                         const void* offset)
{
    if (d->src_format == ASCQ_QDST_FP4_E2M1 || d->src_format == ASCQ_QDST_FP4_E1M2) {
        antiquant_fp4(d, (uint16_t*)dst, src, (const uint8_t*)scale);
        return 0;
    }
    size_t n = d->n, rows = n ? d->cal_count / n : 0;
    int along_n = (d->k_dim == 1) != (d->is_transpose != 0);
    size_t ppr = d->group_size ? (n + d->group_size - 1) / d->group_size : 0;
    int ct = d->compute == ASCQ_COMPUTE_F32 ? ASCQ_F32 : d->scale_dtype;
#pragma omp parallel for schedule(static) if (rows * n > 65536)
    for (size_t i = 0; i < rows; ++i) {
        for (size_t j = 0; j < n; ++j) {
            size_t e = i * n + j, pi;
            if (d->policy == ASCQ_PER_TOKEN) {
                pi = i;
            } else if (d->policy == ASCQ_PER_CHANNEL) {
                pi = j; /* AntiQuantize PER_CHANNEL: antiquantize_3510_impl.h:319-350 */
            } else if (d->policy == ASCQ_PER_TENSOR) {
                pi = 0;
            } else if (along_n) {
                pi = i * ppr + j / d->group_size;
            } else {
                pi = (i / d->group_size) * n + j;
            }
            float x = d->src_format == ASCQ_QDST_I8     ? (float)(int8_t)src[e]
                      : d->src_format == ASCQ_QDST_HIF8 ? orc_hif8_to_f32(src[e])
                                                        : orc_fp8_to_f32(src[e], d->src_format == ASCQ_QDST_FP8_E5M2);
            float s, o = 0.0f;
            if (d->policy == ASCQ_PER_TENSOR) {
                /* scalars of the output's type (antiquantize_3510_impl.h:253-283) */
                s = d->dst_dtype == ASCQ_F16 ? orc_f16_to_f32(orc_f32_to_f16(d->scale))
                                             : orc_bf16_to_f32(orc_f32_to_bf16(d->scale));
                if (d->has_offset) {
                    o = d->dst_dtype == ASCQ_F16 ? orc_f16_to_f32(orc_f32_to_f16(d->offset))
                                                 : orc_bf16_to_f32(orc_f32_to_bf16(d->offset));
                }
            } else {
                s = load_as_f32(scale, pi, d->scale_dtype);
                o = d->has_offset ? load_as_f32(offset, pi, d->scale_dtype) : 0.0f;
            }
            float v;
            if (ct == ASCQ_F16) {
                uint16_t t = orc_f32_to_f16(x);
                if (d->has_offset) {
                    t = orc_f16_add(t, orc_f32_to_f16(o));
                }
                v = orc_f16_to_f32(orc_f16_mul(t, orc_f32_to_f16(s)));
            } else if (ct == ASCQ_BF16) {
                uint16_t t = orc_f32_to_bf16(x);
                if (d->has_offset) {
                    t = orc_bf16_add(t, orc_f32_to_bf16(o));
                }
                v = orc_bf16_to_f32(orc_bf16_mul(t, orc_f32_to_bf16(s)));
            } else {
                volatile float t = x;
                if (d->has_offset) {
                    volatile float t2 = t + o;
                    t = t2;
                }
                volatile float t3 = t * s;
                v = t3;
            }
            if (d->dst_dtype == ASCQ_F32) {
                ((float*)dst)[e] = v;
            } else if (d->dst_dtype == ASCQ_F16) {
                ((uint16_t*)dst)[e] = ct == ASCQ_F16 ? orc_f32_to_f16(v) : f32_to_f16_sat(v);
            } else {
                ((uint16_t*)dst)[e] = ct == ASCQ_BF16 ? orc_f32_to_bf16(v) : f32_to_bf16_sat(v);
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------- W8A16 */
/* Matmul with A half and B int8 that is de-quantised on the way in: B goes through AscendAntiQuant<int8_t, half>
 * (half math: f16(w) + offset, then * scale, one rounding each;
 * ref: impl/adv_api/detail/matmul/stage/copy_cube_in/antiquant/antiquant_processor_using_ub.h:53-130 calling
 * impl/adv_api/detail/quantization/antiquant/ascend_antiquant_impl.h) with one scalar pair
 * (SetAntiQuantScalar) or one pair per output channel (SetAntiQuantVector, include/adv_api/matmul/matmul.h:161-168),
 * followed by a dot product accumulated wider than the output and rounded once. */
int orc_matmul_w8a16(const ascq_w8a16_desc* d, void* y, const uint16_t* x, const int8_t* w, const uint16_t* offset,
                     const uint16_t* scale)
{
    size_t M = d->m, N = d->n, K = d->k;
    const size_t blk = 64;
    size_t nblk = (N + blk - 1) / blk;
    uint16_t scale_s = orc_f32_to_f16(d->scale), offset_s = orc_f32_to_f16(d->offset);
    float* xf = (float*)malloc(M * K * sizeof(float));
    for (size_t i = 0; i < M * K; ++i) {
        xf[i] = orc_f16_to_f32(x[i]);
    }
#pragma omp parallel
    {
        double* acc = (double*)malloc(M * blk * sizeof(double));
#pragma omp for schedule(dynamic, 1)
        for (size_t b = 0; b < nblk; ++b) {
            size_t c0 = b * blk, c1 = c0 + blk < N ? c0 + blk : N;
            for (size_t t = 0; t < M * blk; ++t) {
                acc[t] = 0.0;
            }
            for (size_t kk = 0; kk < K; ++kk) {
                for (size_t j = c0; j < c1; ++j) {
                    uint16_t h = orc_f32_to_f16((float)(d->trans_b ? w[j * K + kk] : w[kk * N + j]));
                    if (d->has_offset) {
                        h = orc_f16_add(h, d->per_tensor ? offset_s : offset[j]);
                    }
                    double wd = (double)orc_f16_to_f32(orc_f16_mul(d->per_tensor ? scale_s : scale[j], h));
                    for (size_t i = 0; i < M; ++i) {
                        acc[i * blk + (j - c0)] += (double)xf[i * K + kk] * wd;
                    }
                }
            }
            for (size_t i = 0; i < M; ++i) {
                for (size_t j = c0; j < c1; ++j) {
                    double v = acc[i * blk + (j - c0)];
                    if (d->out_dtype == ASCQ_F32) {
                        ((float*)y)[i * N + j] = (float)v;
                    } else {
                        ((uint16_t*)y)[i * N + j] = orc_f64_to_f16(v);
                    }
                }
            }
        }
        free(acc);
    }
    free(xf);
    return 0;
}

/* ------------------------------------------------ block-scaled (MX) matmul */
/* Restates the golden of the reference's MmadMx examples: every operand element is its format's value times
 * 2^(scale - 127) of its row and block of 32 k, the product of the two decompressed matrices is formed in float64 and
 * rounded to the output type (examples/01_simd_cpp_api/03_basic_api/03_matrix_compute/mmad_mx/scripts/
 * gen_data.py:52-83,117-126; .../matmul_mxfp4_basic_api_high_performance/scripts/gen_data.py:50-63); a float32 bias
 * is added to the float32 result (gen_data.py:123-126).  b is [n, k] (the transposed right matrix the examples
 * write), 4-bit operands two per byte with the even k in the low nibble (pack_fp4_to_fp4x2, gen_data.py:38-49).
 * rows [r0, r1) and columns [c0, c1) are computed (the others of c are left alone).  Test infrastructure only. */
static double mx_elem(const uint8_t* row, size_t k, int fmt)
{
    if (fmt == ASCQ_QDST_FP8_E4M3FN || fmt == ASCQ_QDST_FP8_E5M2) {
        return (double)orc_fp8_to_f32(row[k], fmt == ASCQ_QDST_FP8_E5M2);
    }
    return (double)orc_fp4_to_f32((uint8_t)((row[k >> 1] >> (4 * (k & 1))) & 15), fmt == ASCQ_QDST_FP4_E1M2);
}

int orc_matmul_mx(const ascq_mx_desc* d, void* c, const uint8_t* a, const uint8_t* b, const uint8_t* sa,
                  const uint8_t* sb, const float* bias, uint32_t r0, uint32_t r1, uint32_t c0, uint32_t c1)
{
    const size_t K = d->k, N = d->n, SK = d->scale_k;
    const size_t arb = (d->a_format == ASCQ_QDST_FP4_E2M1 || d->a_format == ASCQ_QDST_FP4_E1M2) ? K / 2 : K;
    const size_t brb = (d->b_format == ASCQ_QDST_FP4_E2M1 || d->b_format == ASCQ_QDST_FP4_E1M2) ? K / 2 : K;
    /* decompress the columns once */
    double* bd = (double*)malloc((size_t)(c1 - c0) * K * sizeof(double));
    if (!bd) {
        return -1;
    }
#pragma omp parallel for schedule(static)
    for (long j = c0; j < (long)c1; ++j) {
        for (size_t k = 0; k < K; ++k) {
            bd[(size_t)(j - c0) * K + k] = mx_elem(b + (size_t)j * brb, k, d->b_format) * ldexp(1.0, (int)sb[(size_t)j * SK + k / 32] - 127);
        }
    }
#pragma omp parallel
    {
        double* ad = (double*)malloc(K * sizeof(double));
#pragma omp for schedule(dynamic, 1)
        for (long i = r0; i < (long)r1; ++i) {
            for (size_t k = 0; k < K; ++k) {
                ad[k] = mx_elem(a + (size_t)i * arb, k, d->a_format) * ldexp(1.0, (int)sa[(size_t)i * SK + k / 32] - 127);
            }
            for (size_t j = c0; j < c1; ++j) {
                const double* bj = bd + (j - c0) * K;
                double acc = 0.0;
                for (size_t k = 0; k < K; ++k) acc += ad[k] * bj[k];
                float v = (float)acc;
                if (d->has_bias) {
                    v = v + bias[j];
                }
                const size_t idx = (size_t)i * N + j;
                if (d->out_dtype == ASCQ_F32) {
                    ((float*)c)[idx] = v;
                } else if (d->out_dtype == ASCQ_BF16) {
                    ((uint16_t*)c)[idx] = orc_f32_to_bf16(v);
                } else {
                    ((uint16_t*)c)[idx] = orc_f32_to_f16(v);
                }
            }
        }
        free(ad);
    }
    free(bd);
    return 0;
}

/* ------------------------------------------------ vectorised array helpers */
void orc_f32_to_f16_array(uint16_t* dst, const float* src, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_f16(src[i]);
}
void orc_f16_to_f32_array(float* dst, const uint16_t* src, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f16_to_f32(src[i]);
}
void orc_f32_to_bf16_array(uint16_t* dst, const float* src, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f32_to_bf16(src[i]);
}
void orc_f16_mul_array(uint16_t* dst, const uint16_t* a, const uint16_t* b, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f16_mul(a[i], b[i]);
}
void orc_f16_add_array(uint16_t* dst, const uint16_t* a, const uint16_t* b, size_t n)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_f16_add(a[i], b[i]);
}
void orc_round_sat8_array(int8_t* dst, const float* src, size_t n, int round_mode)
{
    for (size_t i = 0; i < n; ++i) dst[i] = orc_round_sat8((double)src[i], round_mode);
}
