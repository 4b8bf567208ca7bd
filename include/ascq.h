/*
 * ascq.h - C ABI of libascq: the quantized-inference operators of the Ascend C
 * devkit (AscendQuant / AscendDequant / AscendAntiQuant, the int8 Matmul quant
 * path, the quantized grouped matmul, W4A16) implemented for one AMD MI355X
 * (gfx950).
 *
 * Every tensor argument is a DEVICE (HBM) pointer owned by the caller.  A call
 * validates its descriptor on the host, enqueues HIP kernels on `stream`
 * (a hipStream_t passed as void*; NULL = the default stream) and returns without
 * synchronising.  The library allocates nothing and never writes an input.
 * All entry points are thread-safe; the only state is a thread-local error
 * string (ascq_last_error).  Validation happens before the first HIP call, so
 * every error path can be exercised on a machine without a GPU.
 *
 * Citations "ref:" name files of the asc-devkit reference tree whose interface
 * the entry point replaces.
 */
#ifndef ASCQ_H
#define ASCQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ status */
typedef enum ascq_status {
    ASCQ_OK = 0,
    ASCQ_EINVAL = 1,       /* descriptor violates a shape / count rule           */
    ASCQ_EUNSUPPORTED = 2, /* dtype / mode combination the operator does not have */
    ASCQ_EALIGN = 3,       /* a 32-byte row rule or pointer alignment is violated */
    ASCQ_EHIP = 4,         /* a HIP runtime call failed (launch, no device)       */
    ASCQ_ENULL = 5         /* a required pointer is NULL                          */
} ascq_status;

/* -------------------------------------------------------------------- enums */
typedef enum ascq_dtype {
    ASCQ_F16 = 0,
    ASCQ_BF16 = 1,
    ASCQ_F32 = 2,
    ASCQ_I8 = 3,
    ASCQ_I4 = 4, /* two per byte, element 2j in the low nibble (ref: impl/utils/common_types.h:57-111) */
    ASCQ_I32 = 5,
    ASCQ_U64 = 6, /* fixpipe quant parameter word, fp32 scale in the low 32 bits */
    ASCQ_E8M0 = 7 /* fp8_e8m0_t: one byte, the value 2^(code - 127); code 255 is NaN (scales of the fp4 sources) */
} ascq_dtype;

/* ref: include/adv_api/quantization/ascend_quant_utils.h:73-80 (AscendQuantPolicy) */
typedef enum ascq_policy {
    ASCQ_PER_TENSOR = 0,
    ASCQ_PER_CHANNEL = 1,
    ASCQ_PER_TOKEN = 2,
    ASCQ_PER_GROUP = 3,
    /* declared by the reference (same header, and ascend_dequant_utils.h:37), implemented by none of its operators:
       every entry point answers them with ASCQ_EUNSUPPORTED */
    ASCQ_PER_CHANNEL_PER_GROUP = 4,
    ASCQ_PER_TOKEN_PER_GROUP = 5
} ascq_policy;

/* ref: impl/basic_api/utils/kernel_utils_mode.h:94-109 (RoundMode), same values */
typedef enum ascq_round_mode {
    ASCQ_CAST_NONE = 0, /* == RINT whenever precision is lost */
    ASCQ_CAST_RINT = 1, /* half to even */
    ASCQ_CAST_FLOOR = 2,
    ASCQ_CAST_CEIL = 3,
    ASCQ_CAST_ROUND = 4, /* half away from zero */
    ASCQ_CAST_TRUNC = 5,
    /* Declared so that they can be named and refused (ASCQ_EUNSUPPORTED): no operator of this library documents ODD,
     * and HYBRID (hifloat8 destinations only) has no usable specification in the reference: its one executable
     * statement, examples/.../matmul_fp8/scripts/hif8.py, rounds exactly representable values upward in its float32
     * path (:121-140: the comparison of the discarded bits with their own low half holds for 0 >= 0) and drops the
     * carry into the exponent in its float16 path (:160-178). */
    ASCQ_CAST_ODD = 6,
    ASCQ_CAST_HYBRID = 7
} ascq_round_mode;

/* Which arithmetic contract AscendQuant follows (the reference has three). */
typedef enum ascq_quant_compute {
    ASCQ_COMPUTE_F16 = 0,     /* AscendQuant per-tensor / per-channel: every intermediate is fp16
                                 (ref: impl/.../quant/ascend_quant_pre_impl.h:101-164,320-397)      */
    ASCQ_COMPUTE_SCALE_T = 1, /* AscendQuant PER_TOKEN / PER_GROUP: math in the scale dtype
                                 (ref: impl/.../quant/ascend_quant_per_group_3510_impl.h:142-178)   */
    ASCQ_COMPUTE_F32 = 2      /* Quantize: always fp32 (ref: impl/.../quantize/quantize_impl.h:641-968) */
} ascq_quant_compute;

/* Destination format of AscendQuant / Quantize.  The 8-bit floats are the OCP formats the reference names
 * fp8_e4m3fn_t (bias 7, no infinity, NaN = S.1111.111, max 448) and fp8_e5m2_t (bias 15, max 57344)
 * (ref: docs/zh/api/SIMD-API/基础API/数据结构/内置数据类型.md table 5). */
typedef enum ascq_quant_dst {
    ASCQ_QDST_I8 = 0,
    ASCQ_QDST_FP8_E4M3FN = 1,
    ASCQ_QDST_FP8_E5M2 = 2,
    /* 4-bit floats, two per byte with the even element in the low nibble (the packing rule the reference states for
     * int4x2 and both fp4x2 types together: docs/zh/api/SIMD-API/C-API/reg/reg_data_types/data_type_definition.md:17):
     * sign, then e2m1 (bias 1; 0, 0.5, 1, 1.5, 2, 3, 4, 6) or e1m2 (bias 1; 0, 0.25 .. 1.75 in steps of 0.25). */
    ASCQ_QDST_FP4_E2M1 = 3,
    ASCQ_QDST_FP4_E1M2 = 4,
    /* hifloat8_t: sign, a prefix-coded field that says how many exponent bits follow, a sign-magnitude exponent and
     * 3 / 3 / 3 / 2 / 1 mantissa bits for |exponent| 0 / 1 / 2-3 / 4-7 / 8-15; codes 1..7 are 2^-22 .. 2^-16; 0x80 is
     * NaN, 0x6F / 0xEF the infinities, 0x6E = 2^15 the largest finite value (the codec the reference ships as
     * examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_fp8/scripts/hif8.py).  As a destination (AscendQuant
     * per tensor / per channel / PER_TOKEN / PER_GROUP, Quantize: AscendQuant.md table 4) the value is computed like
     * the int8 result, in the same arithmetic type, then cast with RoundMode::CAST_ROUND (nearest, ties away from
     * zero), saturating: every round mode except HYBRID means that cast, as in the reference
     * (ascend_quant_3510_impl.h:900-933). */
    ASCQ_QDST_HIF8 = 5
} ascq_quant_dst;

typedef enum ascq_offset_kind { ASCQ_OFFSET_NONE = 0, ASCQ_OFFSET_SCALAR = 1, ASCQ_OFFSET_TENSOR = 2 } ascq_offset_kind;

/* ref: impl/basic_api/utils/kernel_utils_mode.h:181-184 (DeQuantMode) */
typedef enum ascq_dequant_mode { ASCQ_DEQUANT_WITH_SINGLE_ROW = 0, ASCQ_DEQUANT_WITH_MULTI_ROW = 1 } ascq_dequant_mode;

/* ------------------------------------------------------------ AscendQuant */
/*
 * ref: include/adv_api/quantization/ascend_quant.h:63-762, quantize.h.
 * dst int8 [cal_count]; src [cal_count] of src_dtype (F16|BF16|F32).
 *   PER_TENSOR : scalar `scale`/`offset`; elements = cal_count.
 *   PER_CHANNEL: scale tensor [scale_count] (= n); rows = cal_count / scale_count.
 *   PER_TOKEN  : scale [m]; rows = cal_count / n.
 *   PER_GROUP  : k_dim=1: scale [m, ceil(n/group_size)]; k_dim=0: scale [ceil(m/group_size), n].
 * Offset follows the scale's indexing when offset_kind == TENSOR, is the scalar
 * `offset` when SCALAR.  dst must not overlap src: a call whose byte ranges intersect returns ASCQ_EINVAL.  (The
 * reference lets the destination reuse the source's memory, docs/zh/api/SIMD-API/高阶API/量化操作/AscendQuant.md:435:
 * one core walks its tile in order.  Here thousands of wavefronts read and write at once, and an output byte lies
 * on top of an input element that another wavefront has yet to read.)  The same holds for ascq_dequant,
 * ascq_antiquant and ascq_antiquant_policy.
 * COMPUTE_F16:  y = sat8(rint( f16( f16( f16(x) * f16(s) ) + f16(o) ) ))   (policy TENSOR | CHANNEL)
 * COMPUTE_SCALE_T / F32: v = cvt(x) * s [+ o] with one rounding per operation in the compute
 *               type, y = sat8(round_mode(v)).
 * Tensor scale/offset dtype = scale_dtype (COMPUTE_F16: must equal src_dtype).
 * dst_format FP8_E4M3FN / FP8_E5M2 (one byte per element): the arithmetic is fp32 whatever `compute` says
 *               (source and parameters widened, one rounding per operation), then one conversion to the 8-bit
 *               float, round-half-even, saturating to the largest finite value (448 / 57344); the reference falls
 *               back to this rounding for every round_mode
 *               (ref: impl/adv_api/detail/quantization/quant/ascend_quant_per_group_3510_impl.h:33-79,
 *               impl/adv_api/detail/quantization/quantize/quantize_impl.h:64-73).  NaN gives +0, as the reference's
 *               saturating casts do (docs/zh/api/附录/Reg矢量计算接口边界值汇总.md, rows float/fp8_e5m2_t; the table
 *               leaves the e4m3 NaN cell empty, the same is done there).
 * dst_format FP4_E2M1 / FP4_E1M2 (dst holds cal_count / 2 bytes): PER_GROUP with COMPUTE_SCALE_T only, (src, scale)
 *               = (half, half), (half, float), (bfloat16, bfloat16), (bfloat16, float); v = cvt(x) * s in the scale
 *               type, one rounding; the offset is not applied ("fp4 doesn't count offset"); then bf16(v) (half-even)
 *               and bf16 -> fp4 with round_mode, saturating to +-6 / +-1.75, NaN -> +0.  n is a multiple of 8.
 *               (ref: impl/adv_api/detail/quantization/quant/ascend_quant_per_group_3510_impl.h:346-379, 1383-1385;
 *               ascend_quant_3510_impl.h:994-1032; boundary values: the table named above, rows
 *               bfloat16_t/fp4x2_e2m1_t and bfloat16_t/fp4x2_e1m2_t.)
 */
typedef struct ascq_quant_desc {
    int32_t policy;      /* ascq_policy */
    int32_t src_dtype;   /* ASCQ_F16 | ASCQ_BF16 | ASCQ_F32 */
    int32_t scale_dtype; /* dtype of the scale/offset tensors */
    int32_t compute;     /* ascq_quant_compute */
    int32_t round_mode;  /* an ascq_round_mode value; COMPUTE_F16 always rounds half-even */
    int32_t offset_kind; /* ascq_offset_kind */
    int32_t k_dim;       /* PER_GROUP: 1 = groups along n, 0 = groups along m */
    float scale;         /* PER_TENSOR scale */
    float offset;        /* scalar offset */
    uint32_t m, n;       /* PER_TOKEN / PER_GROUP row count and row length; PER_CHANNEL: n = scale_count */
    uint32_t cal_count;  /* number of elements processed */
    uint32_t group_size; /* PER_GROUP */
    int32_t dst_format;  /* ascq_quant_dst; 0 = int8 */
} ascq_quant_desc;

int ascq_quant(const ascq_quant_desc* desc, void* dst, const void* src, const void* scale, const void* offset,
               void* stream);

/*
 * Dynamic per-token quantisation of an activation matrix (no single reference
 * op: the reference composes it from ReduceMax/Abs and AscendQuant PER_TOKEN,
 * ref: impl/.../quant/ascend_quant_per_group_3510_impl.h:142-178).
 * x [m, n] F16|BF16|F32 row-major -> q int8 [m, n], tok_scale f32 [m]:
 *   amax = max_j |f32(x[i,j])|;  tok_scale[i] = amax / 127.0f (1.0f when amax == 0);
 *   q[i,j] = sat8(rint( f32(x[i,j]) * (127.0f / amax) ))      (0 when amax == 0).
 */
int ascq_dynamic_quant_per_token(int32_t src_dtype, uint32_t m, uint32_t n, void* q, void* tok_scale, const void* x,
                                 void* stream);

/* ---------------------------------------------------------- AscendDequant */
/*
 * ref: include/adv_api/quantization/ascend_dequant.h:58-305, ascend_dequant_utils.h:26-44.
 * src int32 (or f32 for PER_TOKEN/PER_GROUP) [m, n]; dst [m, n_dst] where
 * n_dst = n rounded up so that a dst row is a multiple of 32 bytes.
 *   j <  cal_count: dst[i,j] = dstT( f32(src[i,j]) * f32(scale) )
 *   cal_count <= j < n: dst[i,j] = dstT( f32(src[i,j]) )      (converted, not scaled)
 *   n <= j < n_dst: not written.
 * scale: PER_TENSOR scalar `scale`; PER_CHANNEL tensor [>=cal_count] of F32 | BF16 | U64
 * (U64: the low 32 bits are the fp32 scale); PER_TOKEN [m]; PER_GROUP as for quant.
 * PER_TOKEN / PER_GROUP (AscendDeQuantParam): cal_count counts elements, a multiple of n and at most m * n; the
 * first cal_count / n rows are processed and every column of them is scaled (ref: impl/adv_api/detail/quantization/
 * dequant/ascend_dequant_3510_impl.h:230, 341, 533).
 * SINGLE_ROW mode applies the reference's {1, m*n, n} -> {m, n, n} reshape rule.
 */
typedef struct ascq_dequant_desc {
    int32_t policy;      /* ascq_policy */
    int32_t src_dtype;   /* ASCQ_I32 (ASCQ_F32 allowed for PER_TOKEN / PER_GROUP) */
    int32_t scale_dtype; /* ASCQ_F32 | ASCQ_BF16 | ASCQ_U64 (also F16 for PER_TOKEN / PER_GROUP) */
    int32_t dst_dtype;   /* ASCQ_F16 | ASCQ_BF16 | ASCQ_F32 */
    int32_t mode;        /* ascq_dequant_mode */
    int32_t k_dim;       /* PER_GROUP axis */
    float scale;         /* PER_TENSOR scalar */
    uint32_t m, n, cal_count;
    uint32_t group_size;
} ascq_dequant_desc;

int ascq_dequant(const ascq_dequant_desc* desc, void* dst, const void* src, const void* scale, void* stream);

/* Number of dst elements per row (n rounded up to a 32-byte multiple of dst_dtype). */
uint32_t ascq_dequant_dst_stride(int32_t dst_dtype, uint32_t n);

/* -------------------------------------------------------- AscendAntiQuant */
/*
 * ref: include/adv_api/quantization/ascend_antiquant.h (10 overloads), ascend_antiquant_utils.h:27-32.
 * Not transposed: src [k, n], params [G, n], group = k / G:  dst[i][j] = scale[i/group][j] * (src[i][j] + offset[i/group][j])
 * Transposed    : src [n, k], params [n, G], group = k / G:  dst[i][j] = scale[i][j/group] * (src[i][j] + offset[i][j/group])
 * G = shape_info scale height (not transposed) / scale width (transposed); 0 means 1.
 * dst F16 : a = f16( f16(src) + off ), dst = f16( scale * a )           (fp16 math)
 * dst BF16: dst = bf16( (f32(src) + f32(off)) * f32(scale) )             (fp32 math)
 * src I8 or I4 (packed, low nibble first along the contiguous axis).
 * per_tensor != 0: `scale` / `offset` scalars are used instead of tensors.
 */
typedef struct ascq_antiquant_desc {
    int32_t src_dtype;    /* ASCQ_I8 | ASCQ_I4 */
    int32_t dst_dtype;    /* ASCQ_F16 | ASCQ_BF16 (= dtype of scale / offset tensors) */
    int32_t is_transpose; /* 0: src [k, n]; 1: src [n, k] */
    int32_t has_offset;
    int32_t per_tensor;
    float scale, offset;  /* per_tensor scalars (rounded once to dst_dtype) */
    uint32_t k, n;
    uint32_t offset_height, offset_width, scale_height, scale_width; /* AntiQuantShapeInfo */
} ascq_antiquant_desc;

int ascq_antiquant(const ascq_antiquant_desc* desc, void* dst, const void* src, const void* offset, const void* scale,
                   void* stream);

/*
 * AscendAntiQuant<dstT, srcT, scaleT, config, policy> for PER_TOKEN / PER_GROUP, and AntiQuantize
 * (ref: include/adv_api/quantization/ascend_antiquant.h, the AscendAntiQuantParam overloads;
 *  impl/adv_api/detail/quantization/antiquant/ascend_antiquant_3510_impl.h:1386-1403 (source conversion),
 *  :1458-1495 (per token), :2170-2222 (dispatch); type table docs/zh/api/SIMD-API/高阶API/量化操作/AscendAntiQuant.md 表3).
 * src [m, n] one byte per element: int8, fp8_e4m3fn or fp8_e5m2 (src_format, an ascq_quant_dst value);
 * dst [m, n] of dst_dtype; only the first cal_count elements (a multiple of n) are processed.
 *   PER_TOKEN: scale / offset [m].
 *   PER_GROUP: the group axis is k_dim XOR is_transpose: 1 = along n, parameters [m, ceil(n / group_size)];
 *              0 = along m, parameters [ceil(m / group_size), n].  The data stay [m, n] row-major either way.
 *   v = ct(src) ; v = ct(v + offset) if has_offset ; v = ct(v * scale) ; dst = dstT(v)
 * with ct = the scale dtype (ASCQ_COMPUTE_SCALE_T: AscendAntiQuant) or fp32 (ASCQ_COMPUTE_F32: AntiQuantize); every
 * source value is exact in every ct.  A 16-bit ct requires dst_dtype == scale_dtype; an fp32 result is rounded
 * half-even to a 16-bit dst, saturating at the largest finite value (NaN -> +0).
 *   fp4 sources (src_format ASCQ_QDST_FP4_E2M1 / FP4_E1M2: two values per byte, even element in the low nibble, src
 *              holds cal_count / 2 bytes): PER_GROUP only, scale_dtype ASCQ_E8M0 (one byte per group, same indexing
 *              as above), no offset, dst half | bfloat16: dst = bf16(src) * bf16(2^(code - 127)) as a bfloat16
 *              product (exact: at most 3 significant bits times a power of two; overflow gives infinity), a scale
 *              code of 255 is NaN; a half dst is the saturating half-even cast of that product (NaN -> +0).
 *              n % 8 == 0.  (ref: impl/adv_api/detail/quantization/antiquant/ascend_antiquant_3510_impl.h:49-57
 *              (codes 0 and 255), :1727-1779 (groups along n), :1793-1850 (along m); AscendAntiQuant.md 表3.)
 *   PER_CHANNEL (AntiQuantize only, ASCQ_COMPUTE_F32): scale / offset [n] of dst_dtype (half | bfloat16).
 *   PER_TENSOR  (AntiQuantize only, ASCQ_COMPUTE_F32): the scalars `scale` / `offset` of the descriptor, taken as
 *              dst_dtype values (rounded once to it); the scale / offset pointers are ignored.
 *              (ref: impl/adv_api/detail/quantization/antiquantize/antiquantize_impl.h:42-45, 70-110;
 *               antiquantize_3510_impl.h:253-362: fp32 arithmetic, saturating cast to half / bfloat16.)
 */
typedef struct ascq_antiquant_policy_desc {
    int32_t policy;      /* ASCQ_PER_TOKEN | ASCQ_PER_GROUP; with ASCQ_COMPUTE_F32 also PER_TENSOR | PER_CHANNEL */
    int32_t src_format;  /* ASCQ_QDST_I8 | ASCQ_QDST_FP8_E4M3FN | ASCQ_QDST_FP8_E5M2 | ASCQ_QDST_FP4_E2M1 | _E1M2 */
    int32_t scale_dtype; /* ASCQ_F16 | ASCQ_BF16 | ASCQ_F32: dtype of the scale / offset tensors; ASCQ_E8M0 for fp4 */
    int32_t dst_dtype;   /* ASCQ_F16 | ASCQ_BF16 | ASCQ_F32 */
    int32_t compute;     /* ASCQ_COMPUTE_SCALE_T | ASCQ_COMPUTE_F32 */
    int32_t has_offset;
    int32_t is_transpose;
    int32_t k_dim;       /* PER_GROUP: AscendAntiQuantConfig::kDim */
    uint32_t m, n;
    uint32_t cal_count;
    uint32_t group_size; /* PER_GROUP: positive multiple of 32 */
    float scale, offset; /* PER_TENSOR scalars */
} ascq_antiquant_policy_desc;

int ascq_antiquant_policy(const ascq_antiquant_policy_desc* desc, void* dst, const void* src, const void* scale,
                          const void* offset, void* stream);

/* ------------------------------------------------- Matmul int8 quant path */
typedef enum ascq_mm_quant_mode {
    ASCQ_MM_QUANT_NONE = 0,   /* int32 out */
    ASCQ_MM_QUANT_SCALAR = 1, /* SetQuantScalar (ref: impl/adv_api/detail/matmul/matmul_impl_base.h:355-366) */
    ASCQ_MM_QUANT_VECTOR = 2  /* SetQuantVector, one parameter per output channel (ref: :367-378) */
} ascq_mm_quant_mode;

typedef enum ascq_mm_scale_format {
    ASCQ_MM_SCALE_U64 = 0, /* fixpipe word: scale = f32(bits[31:0] & 0xFFFFE000)  (1-8-10 float), REQ8: bits[45:37]
                              offset, bit 46 sign (ref: examples/.../fixpipe_l0c2gm/scripts/gen_data_s322f16.py:37-66).
                              Mode-control bit 36 (scalar word or any word of a vector): the accumulator is first
                              shifted right arithmetically by bits [35:32] and saturated, to the half range with one
                              rounding to half for F16 outputs (gen_data_s322f16.py:84-90), to the int16 range for I8
                              outputs (gen_data_s322s8.py:84-86); BF16 / F32 outputs, which no reference script
                              covers, take the shifted value unsaturated.  The fixpipe's separate relu_pre word
                              (another scale for negative accumulators, gen_data_s322f16.py:20-34,92-97) is not part
                              of SetQuantScalar / SetQuantVector and has no field here */
    ASCQ_MM_SCALE_F32 = 1  /* plain fp32, all 23 mantissa bits used */
} ascq_mm_scale_format;

/* Layout of the B (weight) matrix in memory. */
typedef enum ascq_mm_b_format {
    ASCQ_MM_B_ND = 0, /* row-major [k, n] ([n, k] with trans_b) */
    ASCQ_MM_B_NZ = 1  /* the reference's fractal weight format for int8: [n/32][k/16][16][32], i.e. panels of 32
                         columns, each a row-major [k][32] block; element (k, j) lies at
                         ((j/32) * K + k) * 32 + j % 32
                         (ref: examples/.../quant_group_matmul_high_performance/scripts/gen_data.py:62-65;
                         CubeFormat::NZ of MatmulType, include/adv_api/matmul/matmul.h).
                         Needs n % 32 == 0, k % 128 == 0, k * n < 2^32, no transposition. */
} ascq_mm_b_format;

typedef enum ascq_mm_bias_kind {
    ASCQ_MM_BIAS_NONE = 0,
    ASCQ_MM_BIAS_I32_PRE = 1,   /* int32 [n], initial value of the accumulator
                                   (ref: impl/adv_api/detail/matmul/stage/compute/mmad_compute.h:40-82) */
    ASCQ_MM_BIAS_F32_POST = 2,  /* fp32 [n] added after dequant */
    ASCQ_MM_BIAS_BF16_POST = 3  /* bf16 [n] added after dequant (widened to fp32) */
} ascq_mm_bias_kind;

typedef enum ascq_mm_activation {
    ASCQ_MM_ACT_NONE = 0,
    ASCQ_MM_ACT_FASTER_GELU = 1, /* x*exp(0.851(x-|x|))/(1+exp(-1.702|x|)) (ref: examples/.../quant_group_matmul_high_performance/scripts/gen_data.py:19-23) */
    /* SwiGLU over interleaved column pairs: column 2j of the matmul is src0, column 2j + 1 is src1, and output
       column j (C is [m, n / 2]) is src0 * swish(src1) with swish(x) = x / (1 + exp(-beta x)), computed in fp32 in
       the reference's order: t = x * (-beta); e = exp(t); d = e + 1; s = x / d; out = src0 * s, one rounding each
       (ref: impl/adv_api/detail/activation/swiglu/swiglu_common_impl.h:154-190; golden
       examples/.../01_activation/swiglu/scripts/gen_data.py:32).  n must be even, the output floating point
       (F16 / BF16 / F32); beta is ascq_matmul_desc.act_beta.  A gate / up projection whose weight columns are
       stored interleaved (up_0, gate_0, up_1, gate_1, ...) produces silu(gate) * up directly with beta = 1. */
    ASCQ_MM_ACT_SWIGLU = 2
} ascq_mm_activation;

/*
 * ref: include/adv_api/matmul/matmul.h:175-185 (SetQuantScalar/SetQuantVector),
 *      impl/adv_api/detail/matmul/stage/copy_cube_out/quant/quant_processor_fixpipe.h:74-222.
 * A int8 [m, k] (trans_a: [k, m]); B int8 [k, n] (trans_b: [n, k]); row-major, dense.
 *   acc[i,j] = sum_k A[i,k]*B[k,j] (+ bias_i32[j])                          exact int32
 *   QUANT_NONE: C int32 = acc.
 *   else v = f32(acc) * s_j  [* tok_scale[i]]  [+ bias_post[j]]  [act]      one fp32 rounding per op
 *        (ASCQ_MM_ACT_SWIGLU combines the v of columns 2j and 2j + 1 into output column j: C is [m, n / 2])
 *        C = F16: f16(v) saturated to +-65504;  BF16: bf16 rne;  F32: v;
 *            I8 (U64 format only): sat( sat9(rint(v)) + offset9 ), offset9 = bits[45:37] taken as unsigned,
 *            saturating to int8 when bit 46 is set and to uint8 otherwise.
 */
typedef struct ascq_matmul_desc {
    uint32_t m, n, k;
    int32_t trans_a, trans_b;
    int32_t out_dtype;     /* ASCQ_I32 | ASCQ_F16 | ASCQ_BF16 | ASCQ_F32 | ASCQ_I8 */
    int32_t quant_mode;    /* ascq_mm_quant_mode */
    int32_t scale_format;  /* ascq_mm_scale_format */
    int32_t bias_kind;     /* ascq_mm_bias_kind */
    int32_t has_tok_scale; /* fp32 [m] multiplied after the channel scale */
    int32_t activation;    /* ascq_mm_activation */
    int32_t b_format;      /* ascq_mm_b_format; for the grouped matmul every group's [k, n] block is in this format */
    uint64_t quant_scalar; /* QUANT_SCALAR: U64 word, or fp32 bits in the low half for F32 format */
    float act_beta;        /* ASCQ_MM_ACT_SWIGLU: the constant of the swish function (1 = SiLU); ignored otherwise */
    int32_t reserved;      /* set to 0 */
} ascq_matmul_desc;

int ascq_matmul_w8a8(const ascq_matmul_desc* desc, void* c, const void* a, const void* b, const void* bias,
                     const void* quant_vector, const void* tok_scale, void* workspace, size_t workspace_bytes,
                     void* stream);
/* The workspace ascq_matmul_w8a8 needs for this descriptor with operands aligned to 16 bytes (0 for most shapes; the
 * partial sums of the few-row kernels; with ASCQ_MM_ACT_SWIGLU outside the large tile kernel the raw accumulators
 * [m][n]).  A call that needs more than it was given (SwiGLU on misaligned operands) names the size in its error. */
int ascq_matmul_w8a8_workspace_size(const ascq_matmul_desc* desc, size_t* bytes);

/*
 * The same matmul for few activation rows (decode, small batches) on weights pre-packed for this GPU, the step the
 * reference does offline for its own L1 / L0 layout (examples/.../quant_group_matmul_high_performance/scripts/
 * gen_data.py:62-64 packs ND -> NZ before the kernel runs).  ascq_pack_weight_w8 turns B int8 [k, n] (trans_b: [n, k])
 * into ascq_pack_weight_w8_size(k, n) bytes: slabs of 16 columns, each one contiguous run of tiles of 64 k (1 KiB: lane l
 * of a wavefront owns column l % 16 and the 16 consecutive bytes k 16 (l / 16) .. + 15); columns past n and k past the
 * end hold 0, and 16 tiles of zeros follow the last slab.
 * ascq_matmul_w8a8_packed computes exactly what ascq_matmul_w8a8 computes (same descriptor, epilogues - SwiGLU
 * included - and outputs; desc.trans_b is ignored, desc.trans_a is not supported) in one launch with no workspace: a
 * workgroup owns whole columns, its wavefronts split k, and integer partial sums are exact in any order.  Up to 16
 * rows (fewer at long k: 13 at k = 11008, n = 4096) the activations stay in LDS and the weights stream past them
 * once.  More rows with k up to 16384 turn the roles round: a workgroup first fetches the weights of its columns into
 * registers and then streams the activations past them, still in one launch.  Every workgroup reads all of the
 * activations there, so from a few hundred rows on (always above 512; between 129 and 512 by an estimate of both
 * times) the call runs the tile kernels of ascq_matmul_w8a8 instead, which read the packed tiles as they lie (n % 16 ==
 * 0 and k % 128 == 0; other shapes stay with the registers form): weights packed for decode serve prefill at the speed
 * of unpacked ones, without a second copy.  With k above 16384 the rows that do not fit the LDS take one pass over the
 * weights per group that does.  Requires k % 64 == 0 and a, w_packed 16-byte aligned.
 * ref: include/adv_api/matmul/matmul.h:175-185 (the Matmul object and its quant epilogue)
 */
int ascq_pack_weight_w8_size(uint32_t k, uint32_t n, size_t* bytes);
int ascq_pack_weight_w8(const void* b, void* w_packed, uint32_t k, uint32_t n, int32_t trans_b, void* stream);
int ascq_matmul_w8a8_packed(const ascq_matmul_desc* desc, void* c, const void* a, const void* w_packed, const void* bias,
                            const void* quant_vector, const void* tok_scale, void* stream);

/*
 * Matmul<int4b_t A, int4b_t B, C>: the same descriptor, epilogues and outputs as ascq_matmul_w8a8 with both operands
 * packed two int4 per byte, even element in the low nibble: A [m, k/2] bytes, B [k, n/2] bytes ([n, k/2] with
 * trans_b).  trans_a is not supported (the reference's rule for an int4 A), b_format is ND, k is even, n is even
 * unless trans_b.  Both operands are widened to int8 in the workspace (mandatory; size from the query below), then the
 * int8 matmul runs.  a, b and the workspace are 16-byte aligned.
 * ref: examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_int4/matmul_int4.asc:52-58, 155; README.md
 *      ("Constraints"); packing: scripts/gen_data.py:32-42.
 */
int ascq_matmul_w4a4(const ascq_matmul_desc* desc, void* c, const void* a, const void* b, const void* bias,
                     const void* quant_vector, const void* tok_scale, void* workspace, size_t workspace_bytes,
                     void* stream);
int ascq_matmul_w4a4_workspace_size(const ascq_matmul_desc* desc, size_t* bytes);
/* int4 (two per byte, even element in the low nibble) -> int8, `elements` values (even); 16-byte aligned pointers. */
int ascq_unpack_int4(void* dst, const void* src, size_t elements, void* stream);

/*
 * The launch plan of a matmul call: which kernel family the library picks for these arguments and how it tiles the
 * problem.  The counterpart of the host-side tiling result the reference computes before a launch
 * (ref: include/adv_api/matmul/matmul_tilingdata.h:21-72, TCubeTiling: usedCoreNum ~ workgroups, baseM / baseN /
 * baseK ~ tile_m / tile_n / tile_k, shareL1Size ~ lds_bytes); here it is informational, the call plans by itself.
 */
typedef enum ascq_mm_kernel {
    ASCQ_MM_KERNEL_GENERIC = 0,      /* one lane per output element: unaligned or transposed-A inputs */
    ASCQ_MM_KERNEL_STREAM = 1,       /* few rows: weight streams, one per SIMD, then a kernel that adds their pieces */
    ASCQ_MM_KERNEL_DMA_128 = 2,      /* m <= 512: 128 x 128 direct-to-LDS tiles, K split over workgroups when a
                                        workspace is given (k_splits > 1: a second kernel adds the partial tiles) */
    ASCQ_MM_KERNEL_DMA_256 = 3,      /* 256 x 256 direct-to-LDS tiles; a last partial round of the chip may be run
                                        by further workgroups of the same launch with 256 x narrow_tile_n tiles */
    ASCQ_MM_KERNEL_STAGED = 4        /* register-staged tiles: K not a multiple of 128, or n not a multiple of 16
                                        (a transposed B otherwise runs on the direct-to-LDS kernels like a plain one) */
} ascq_mm_kernel;

typedef struct ascq_matmul_plan {
    int32_t kernel;             /* ascq_mm_kernel */
    uint32_t tile_m, tile_n;    /* rows x columns of C per workgroup (per wavefront stream for KERNEL_STREAM: the
                                   rows x columns a stream accumulates at a time); 1 x 1 for KERNEL_GENERIC */
    uint32_t tile_k;            /* K per main-loop step */
    uint32_t workgroups;        /* workgroups of the main launch */
    uint32_t k_splits;          /* partial sums per output element (1: the main kernel writes C itself) */
    uint32_t launches;          /* kernel launches per call */
    uint32_t lds_bytes;         /* LDS per workgroup of the main launch */
    uint32_t narrow_tile_n;     /* KERNEL_DMA_256: columns per tile of the narrow tiles, 0 if there are none */
    uint32_t narrow_workgroups; /* workgroups that run them, beyond `workgroups` */
    size_t workspace_bytes;     /* bytes of the workspace this plan uses (0: the call runs without) */
} ascq_matmul_plan;

/* Same arguments as ascq_matmul_w8a8 (pointers are only inspected: NULL checks and alignment), no launch. */
int ascq_matmul_w8a8_plan(const ascq_matmul_desc* desc, const void* c, const void* a, const void* b, const void* bias,
                          const void* quant_vector, const void* tok_scale, const void* workspace,
                          size_t workspace_bytes, ascq_matmul_plan* plan);

/*
 * The W8A8 linear with dynamic activation quantisation in one call:
 *   q, tok = ascq_dynamic_quant_per_token(x) ;  c = ascq_matmul_w8a8(q, b, ..., tok_scale = tok)
 * with exactly those results.  x [m, k] of x_dtype (ASCQ_F16 | ASCQ_BF16 | ASCQ_F32); desc as for ascq_matmul_w8a8 with
 * a dequantising epilogue (quant_mode SCALAR or VECTOR, floating-point out_dtype); desc->has_tok_scale is ignored.
 * The two kernels run one after the other on the stream, with q and tok in the workspace (sized by
 * ascq_linear_w8a8_dynamic_workspace_size; always required, whatever kernel runs).  Decode calls - half or bfloat16 x
 * on weights kept as [n, k] (desc->trans_b), k a multiple of 64, up to 7 rows at k = 4096, 4 at 7168, 2 at 14848 - are
 * one launch: the weight-streaming kernel quantises x itself on its way into LDS (the same bits; the workspace is not
 * touched).  No single reference operator does this: the reference composes it from
 * ReduceMax / AscendQuant PER_TOKEN (ascend_quant_per_group_3510_impl.h:142-178) and Matmul (matmul.h:175-185).
 */
int ascq_linear_w8a8_dynamic(const ascq_matmul_desc* desc, int32_t x_dtype, void* c, const void* x, const void* b,
                             const void* bias, const void* quant_vector, void* workspace, size_t workspace_bytes,
                             void* stream);
int ascq_linear_w8a8_dynamic_workspace_size(const ascq_matmul_desc* desc, size_t* bytes);

/*
 * The same linear on weights packed once by ascq_pack_weight_w8 (see ascq_matmul_w8a8_packed for the layout and what
 * the descriptor may ask for: no trans_a, no NZ, k % 64 == 0; desc->trans_b is ignored).  Results are those
 * of ascq_linear_w8a8_dynamic on the unpacked weights, bit for bit.  Up to 8 rows of half or bfloat16 x are one launch
 * (the packed decode kernel quantises x itself); otherwise the quantiser kernel runs first and
 * ascq_matmul_w8a8_packed after it, with q and the token scales in the workspace.  The workspace holds
 * round256(m * k) + round256(4 * m) bytes; ascq_linear_w8a8_dynamic_workspace_size covers that.
 * It has no counterpart in the reference (which composes the linear from ReduceMax / AscendQuant PER_TOKEN and Matmul,
 * ascend_quant_per_group_3510_impl.h:142-178, matmul.h:175-185, on weights it packs offline, gen_data.py:62-64).
 */
int ascq_linear_w8a8_dynamic_packed(const ascq_matmul_desc* desc, int32_t x_dtype, void* c, const void* x,
                                    const void* w_packed, const void* bias, const void* quant_vector, void* workspace,
                                    size_t workspace_bytes, void* stream);

/*
 * ascq_linear_w8a8_dynamic without a workspace argument and without any allocation (no hipMalloc / hipFree, here or in
 * anything it calls).  It has no counterpart in the reference; it is for callers that cannot allocate device memory:
 * code under stream capture, tight serving loops, harnesses that forbid hipMalloc.  The scratch (quantised
 * activations, token scales, partial sums of the small-m kernels) is a device array of ASCQ_STATIC_SCRATCH_BYTES that
 * is part of the library; every GPU the library runs on holds its own copy until the process ends.  Shapes whose
 * ascq_linear_w8a8_dynamic_workspace_size exceeds that size are rejected with ASCQ_EINVAL (k = 4096, n = 11008 fits
 * with 1, 16, 128 and 2048 rows; 32 rows need 32 MiB of partial sums and do not).  Results are those of
 * ascq_linear_w8a8_dynamic, bit for bit.  All calls on one GPU share the one array: calls that overlap in time on
 * the same GPU (two streams, two threads) race; serialise them or use the workspace form.  The first call on a device
 * looks the array's address up (hipGetSymbolAddress); make that call outside stream capture.
 */
#define ASCQ_STATIC_SCRATCH_BYTES (24u << 20)
int ascq_linear_w8a8_dynamic_noalloc(const ascq_matmul_desc* desc, int32_t x_dtype, void* c, const void* x, const void* b,
                                     const void* bias, const void* quant_vector, void* stream);

/* ------------------------------------------------ quantized grouped matmul */
typedef enum ascq_group_list_kind {
    ASCQ_GROUP_LIST_COUNTS = 0,    /* rows per group (ref: examples/.../quant_group_matmul_custom.asc:264) */
    ASCQ_GROUP_LIST_PREFIX_SUM = 1 /* inclusive prefix sums */
} ascq_group_list_kind;

/*
 * ref: examples/01_simd_cpp_api/05_best_practices/03_fusion_compute/quant_group_matmul_high_performance/
 *      quant_group_matmul_custom.asc:255-454.
 * x int8 [m, k]; w int8 [groups, k, n]; scale fp32 [groups, n]; tok_scale fp32 [m] (optional);
 * bias [groups, n] per mm.bias_kind; group_list int64 [groups] (device).  Rows of group g are
 * [off_g, off_g + cnt_g); rows beyond the last group are not written; groups with cnt <= 0 are skipped.
 *   y[i,j] = out( act( (f32(acc) * scale[g][j]) * tok_scale[i] + bias[g][j] ) )
 * mm.m is the row capacity of x / y, mm.quant_mode must be QUANT_VECTOR, scale_format F32.
 */
typedef struct ascq_group_matmul_desc {
    ascq_matmul_desc mm;
    uint32_t groups;
    int32_t group_list_kind; /* ascq_group_list_kind */
} ascq_group_matmul_desc;

int ascq_group_matmul_w8a8(const ascq_group_matmul_desc* desc, void* y, const void* x, const void* w,
                           const void* bias, const void* scale, const void* tok_scale, const int64_t* group_list,
                           void* stream);

/* ------------------------------------------------------------------- W4A16 */
/*
 * W4A16 weight-only linear = AscendAntiQuant<int4b_t, half> (per-group along k,
 * ref: include/adv_api/quantization/ascend_antiquant.h:50-54) feeding a half GEMV/GEMM.
 * x f16 [m, k]; w int4 [k, n] packed along n (n even); scale, offset f16 [k/group_size, n].
 *   wdq[k,j] = f16( scale[k/g][j] * f16( f16(w[k,j]) + offset[k/g][j] ) )     (offset optional)
 *   y[i,j]   = f16( sum_k f32(x[i,k]) * f32(wdq[k,j]) )                       fp32 accumulation
 * workspace: ascq_matmul_w4a16_workspace_size bytes of scratch for the partial sums of the weight streams (contents
 * need not be initialised); calls that share a workspace must not overlap.
 */
typedef enum ascq_w4a16_mode {
    ASCQ_W4A16_PER_WEIGHT = 0, /* wdq rounded to half per weight, the formula above: AscendAntiQuant's own arithmetic */
    /*
     * Scale and offset applied once per quantisation group to fp32 sums, with no rounding per weight:
     *   y[i,j] = f16( sum_g f32(scale[g][j]) * ( sum_{k in g} x[i,k] * w[k,j] + f32(offset[g][j]) * sum_{k in g} x[i,k] ) )
     * The same real-number value as the per-weight form without its 2 * k roundings to half; the two forms differ by
     * about 3e-4 of the result's magnitude, inside the tolerance of a half output (1 bf16 ulp).  Honoured by
     * ascq_matmul_w4a16_packed when group_size is a multiple of 128; elsewhere the per-weight form runs.
     */
    ASCQ_W4A16_GROUP_SUM = 1
} ascq_w4a16_mode;

typedef struct ascq_w4a16_desc {
    uint32_t m, n, k;
    uint32_t group_size;
    int32_t has_offset;
    int32_t mode; /* ascq_w4a16_mode; 0 = the reference's per-weight arithmetic */
} ascq_w4a16_desc;

int ascq_matmul_w4a16(const ascq_w4a16_desc* desc, void* y, const void* x, const void* w, const void* scale,
                      const void* offset, void* workspace, size_t workspace_bytes, void* stream);
int ascq_matmul_w4a16_workspace_size(const ascq_w4a16_desc* desc, size_t* bytes);

/*
 * The same operator on weights pre-packed for this GPU (the step the reference does offline for its own L1 / L0
 * layout: examples/.../quant_group_matmul_high_performance/scripts/gen_data.py:62-64 packs ND -> NZ before the kernel
 * runs).  ascq_pack_weight_w4 turns w int4 [k, n] (two per byte along n, even column in the low nibble) into
 * ascq_pack_weight_w4_size(k, n) bytes: slabs of 16 columns, each one contiguous run of tiles of 128 k (1 KiB: lane l
 * of a wavefront owns column l % 16 and k 32 (l / 16) .. + 31; dword d of its 16 bytes holds k + 8 d .. + 7 with k
 * offsets 0..7 in nibbles 0 4 1 5 2 6 3 7, nibbles stored as w + 8); columns past n and k past the end hold w = 0, and
 * 16 tiles of w = 0 follow the last slab.  scale / offset stay [k / group_size, n].
 * ascq_matmul_w4a16_packed computes exactly what ascq_matmul_w4a16 computes (same roundings per weight, fp32 sums, one
 * rounding to half) in one launch with no workspace: a workgroup owns whole columns and adds its wavefronts' partial
 * sums in a fixed order, so repeated calls give identical bits.  Up to 4 activation rows (decode) its wavefronts
 * split k and add their sums in LDS; 5 to 16 rows run one wavefront per slab with the activations shared chunk by
 * chunk; more rows take further passes of 16 over the weights.  Requires k % 128 == 0, n % 8 == 0, group_size =
 * 32 * 2^i (ASCQ_EUNSUPPORTED otherwise: use ascq_matmul_w4a16), and x, w_packed, scale, offset 16-byte aligned.
 */
int ascq_pack_weight_w4_size(uint32_t k, uint32_t n, size_t* bytes);
int ascq_pack_weight_w4(const void* w, void* w_packed, uint32_t k, uint32_t n, void* stream);
int ascq_matmul_w4a16_packed(const ascq_w4a16_desc* desc, void* y, const void* x, const void* w_packed,
                             const void* scale, const void* offset, void* stream);

/* ------------------------------------------------------------------- W8A16 */
/*
 * Matmul with A half and B int8 de-quantised on the way in ("anti-quant" matmul): the B matrix is turned into half by
 * AscendAntiQuant<int8_t, half> with one scalar pair (SetAntiQuantScalar, MatmulConfig::isPerTensor) or one pair per
 * output channel (SetAntiQuantVector), then a half matmul with fp32 accumulation.
 * ref: include/adv_api/matmul/matmul.h:161-168;
 *      impl/adv_api/detail/matmul/stage/copy_cube_in/antiquant/antiquant_processor_using_ub.h:53-130.
 * x f16 [m, k]; w int8 [k, n], or [n, k] with trans_b (the reference's isTransposeB: SetTensorB(b, true));
 * scale, offset f16 [n] (per channel) or the desc's scalars (per tensor).
 *   wdq[k,j] = f16( scale[j] * f16( f16(w[k,j]) + offset[j] ) )               (offset iff has_offset)
 *   y[i,j]   = out( sum_k f32(x[i,k]) * f32(wdq[k,j]) )                       fp32 accumulation
 * Few activation rows (decode) run weight-streaming kernels: the weights are read once per 32 rows of x ([k, n]) or
 * per 16 rows ([n, k]).  With trans_b a column's weights are one contiguous run, so whole columns belong to one
 * workgroup: one launch, no workspace (the size query answers 0), identical bits from call to call; that form needs
 * k % 128 == 0 and 16-byte aligned x and w (other shapes and alignments run a slow kernel with one lane per output
 * element, as they do for [k, n] weights).
 * Many rows (more than 32 on [n, k] weights, more than 96 on [k, n]) run a half GEMM on 128 x 128 tiles whose B-tile
 * loader de-quantises; [k, n] weights are first copied transposed into the workspace (k * n bytes, which the size query
 * then asks for; given less, the call falls back to one pass over the weights per 32 rows).
 * workspace: ascq_matmul_w8a16_workspace_size bytes (contents need not be initialised); calls that share a
 * workspace must not overlap.
 */
/* How the de-quantisation is carried out (ascq_w8a16_desc.mode).
 * PER_WEIGHT (0, the default): the reference's arithmetic, f16(scale * f16(f16(w) + offset)) for every weight, then the
 *   half matmul with fp32 sums.
 * CHANNEL_SUM: y[i,j] = out( scale[j] * ( sum_k x[i,k] w[k,j] + offset[j] * sum_k x[i,k] ) ) with both sums in fp32 and
 *   the int8 weights as exact halves: scale and offset applied once per output instead of twice rounded per weight.
 *   Not the reference's bits; within one bf16 ulp and 1e-3 relative of them (and closer to the exact value of the
 *   quantised product).  Honoured for up to 4 rows on [n, k] weights (trans_b) with k % 128 == 0; elsewhere the
 *   per-weight form runs. */
typedef enum ascq_w8a16_mode { ASCQ_W8A16_PER_WEIGHT = 0, ASCQ_W8A16_CHANNEL_SUM = 1 } ascq_w8a16_mode;

typedef struct ascq_w8a16_desc {
    uint32_t m, n, k;
    int32_t per_tensor;  /* 1: scale / offset below (SetAntiQuantScalar); 0: vectors of n halves (SetAntiQuantVector) */
    int32_t has_offset;  /* MatmulConfig::hasAntiQuantOffset */
    float scale, offset; /* per-tensor parameters, rounded to half as the reference's half scalars */
    int32_t out_dtype;   /* ASCQ_F16 | ASCQ_F32 */
    int32_t trans_b;     /* 0: w is [k, n]; 1: w is [n, k] */
    int32_t mode;        /* ascq_w8a16_mode */
} ascq_w8a16_desc;

int ascq_matmul_w8a16(const ascq_w8a16_desc* desc, void* y, const void* x, const void* w, const void* offset,
                      const void* scale, void* workspace, size_t workspace_bytes, void* stream);
int ascq_matmul_w8a16_workspace_size(const ascq_w8a16_desc* desc, size_t* bytes);

/* --------------------------------------------- block-scaled (MX) matmul */
/*
 * MmadMx as a whole-matrix operator: c[m, n] = sum_k A[i, k] * B[j, k] (+ bias[j]) with
 *   A[i, k] = value(a[i, k]) * 2^(a_scale[i, k / 32] - 127),  B[j, k] = value(b[j, k]) * 2^(b_scale[j, k / 32] - 127):
 * every 32 consecutive k of a row share one fp8_e8m0 scale.  a is [m, k] and b is [n, k] (the right matrix and its
 * scales transposed, the form the reference's examples feed), row-major; 4-bit formats are packed two per byte along k,
 * even k in the low nibble, rows of k / 2 bytes (k even).  a_scale is [m, scale_k] and b_scale [n, scale_k] bytes with
 * scale_k >= ceil(k / 32) (the reference rounds it up to an even number).  Products and sums are fp32 in the matrix
 * core (exact products; the sum's order is the hardware's), c is rounded once: the reference's golden is the float64
 * product rounded to the output type, compared at rtol = atol = 1e-3.
 * a_format / b_format: ASCQ_QDST_FP8_E4M3FN | ASCQ_QDST_FP8_E5M2 | ASCQ_QDST_FP4_E2M1 | ASCQ_QDST_FP4_E1M2.
 * Two 8-bit operands, or two e2m1 operands, with k % 128 == 0 (8-bit) / k % 256 == 0 (4-bit), 16-byte aligned a, b and
 * scale_k % 8 == 0, scale_k >= 16 run v_mfma_scale_f32_32x32x64_f8f6f4 on 256 x 256 tiles straight from the given buffers.  Other
 * format pairs first widen their 4-bit operands in the workspace (two e1m2 operands to 6-bit e2m3 codes, anything else
 * to e4m3; both exact); other shapes take a kernel with one
 * lane per output element.
 * ref: include/basic_api/kernel_operator_mm_intf.h:321-340 (MmadMx), examples/01_simd_cpp_api/03_basic_api/
 *      03_matrix_compute/mmad_mx/README.md:5,131-152 and scripts/gen_data.py:52-140 (layouts, golden),
 *      examples/01_simd_cpp_api/05_best_practices/01_matrix_compute/matmul_mxfp4_basic_api_high_performance/
 *      scripts/gen_data.py:36-72 (m = n = k = 8192, bfloat16 output).
 */
typedef struct ascq_mx_desc {
    uint32_t m, n, k;
    uint32_t scale_k;    /* bytes per row of a_scale / b_scale */
    int32_t a_format;    /* ascq_quant_dst: FP8_E4M3FN, FP8_E5M2, FP4_E2M1, FP4_E1M2 */
    int32_t b_format;
    int32_t out_dtype;   /* ASCQ_F32 | ASCQ_BF16 | ASCQ_F16 */
    int32_t has_bias;    /* bias is fp32 [n], added to the fp32 sum before the rounding */
} ascq_mx_desc;

int ascq_matmul_mx(const ascq_mx_desc* desc, void* c, const void* a, const void* b, const void* a_scale,
                   const void* b_scale, const void* bias, void* workspace, size_t workspace_bytes, void* stream);
int ascq_matmul_mx_workspace_size(const ascq_mx_desc* desc, size_t* bytes);

/* --------------------------------------------- host "tiling" size queries */
/*
 * Scratch-size queries with the reference's answers, for callers that size a
 * shared temporary buffer from them.  On the GPU the elementwise operators need
 * no scratch; the values are the reference's so that existing host code keeps
 * working.  ref: impl/adv_api/tiling/quantization/ascend_quant_tiling_impl.cpp:31-68,
 * ascend_dequant_tiling_impl.cpp, ascend_antiquant_tiling_impl.cpp.
 */
int ascq_get_ascend_quant_max_min_tmp_size(const uint32_t* shape, uint32_t ndim, uint32_t type_size,
                                           uint32_t* max_value, uint32_t* min_value);
int ascq_get_ascend_dequant_max_min_tmp_size(const uint32_t* shape, uint32_t ndim, uint32_t type_size,
                                             uint32_t* max_value, uint32_t* min_value);
int ascq_get_ascend_antiquant_max_min_tmp_size(const uint32_t* src_shape, uint32_t src_ndim,
                                               const uint32_t* scale_shape, uint32_t scale_ndim, int32_t is_transpose,
                                               int32_t input_dtype, int32_t output_dtype, uint32_t* max_value,
                                               uint32_t* min_value);
/*
 * The reference's Get*TmpBufferFactorSize: a temporary buffer of maxLiveNodeCount * (bytes processed at once) + extraBuf
 * bytes serves the operator (ascend_quant_tiling_impl.cpp:57-61, ascend_dequant_tiling_impl.cpp:67-81,
 * ascend_antiquant_tiling_impl.cpp:145-169; GetQuantizeTmpBufferFactorSize answers as the AscendQuant form).  Same
 * values, for host code that sizes a shared buffer from them; input_format of the AntiQuant form is an ascq_quant_dst
 * value (the source formats of ascq_antiquant_policy; int4 sources answer as ASCQ_QDST_I8).
 */
int ascq_get_ascend_quant_tmp_buffer_factor_size(uint32_t* max_live_node_count, uint32_t* extra_buf);
int ascq_get_ascend_dequant_tmp_buffer_factor_size(const uint32_t* shape, uint32_t ndim, uint32_t* max_live_node_count,
                                                   uint32_t* extra_buf);
int ascq_get_ascend_antiquant_tmp_buffer_factor_size(const uint32_t* src_shape, uint32_t src_ndim,
                                                     const uint32_t* scale_shape, uint32_t scale_ndim,
                                                     int32_t is_transpose, int32_t input_format, int32_t output_dtype,
                                                     uint32_t* max_live_node_count, uint32_t* extra_buf);

/* -------------------------------------------------------------- utilities */
/* Pack an fp32 scale (and optional REQ8 offset / sign) into the fixpipe uint64 word. Host-side, pure. */
uint64_t ascq_pack_quant_param(float scale, int32_t offset9, int32_t is_signed);
/*
 * Weight pre-pack: int8 [groups][k][n] (row-major, "ND") -> the fractal "NZ" layout
 * [groups][n/32][k/16][16][32] that ASCQ_MM_B_NZ consumes (element (g, kk, c) at
 * ((g * n/32 + c/32) * k + kk) * 32 + c%32).  k % 16 == 0, n % 32 == 0, both
 * pointers 16-byte aligned, dst != src.  The device-side form of the packing the
 * reference does offline.
 * ref: examples/01_simd_cpp_api/05_best_practices/03_fusion_compute/
 *      quant_group_matmul_high_performance/scripts/gen_data.py:62-64
 */
int ascq_pack_weight_nz(uint32_t groups, uint32_t k, uint32_t n, void* dst, const void* src, void* stream);
/* Fill `bytes` of device memory with zero using a kernel (safe inside stream capture). */
int ascq_zero_fill(void* ptr, size_t bytes, void* stream);
const char* ascq_last_error(void);
const char* ascq_version(void);

#ifdef __cplusplus
}
#endif
#endif /* ASCQ_H */
