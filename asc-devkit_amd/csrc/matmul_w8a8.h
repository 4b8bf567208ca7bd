// Shared between the translation units of the int8 matmul: parameter blocks and the per-element epilogue.
#pragma once
#include "ascq_common.h"
#include "ascq_device.h"

namespace ascq {

struct EpiParams {
    void* c;
    const void* bias;
    const void* quant;  // uint64 words or fp32 scales, one per output channel (VECTOR mode)
    const float* tok_scale;
    uint32_t ldc;
    int out_dtype, quant_mode, scale_format, bias_kind, has_tok, activation;
    uint64_t quant_scalar;
    float act_beta;  // SwiGLU
};

struct GemmParams {
    const int8_t* a;
    const int8_t* b;
    uint32_t m, n, k;
    uint32_t b_nz;  // B is in the fractal layout [n/32][k][32] (direct-to-LDS tile kernels only)
    uint32_t tiles_m, tiles_n;
    uint32_t k_splits, k_per_split;  // split-K: bytes of K per grid.z slice (multiple of kBK)
    int32_t* partial;                // split-K int32 accumulator [m, n]
    // grouped
    const int64_t* group_list;
    uint32_t groups;
    int group_list_kind;
    EpiParams epi;
};

struct ChannelQ {
    float s;
    int off9;
    int ctl;  // bit 0: saturate the 8-bit result as signed; bit 1: pre-shift on; bits [5:2]: the pre-shift
};

__device__ __forceinline__ ChannelQ load_channel_q(const EpiParams& e, size_t col)
{
    ChannelQ q{1.0f, 0, 1};
    if (e.quant_mode == ASCQ_MM_QUANT_NONE) {
        return q;
    }
    uint64_t w;
    if (e.quant_mode == ASCQ_MM_QUANT_VECTOR) {
        if (e.scale_format == ASCQ_MM_SCALE_U64) {
            w = static_cast<const uint64_t*>(e.quant)[col];
        } else {
            w = __float_as_uint(static_cast<const float*>(e.quant)[col]);
        }
    } else {
        w = e.quant_scalar;
    }
    uint32_t lo = static_cast<uint32_t>(w);
    if (e.scale_format == ASCQ_MM_SCALE_U64) {
        lo &= 0xFFFFE000u;  // the fixpipe reads sign, 8 exponent and 10 mantissa bits
        q.off9 = static_cast<int>((w >> 37) & 0x1FF);
        // sign bit 46 -> bit 0; mode-control bit 36 -> bit 1; shift bits [35:32] -> bits [5:2]
        q.ctl = static_cast<int>((w >> 46) & 1) | static_cast<int>((w >> 35) & 2) | static_cast<int>((w >> 30) & 0x3C);
    }
    q.s = __uint_as_float(lo);
    return q;
}

// FasterGelu, x * exp(0.851 (x - |x|)) / (1 + exp(-1.702 |x|)) = x / (1 + exp(-1.702 x)): the reference's form keeps
// both exponentials at or below 1 for its vector unit; the quotient form needs one exponential, and its overflow is
// harmless in fp32 (exp -> inf gives 1 / inf = 0, the right limit; exp -> 0 gives x).  The exponential and the
// reciprocal are the hardware's approximations (about one fp32 ulp each), far inside one ulp of the 16-bit outputs
// this activation is used with.
__device__ __forceinline__ float faster_gelu(float x)
{
    const float e = __builtin_amdgcn_exp2f((-1.702f * 1.44269504088896341f) * x);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// SwiGLU of one column pair in fp32, one rounding per step, in the order of the reference's vector instructions
// (Muls by -beta, Exp, Adds 1, Div, Mul: impl/adv_api/detail/activation/swiglu/swiglu_common_impl.h:154-190).
__device__ __forceinline__ float swiglu(float src0, float src1, float beta)
{
    const float t = src1 * (-1.0f * beta);
    const float d = expf(t) + 1.0f;
    return src0 * (src1 / d);
}

// The accumulator as the float the scale multiplies.  A quant word with the mode-control bit set shifts the accumulator
// right (arithmetically) first and saturates the result: to the half range with one rounding to half for half outputs
// (ref: fixpipe_l0c2gm/scripts/gen_data_s322f16.py:84-90), to the int16 range for 8-bit outputs
// (gen_data_s322s8.py:84-86); other outputs take the shifted value as it is.
__device__ __forceinline__ float accumulator_value(int32_t acc, int ctl, int out_dtype)
{
    if (ctl & 2) {
        const int32_t sh = acc >> ((ctl >> 2) & 15);
        if (out_dtype == ASCQ_F16) {
            const float f = fminf(fmaxf(static_cast<float>(sh), -65504.0f), 65504.0f);  // exact below 2^24, monotonic above
            return static_cast<float>(static_cast<_Float16>(f));
        }
        if (out_dtype == ASCQ_I8) {
            return static_cast<float>(min(max(sh, -32768), 32767));
        }
        return static_cast<float>(sh);
    }
    return static_cast<float>(acc);
}

// v of one accumulator before any activation: channel scale, token scale, post-dequant bias.
__device__ __forceinline__ float epilogue_value(const EpiParams& e, int32_t acc, const ChannelQ& q, float tok, float bias_post)
{
    float v = accumulator_value(acc, q.ctl, e.out_dtype) * q.s;
    if (e.has_tok) {
        v = v * tok;
    }
    if (e.bias_kind >= ASCQ_MM_BIAS_F32_POST) {
        v = v + bias_post;
    }
    return v;
}

// Stores one floating-point value of the SwiGLU epilogue (C is [m, n / 2], e.ldc = n / 2).
__device__ __forceinline__ void store_float_out(const EpiParams& e, size_t idx, float v)
{
    if (e.out_dtype == ASCQ_BF16) {
        static_cast<uint16_t*>(e.c)[idx] = static_cast<uint16_t>(f32_to_bf16_bits(v));
    } else if (e.out_dtype == ASCQ_F16) {
        static_cast<uint16_t*>(e.c)[idx] = static_cast<uint16_t>(f32_to_half_bits_sat(v));
    } else {
        static_cast<float*>(e.c)[idx] = v;
    }
}

// Everything after the int32 accumulator, for one output element.  `bias_post` is already widened to fp32.
// kOut is the output dtype, or -1 for "no quantisation" (raw int32).
template <int kOut>
__device__ __forceinline__ void epilogue_store(const EpiParams& e, size_t row, size_t col, int32_t acc,
                                               const ChannelQ& q, float tok, float bias_post)
{
    const size_t idx = row * e.ldc + col;
    if constexpr (kOut < 0) {
        static_cast<int32_t*>(e.c)[idx] = acc;
    } else {
        float v = accumulator_value(acc, q.ctl, kOut) * q.s;
        if (e.has_tok) {
            v = v * tok;
        }
        if (e.bias_kind >= ASCQ_MM_BIAS_F32_POST) {
            v = v + bias_post;
        }
        if (e.activation == ASCQ_MM_ACT_FASTER_GELU) {
            v = faster_gelu(v);
        }
        if constexpr (kOut == ASCQ_BF16) {
            static_cast<uint16_t*>(e.c)[idx] = static_cast<uint16_t>(f32_to_bf16_bits(v));
        } else if constexpr (kOut == ASCQ_F16) {
            static_cast<uint16_t*>(e.c)[idx] = static_cast<uint16_t>(f32_to_half_bits_sat(v));
        } else if constexpr (kOut == ASCQ_F32) {
            static_cast<float*>(e.c)[idx] = v;
        } else {  // int8 / uint8 requantisation
            float r = fminf(fmaxf(__builtin_rintf(v), -256.0f), 255.0f);
            int t = ((v != v) ? 0 : static_cast<int>(r)) + q.off9;
            t = (q.ctl & 1) ? min(max(t, -128), 127) : min(max(t, 0), 255);
            static_cast<uint8_t*>(e.c)[idx] = static_cast<uint8_t>(t);
        }
    }
}

// Calls f(tag) with the compile-time output kind selected by the (uniform) runtime descriptor.
template <int k>
struct OutTag {
    static constexpr int value = k;
};
template <class F>
__device__ __forceinline__ void dispatch_out(const EpiParams& e, F&& f)
{
    if (e.quant_mode == ASCQ_MM_QUANT_NONE) {
        f(OutTag<-1>{});
    } else if (e.out_dtype == ASCQ_BF16) {
        f(OutTag<ASCQ_BF16>{});
    } else if (e.out_dtype == ASCQ_F16) {
        f(OutTag<ASCQ_F16>{});
    } else if (e.out_dtype == ASCQ_F32) {
        f(OutTag<ASCQ_F32>{});
    } else {
        f(OutTag<ASCQ_I8>{});
    }
}

// The whole epilogue of one output element for kernels that hold one element per lane with the columns of a row in
// neighbouring lanes (columns col and col ^ 1 in lanes l and l ^ 1, both active or both not): with SwiGLU the pair
// exchanges its de-quantised values through the neighbouring lane and the even column stores output column col / 2.
__device__ __forceinline__ void epilogue_store_lanes(const EpiParams& e, size_t row, uint32_t col, int32_t acc,
                                                     const ChannelQ& q, float tok, float bias_post)
{
    if (e.activation == ASCQ_MM_ACT_SWIGLU) {  // uniform
        const float v = epilogue_value(e, acc, q, tok, bias_post);
        const float w = __shfl_xor(v, 1, 64);
        if ((col & 1u) == 0u) {
            store_float_out(e, row * e.ldc + (col >> 1), swiglu(v, w, e.act_beta));
        }
        return;
    }
    dispatch_out(e, [&](auto tag) { epilogue_store<decltype(tag)::value>(e, row, col, acc, q, tok, bias_post); });
}

__device__ __forceinline__ float load_bias_post(const EpiParams& e, size_t col)
{
    if (e.bias_kind == ASCQ_MM_BIAS_F32_POST) {
        return static_cast<const float*>(e.bias)[col];
    }
    if (e.bias_kind == ASCQ_MM_BIAS_BF16_POST) {
        return bf16_bits_to_f32(static_cast<const uint16_t*>(e.bias)[col]);
    }
    return 0.0f;
}



// Large-M kernel built on direct-to-LDS loads and transposing LDS reads (matmul_w8a8_dma.hip).
bool gemm_dma_supported(const GemmParams& p);
// b_nk: B is [n][k] (the transposed operand of the plain matmul); not with grouped or fractal B
// b_layout: 0 B is [k, n] (or fractal), 1 [n, k], 2 the layout of ascq_pack_weight_w8
int launch_gemm_dma(GemmParams& p, bool grouped, hipStream_t st, int b_layout = 0);
uint32_t gemm_dma_skinny_splits(uint32_t m, uint32_t n, uint32_t k);
bool gemm_stream_supported(const GemmParams& p);
size_t gemm_stream_workspace(uint32_t m, uint32_t n, uint32_t k);
int launch_gemm_stream(const GemmParams& p, void* workspace, hipStream_t st);
int launch_gemm_dma_skinny(GemmParams& p, void* workspace, size_t workspace_bytes, hipStream_t st, int b_layout = 0);
// Few rows, B as [n][k]: whole columns per workgroup, one launch, no workspace (matmul_w8a8_nk.hip).
bool gemm_nk_supported(const GemmParams& p);
int launch_gemm_nk(const GemmParams& p, hipStream_t st);
// Few rows on weights packed by ascq_pack_weight_w8 (p.b): whole columns per workgroup, one launch, no workspace
// (matmul_w8a8_packed.hip).
bool gemm_packed_supported(const GemmParams& p);
bool gemm_packed_nk_supported(const GemmParams& p);
int launch_gemm_packed(const GemmParams& p, hipStream_t st, bool b_nk = false);
// Rows of one pass of that kernel (16, fewer when k is long).
uint32_t gemm_packed_pass_rows(const GemmParams& p);
// More rows than one such pass takes (on [n, k] weights up to 224): the weights of a workgroup's columns held in
// registers, the activations streamed past them, one launch (k up to 16384).
bool gemm_ws_supported(const GemmParams& p, bool b_nk);
int launch_gemm_ws(const GemmParams& p, hipStream_t st, bool b_nk);
uint32_t gemm_ws_rounds(const GemmParams& p);
// The same kernel with the per-token quantisation of x (half or bfloat16, [m, k]) inside: m <= 8 rows that fit the LDS.
bool gemm_packed_dyn_fits(uint32_t m, uint32_t k, bool b_nk);
int launch_gemm_packed_dyn(const GemmParams& p, const void* x, bool x_bf16, hipStream_t st, bool b_nk);

}  // namespace ascq
