// AscendQuant / AscendDequant / AscendAntiQuant and the dynamic per-token quantiser as fused gfx950 kernels.
//
// The reference stages data HBM -> on-chip buffer, runs a chain of vector instructions and copies back; here the
// load, the arithmetic and the store are one kernel.  All four operators are HBM-bandwidth bound: every lane moves
// 16-byte vectors, a wavefront touches 1 KiB of contiguous memory per access, and several rows are kept in flight per
// lane so that enough bytes are outstanding to cover HBM latency.  Parameters that are constant along a row of the
// launch (per-channel scale / offset) are loaded once per lane and reused for all its rows.
#include "ascq_common.h"
#include "ascq_device.h"

namespace ascq {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsInFlight = 4;

// Launch shape of the row-wise vector kernels: blockIdx.x walks the lanes of a row, blockIdx.y groups of rows.  The
// block size (256, 128 or 64) is the one that leaves the fewest idle lanes in a row's last block: 11008 columns at 8
// per lane are 10.75 blocks of 128 but 5.4 of 256, and that mostly empty sixth block cost 8 % of the kernel's time.
struct RowLaunch {
    dim3 grid;
    uint32_t block;
};
inline RowLaunch row_launch(uint32_t lanes, uint32_t rows, uint32_t rows_per_group)
{
    uint32_t block = kThreads;
    for (uint32_t b = kThreads / 2; b >= 64u; b /= 2) {
        if ((lanes + b - 1) / b * b < (lanes + block - 1) / block * block) {
            block = b;
        }
    }
    RowLaunch r{dim3((lanes + block - 1) / block, 1), block};
    const uint32_t row_groups = (rows + rows_per_group - 1) / rows_per_group;
    // enough blocks to fill 256 CUs several times over, but no more row groups than exist
    const uint32_t want = (8192u * (kThreads / block) + r.grid.x - 1) / r.grid.x;
    r.grid.y = row_groups < want ? row_groups : want;
    if (r.grid.y > 65535u) r.grid.y = 65535u;
    return r;
}

// ===================================================================== AscendQuant
struct QuantArgs {
    int8_t* dst;
    const void* src;
    const void* scale;
    const void* offset;
    uint32_t rows, n;
    int policy, offset_kind, k_dim, round_mode;
    float sscale, soffset;
    uint32_t group_size, params_per_row;
    int dst_format;  // ascq_quant_dst
};

// the last step: int8 with the requested rounding, hifloat8 (ties away from zero, saturating), or an 8-bit float
// (always half-even, saturating)
template <bool kRint>
__device__ __forceinline__ int quant_final(float t, const QuantArgs& a)
{
    if (a.dst_format == ASCQ_QDST_I8) {
        return round_sat8<kRint>(t, a.round_mode);
    }
    if (a.dst_format == ASCQ_QDST_HIF8) {
        return static_cast<int>(f32_to_hif8_sat(t));
    }
    if (a.dst_format == ASCQ_QDST_FP4_E2M1 || a.dst_format == ASCQ_QDST_FP4_E1M2) {
        // through bfloat16 (half-even), then the 4-bit float with the requested rounding
        const float b = bf16_bits_to_f32(f32_to_bf16_bits(t));
        return static_cast<int>(a.dst_format == ASCQ_QDST_FP4_E1M2 ? f32_to_fp4_sat<true>(b, a.round_mode)
                                                                   : f32_to_fp4_sat<false>(b, a.round_mode));
    }
    return a.dst_format == ASCQ_QDST_FP8_E5M2 ? f32_to_fp8_sat<true>(t) : f32_to_fp8_sat<false>(t);
}

template <int kPar>
__device__ __forceinline__ void quant_params8(const QuantArgs& a, const void* base, float scalar, uint32_t i,
                                              uint32_t j, float (&p)[8])
{
    float s = scalar;
    switch (a.policy) {
        case ASCQ_PER_CHANNEL: load8<kPar>(base, j, p); return;
        case ASCQ_PER_TOKEN: s = load1<kPar>(base, i); break;
        case ASCQ_PER_GROUP:
            if (a.k_dim == 1) {
                s = load1<kPar>(base, static_cast<size_t>(i) * a.params_per_row + j / a.group_size);
            } else {
                load8<kPar>(base, static_cast<size_t>(i / a.group_size) * a.n + j, p);
                return;
            }
            break;
        default: break;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        p[e] = s;
    }
}

template <int kPar>
__device__ __forceinline__ float quant_param1(const QuantArgs& a, const void* base, float scalar, uint32_t i,
                                              uint32_t j)
{
    switch (a.policy) {
        case ASCQ_PER_CHANNEL: return load1<kPar>(base, j);
        case ASCQ_PER_TOKEN: return load1<kPar>(base, i);
        case ASCQ_PER_GROUP:
            if (a.k_dim == 1) {
                return load1<kPar>(base, static_cast<size_t>(i) * a.params_per_row + j / a.group_size);
            }
            return load1<kPar>(base, static_cast<size_t>(i / a.group_size) * a.n + j);
        default: return scalar;
    }
}

// One lane = 8 consecutive columns; blockIdx.y walks groups of kRowsInFlight rows.  Requires n % 8 == 0 and
// 16-byte aligned tensors.
template <int kSrc, int kPar, int kCt, bool kRint>
__global__ __launch_bounds__(kThreads) void quant_vec_kernel(QuantArgs a)
{
    const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) * 8u;
    if (j >= a.n) {
        return;
    }
    const bool row_params = (a.policy == ASCQ_PER_TOKEN || a.policy == ASCQ_PER_GROUP);
    const bool has_off = a.offset_kind != ASCQ_OFFSET_NONE;
    float s[8], o[8];
    if (!row_params) {
        quant_params8<kPar>(a, a.scale, a.sscale, 0, j, s);
        if (a.offset_kind == ASCQ_OFFSET_TENSOR) {
            quant_params8<kPar>(a, a.offset, a.soffset, 0, j, o);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = a.soffset;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            s[e] = Fmt<kCt>::cvt(s[e]);
            o[e] = Fmt<kCt>::cvt(o[e]);
        }
    }
    for (uint32_t r0 = blockIdx.y * kRowsInFlight; r0 < a.rows; r0 += gridDim.y * kRowsInFlight) {
        float x[kRowsInFlight][8];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            if (r0 + u < a.rows) {
                load8<kSrc, true>(a.src, static_cast<size_t>(r0 + u) * a.n + j, x[u]);  // read once: non-temporal
            }
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t r = r0 + u;
            if (r >= a.rows) {
                break;
            }
            if (row_params) {
                quant_params8<kPar>(a, a.scale, a.sscale, r, j, s);
                if (a.offset_kind == ASCQ_OFFSET_TENSOR) {
                    quant_params8<kPar>(a, a.offset, a.soffset, r, j, o);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) o[e] = a.soffset;
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    s[e] = Fmt<kCt>::cvt(s[e]);
                    o[e] = Fmt<kCt>::cvt(o[e]);
                }
            }
            int q[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float t = Fmt<kCt>::mul(Fmt<kCt>::cvt(x[u][e]), s[e]);
                if (has_off) {
                    t = Fmt<kCt>::add(t, o[e]);
                }
                q[e] = quant_final<kRint>(t, a);
            }
            if (a.dst_format == ASCQ_QDST_FP4_E2M1 || a.dst_format == ASCQ_QDST_FP4_E1M2) {
                // two codes per byte, the even element in the low nibble: 8 columns are one dword
                uint32_t out = 0;
#pragma unroll
                for (int e = 0; e < 8; ++e) out |= static_cast<uint32_t>(q[e]) << (4 * e);
                __builtin_nontemporal_store(
                    out, reinterpret_cast<uint32_t*>(a.dst + (static_cast<size_t>(r) * a.n + j) / 2u));
                continue;
            }
            u32x2 out;
            out[0] = pack4_i8(q[0], q[1], q[2], q[3]);
            out[1] = pack4_i8(q[4], q[5], q[6], q[7]);
            __builtin_nontemporal_store(out, reinterpret_cast<u32x2*>(a.dst + static_cast<size_t>(r) * a.n + j));
        }
    }
}

// Any shape / alignment: one element per lane.
template <int kSrc, int kPar, int kCt>
__global__ __launch_bounds__(kThreads) void quant_scalar_kernel(QuantArgs a)
{
    const size_t total = static_cast<size_t>(a.rows) * a.n;
    for (size_t e = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; e < total;
         e += static_cast<size_t>(gridDim.x) * kThreads) {
        const uint32_t i = static_cast<uint32_t>(e / a.n);
        const uint32_t j = static_cast<uint32_t>(e % a.n);
        float s = Fmt<kCt>::cvt(quant_param1<kPar>(a, a.scale, a.sscale, i, j));
        float t = Fmt<kCt>::mul(Fmt<kCt>::cvt(load1<kSrc>(a.src, e)), s);
        if (a.offset_kind != ASCQ_OFFSET_NONE) {
            float o = (a.offset_kind == ASCQ_OFFSET_TENSOR) ? quant_param1<kPar>(a, a.offset, a.soffset, i, j)
                                                            : a.soffset;
            t = Fmt<kCt>::add(t, Fmt<kCt>::cvt(o));
        }
        a.dst[e] = static_cast<int8_t>(quant_final<false>(t, a));
    }
}

// Fast path of the fp16 contract for half sources (per tensor / per channel): the arithmetic stays in packed half
// registers - v_pk_mul_f16, v_pk_add_f16 (one rounding each), v_rndne_f16, packed clamp, v_cvt_i16_f16 - about five
// VALU operations per element instead of the generic path's conversions through fp32.  NaN inputs give an
// unspecified int8 here (they are outside the operator's defined domain).
__device__ __forceinline__ f16x2 h2_from_bits(uint32_t b)
{
    f16x2 r;
    __builtin_memcpy(&r, &b, 4);
    return r;
}

__device__ __forceinline__ uint32_t quant_h2x2_to_i8x4(f16x2 a, f16x2 b)
{
    const f16x2 lo = {static_cast<half_t>(-128.0f), static_cast<half_t>(-128.0f)};
    const f16x2 hi = {static_cast<half_t>(127.0f), static_cast<half_t>(127.0f)};
    a = __builtin_elementwise_min(__builtin_elementwise_max(__builtin_elementwise_rint(a), lo), hi);
    b = __builtin_elementwise_min(__builtin_elementwise_max(__builtin_elementwise_rint(b), lo), hi);
    const s16x2 ia = __builtin_convertvector(a, s16x2);
    const s16x2 ib = __builtin_convertvector(b, s16x2);
    uint32_t ua, ub;
    __builtin_memcpy(&ua, &ia, 4);
    __builtin_memcpy(&ub, &ib, 4);
    return __builtin_amdgcn_perm(ub, ua, 0x06040200u);  // low bytes of the four 16-bit integers
}

__global__ __launch_bounds__(kThreads) void quant_f16_fast_kernel(QuantArgs a)
{
    const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) * 8u;
    if (j >= a.n) {
        return;
    }
    f16x2 s[4], o[4];
    if (a.policy == ASCQ_PER_CHANNEL) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.scale) + j);
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] = h2_from_bits(v[e]);
    } else {
        const half_t hs = static_cast<half_t>(a.sscale);
#pragma unroll
        for (int e = 0; e < 4; ++e) s[e] = f16x2{hs, hs};
    }
    if (a.offset_kind == ASCQ_OFFSET_TENSOR) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.offset) + j);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = h2_from_bits(v[e]);
    } else {
        // no offset: adding +0 changes nothing that survives the conversion to int8
        const half_t ho = static_cast<half_t>(a.offset_kind == ASCQ_OFFSET_NONE ? 0.0f : a.soffset);
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = f16x2{ho, ho};
    }
    const uint16_t* src = static_cast<const uint16_t*>(a.src);
    for (uint32_t r0 = blockIdx.y * kRowsInFlight; r0 < a.rows; r0 += gridDim.y * kRowsInFlight) {
        u32x4 x[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            if (r0 + u < a.rows) {
                x[u] = __builtin_nontemporal_load(
                    reinterpret_cast<const u32x4*>(src + static_cast<size_t>(r0 + u) * a.n + j));
            }
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            if (r0 + u < a.rows) {
                f16x2 t[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    t[e] = h2_from_bits(x[u][e]) * s[e];  // one rounding
                    t[e] = t[e] + o[e];                    // one rounding
                }
                u32x2 out;
                out[0] = quant_h2x2_to_i8x4(t[0], t[1]);
                out[1] = quant_h2x2_to_i8x4(t[2], t[3]);
                __builtin_nontemporal_store(out, reinterpret_cast<u32x2*>(a.dst + static_cast<size_t>(r0 + u) * a.n + j));
            }
        }
    }
}

template <int kSrc, int kPar, int kCt>
int launch_quant(const QuantArgs& a, bool vec, hipStream_t st)
{
    if (vec) {
        const RowLaunch rl = row_launch(a.n / 8, a.rows, kRowsInFlight);
        const dim3 grid = rl.grid;
        const uint32_t block = rl.block;
        const bool rint = a.round_mode == ASCQ_CAST_RINT || a.round_mode == ASCQ_CAST_NONE;
        if constexpr (kSrc == ASCQ_F16 && kCt == ASCQ_F16) {
            // fp16 contract on a half source: scale / offset are half tensors or scalars
            if (rint && a.dst_format == ASCQ_QDST_I8 &&
                (a.policy == ASCQ_PER_TENSOR || (a.policy == ASCQ_PER_CHANNEL && kPar == ASCQ_F16))) {
                quant_f16_fast_kernel<<<grid, block, 0, st>>>(a);
                return launch_status("ascq_quant");
            }
        }
        if (rint) {
            quant_vec_kernel<kSrc, kPar, kCt, true><<<grid, block, 0, st>>>(a);
        } else {
            quant_vec_kernel<kSrc, kPar, kCt, false><<<grid, block, 0, st>>>(a);
        }
    } else {
        size_t total = static_cast<size_t>(a.rows) * a.n;
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        quant_scalar_kernel<kSrc, kPar, kCt><<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(a);
    }
    return launch_status("ascq_quant");
}

// ============================================================ dynamic per-token quant
template <int kBlock = kThreads>
__device__ __forceinline__ float block_max(float v, float* lds)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v = fmaxf(v, __shfl_xor(v, off, 64));
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        lds[wave] = v;
    }
    __syncthreads();
    float r = lds[0];
#pragma unroll
    for (int w = 1; w < kBlock / 64; ++w) {
        r = fmaxf(r, lds[w]);
    }
    return r;
}

// One workgroup per row; the row stays in registers between the abs-max reduction (wavefront shuffles, then LDS
// across the wavefronts) and the quantisation, so it is read from HBM once.  n % 8 == 0, n <= 8 * kBlock * kVecs.
// Rows of up to 4096 elements run on two wavefronts with up to four vectors per lane: against four wavefronts with
// two, 4.5 against 4.7 us per launch at 2048 rows of 4096 bfloat16 (a conversion without the reduction: 3.7 us).
template <int kSrc, int kVecs, int kBlock = kThreads>
__global__ __launch_bounds__(kBlock) void dynq_row_kernel(int8_t* __restrict__ q, float* __restrict__ ts,
                                                          const void* __restrict__ x, uint32_t n)
{
    constexpr int kThreads = kBlock;  // (shadows the file's constant inside this kernel)
    __shared__ float lds[kThreads / 64];
    const uint32_t row = blockIdx.x;
    float v[kVecs][8];
    float amax = 0.0f;
#pragma unroll
    for (int k = 0; k < kVecs; ++k) {
        const uint32_t j = (k * kThreads + threadIdx.x) * 8u;
        if (j < n) {
            load8<kSrc>(x, static_cast<size_t>(row) * n + j, v[k]);
#pragma unroll
            for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(v[k][e]));
        }
    }
    amax = block_max<kBlock>(amax, lds);
    const bool zero = !(amax > 0.0f);
    const float inv = zero ? 0.0f : 127.0f / amax;
    if (threadIdx.x == 0) {
        ts[row] = zero ? 1.0f : amax / 127.0f;
    }
    // |v * inv| <= 127 (1 + 2^-23) by construction, so the product needs no clamp for finite inputs (the median keeps
    // infinities inside int8; NaN becomes -128).  Adding 1.5 * 2^23 rounds the fp32 product to the nearest integer, ties
    // to even, exactly as rint does (the sum's spacing is 1 and the constant is even), and leaves that integer in two's
    // complement in the low mantissa bits: one add replaces rint, the conversion and the sign handling, and one byte
    // permute per pair gathers the low bytes.
#pragma unroll
    for (int k = 0; k < kVecs; ++k) {
        const uint32_t j = (k * kThreads + threadIdx.x) * 8u;
        if (j < n) {
            uint32_t u[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float t = __builtin_amdgcn_fmed3f(v[k][e] * inv, -128.0f, 127.0f);
                u[e] = __float_as_uint(t + 12582912.0f);
            }
            u32x2 out;
            out[0] = __builtin_amdgcn_perm(u[1], u[0], 0x0c0c0400u) | __builtin_amdgcn_perm(u[3], u[2], 0x04000c0cu);
            out[1] = __builtin_amdgcn_perm(u[5], u[4], 0x0c0c0400u) | __builtin_amdgcn_perm(u[7], u[6], 0x04000c0cu);
            *reinterpret_cast<u32x2*>(q + static_cast<size_t>(row) * n + j) = out;
        }
    }
}

// Any n / alignment: two passes over the row (the second one hits in L2).
template <int kSrc>
__global__ __launch_bounds__(kThreads) void dynq_generic_kernel(int8_t* __restrict__ q, float* __restrict__ ts,
                                                                const void* __restrict__ x, uint32_t n)
{
    __shared__ float lds[kThreads / 64];
    const size_t base = static_cast<size_t>(blockIdx.x) * n;
    float amax = 0.0f;
    for (uint32_t j = threadIdx.x; j < n; j += kThreads) {
        amax = fmaxf(amax, fabsf(load1<kSrc>(x, base + j)));
    }
    amax = block_max(amax, lds);
    const bool zero = !(amax > 0.0f);
    const float inv = zero ? 0.0f : 127.0f / amax;
    if (threadIdx.x == 0) {
        ts[blockIdx.x] = zero ? 1.0f : amax / 127.0f;
    }
    for (uint32_t j = threadIdx.x; j < n; j += kThreads) {
        q[base + j] = static_cast<int8_t>(round_sat8<true>(load1<kSrc>(x, base + j) * inv, 0));
    }
}

template <int kSrc>
int launch_dynq(uint32_t m, uint32_t n, void* q, void* ts, const void* x, hipStream_t st)
{
    int8_t* qq = static_cast<int8_t*>(q);
    float* tt = static_cast<float*>(ts);
    const bool vec = (n % 8 == 0) && aligned16(x) && ((reinterpret_cast<uintptr_t>(q) & 7u) == 0);
    if (vec && n <= 1024) {
        dynq_row_kernel<kSrc, 1, 128><<<m, 128, 0, st>>>(qq, tt, x, n);
    } else if (vec && n <= 2048) {
        dynq_row_kernel<kSrc, 2, 128><<<m, 128, 0, st>>>(qq, tt, x, n);
    } else if (vec && n <= 4096) {
        dynq_row_kernel<kSrc, 4, 128><<<m, 128, 0, st>>>(qq, tt, x, n);
    } else if (vec && n <= 8192) {
        dynq_row_kernel<kSrc, 4><<<m, kThreads, 0, st>>>(qq, tt, x, n);
    } else if (vec && n <= 16384) {
        dynq_row_kernel<kSrc, 8><<<m, kThreads, 0, st>>>(qq, tt, x, n);
    } else {
        dynq_generic_kernel<kSrc><<<m, kThreads, 0, st>>>(qq, tt, x, n);
    }
    return launch_status("ascq_dynamic_quant_per_token");
}

// =================================================================== AscendDequant
struct DequantArgs {
    void* dst;
    const void* src;
    const void* scale;
    uint32_t rows, n, cal, dst_stride;
    int policy, k_dim;
    float sscale;
    uint32_t group_size, params_per_row;
};

template <int kPar>
__device__ __forceinline__ float dequant_param1(const DequantArgs& a, uint32_t i, uint32_t j)
{
    switch (a.policy) {
        case ASCQ_PER_CHANNEL: return load1<kPar>(a.scale, j);
        case ASCQ_PER_TOKEN: return load1<kPar>(a.scale, i);
        case ASCQ_PER_GROUP:
            if (a.k_dim == 1) {
                return load1<kPar>(a.scale, static_cast<size_t>(i) * a.params_per_row + j / a.group_size);
            }
            return load1<kPar>(a.scale, static_cast<size_t>(i / a.group_size) * a.n + j);
        default: return a.sscale;
    }
}

// One lane = 8 consecutive columns (two 16-byte loads of int32, one 16-byte store for 16-bit outputs).
// Columns at or beyond cal are converted but not scaled: multiplying by 1.0f is the identity in fp32.
template <int kSrc, int kPar, int kDst>
__global__ __launch_bounds__(kThreads) void dequant_vec_kernel(DequantArgs a)
{
    const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) * 8u;
    if (j >= a.n) {
        return;
    }
    const bool row_params = (a.policy == ASCQ_PER_TOKEN || a.policy == ASCQ_PER_GROUP);
    float s[8];
    if (!row_params) {
        if (a.policy == ASCQ_PER_CHANNEL && j + 8 <= a.cal) {
            load8<kPar>(a.scale, j, s);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                s[e] = (j + e < a.cal) ? dequant_param1<kPar>(a, 0, j + e) : 1.0f;
            }
        }
    }
    for (uint32_t r0 = blockIdx.y * kRowsInFlight; r0 < a.rows; r0 += gridDim.y * kRowsInFlight) {
        float x[kRowsInFlight][8];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            if (r0 + u < a.rows) {
                load8<kSrc, true>(a.src, static_cast<size_t>(r0 + u) * a.n + j, x[u]);  // read once: non-temporal
            }
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t r = r0 + u;
            if (r >= a.rows) {
                break;
            }
            if (row_params) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    s[e] = (j + e < a.cal) ? dequant_param1<kPar>(a, r, j + e) : 1.0f;
                }
            }
            float y[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) y[e] = x[u][e] * s[e];
            store8<kDst, true>(a.dst, static_cast<size_t>(r) * a.dst_stride + j, y);
        }
    }
}

template <int kSrc, int kPar, int kDst>
__global__ __launch_bounds__(kThreads) void dequant_scalar_kernel(DequantArgs a)
{
    const size_t total = static_cast<size_t>(a.rows) * a.n;
    for (size_t e = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; e < total;
         e += static_cast<size_t>(gridDim.x) * kThreads) {
        const uint32_t i = static_cast<uint32_t>(e / a.n);
        const uint32_t j = static_cast<uint32_t>(e % a.n);
        float v = load1<kSrc>(a.src, e);
        if (j < a.cal) {
            v = v * dequant_param1<kPar>(a, i, j);
        }
        store1<kDst>(a.dst, static_cast<size_t>(i) * a.dst_stride + j, v);
    }
}

template <int kSrc, int kPar, int kDst>
int launch_dequant(const DequantArgs& a, bool vec, hipStream_t st)
{
    if (vec) {
        const RowLaunch rl = row_launch(a.n / 8, a.rows, kRowsInFlight);
        dequant_vec_kernel<kSrc, kPar, kDst><<<rl.grid, rl.block, 0, st>>>(a);
    } else {
        size_t total = static_cast<size_t>(a.rows) * a.n;
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        dequant_scalar_kernel<kSrc, kPar, kDst><<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(a);
    }
    return launch_status("ascq_dequant");
}

template <int kSrc, int kPar>
int dispatch_dequant_dst(int dst, const DequantArgs& a, bool vec, hipStream_t st)
{
    switch (dst) {
        case ASCQ_F16: return launch_dequant<kSrc, kPar, ASCQ_F16>(a, vec, st);
        case ASCQ_BF16: return launch_dequant<kSrc, kPar, ASCQ_BF16>(a, vec, st);
        default: return launch_dequant<kSrc, kPar, ASCQ_F32>(a, vec, st);
    }
}

template <int kSrc>
int dispatch_dequant_par(int par, int dst, const DequantArgs& a, bool vec, hipStream_t st)
{
    switch (par) {
        case ASCQ_F16: return dispatch_dequant_dst<kSrc, ASCQ_F16>(dst, a, vec, st);
        case ASCQ_BF16: return dispatch_dequant_dst<kSrc, ASCQ_BF16>(dst, a, vec, st);
        case ASCQ_U64: return dispatch_dequant_dst<kSrc, ASCQ_U64>(dst, a, vec, st);
        default: return dispatch_dequant_dst<kSrc, ASCQ_F32>(dst, a, vec, st);
    }
}

// ================================================================= AscendAntiQuant
struct AntiQuantArgs {
    void* dst;
    const void* src;
    const void* offset;
    const void* scale;
    uint32_t rows, cols;  // rows x cols of src as laid out in memory
    uint32_t groups, group_size;
    int transpose, has_offset, per_tensor;
    float sscale, soffset;
};

template <int kDst>
__device__ __forceinline__ float antiquant_one(float w, float s, float o, bool has_offset)
{
    // half output: f16(scale * f16(f16(w) + off)); bf16 output: bf16((f32(w) + off) * scale)
    constexpr int kCt = (kDst == ASCQ_F16) ? ASCQ_F16 : ASCQ_F32;
    float t = w;
    if (has_offset) {
        t = Fmt<kCt>::add(t, o);
    }
    return Fmt<kCt>::mul(s, t);
}

// One lane = 16 consecutive source elements of a row (16 bytes of int8 or 8 bytes of int4), 32 bytes of output.
// cols % 16 == 0; in the transposed layout additionally group_size % 16 == 0 so that one parameter covers the lane.
template <int kSrc, int kDst>
__global__ __launch_bounds__(kThreads) void antiquant_vec_kernel(AntiQuantArgs a)
{
    const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) * 16u;
    if (j >= a.cols) {
        return;
    }
    float s[16], o[16];
    uint32_t cached_group = 0xFFFFFFFFu;
    for (uint32_t r0 = blockIdx.y * kRowsInFlight; r0 < a.rows; r0 += gridDim.y * kRowsInFlight) {
        u32x4 raw[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            if (r0 + u < a.rows) {
                const size_t e = static_cast<size_t>(r0 + u) * a.cols + j;
                if constexpr (kSrc == ASCQ_I8) {
                    raw[u] = *reinterpret_cast<const u32x4*>(static_cast<const int8_t*>(a.src) + e);
                } else {
                    u32x2 t = *reinterpret_cast<const u32x2*>(static_cast<const uint8_t*>(a.src) + e / 2);
                    raw[u] = u32x4{t[0], t[1], 0u, 0u};
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t r = r0 + u;
            if (r >= a.rows) {
                break;
            }
            // parameters: a [groups, cols] row (not transposed) or one scalar per (row, group) (transposed)
            const uint32_t g = a.per_tensor ? 0u : (a.transpose ? r * a.groups + j / a.group_size : r / a.group_size);
            if (g != cached_group) {
                cached_group = g;
                if (a.per_tensor) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        s[e] = a.sscale;
                        o[e] = a.soffset;
                    }
                } else if (a.transpose) {
                    const float sv = load1<kDst>(a.scale, g);
                    const float ov = a.has_offset ? load1<kDst>(a.offset, g) : 0.0f;
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        s[e] = sv;
                        o[e] = ov;
                    }
                } else {
                    const size_t pi = static_cast<size_t>(g) * a.cols + j;
                    float t0[8], t1[8];
                    load8<kDst>(a.scale, pi, t0);
                    load8<kDst>(a.scale, pi + 8, t1);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        s[e] = t0[e];
                        s[8 + e] = t1[e];
                    }
                    if (a.has_offset) {
                        load8<kDst>(a.offset, pi, t0);
                        load8<kDst>(a.offset, pi + 8, t1);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            o[e] = t0[e];
                            o[8 + e] = t1[e];
                        }
                    }
                }
            }
            float y0[8], y1[8];
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                int w;
                if constexpr (kSrc == ASCQ_I8) {
                    w = static_cast<int>(static_cast<int8_t>((raw[u][e >> 2] >> (8 * (e & 3))) & 0xFFu));
                } else {
                    const uint32_t nib = (raw[u][e >> 3] >> (4 * (e & 7))) & 0xFu;
                    w = static_cast<int>(nib ^ 8u) - 8;
                }
                const float v = antiquant_one<kDst>(static_cast<float>(w), s[e], o[e], a.has_offset != 0);
                if (e < 8) {
                    y0[e] = v;
                } else {
                    y1[e - 8] = v;
                }
            }
            const size_t oe = static_cast<size_t>(r) * a.cols + j;
            store8<kDst, true>(a.dst, oe, y0);
            store8<kDst, true>(a.dst, oe + 8, y1);
        }
    }
}

template <int kSrc, int kDst>
__global__ __launch_bounds__(kThreads) void antiquant_scalar_kernel(AntiQuantArgs a)
{
    const size_t total = static_cast<size_t>(a.rows) * a.cols;
    for (size_t e = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; e < total;
         e += static_cast<size_t>(gridDim.x) * kThreads) {
        const uint32_t i = static_cast<uint32_t>(e / a.cols);
        const uint32_t j = static_cast<uint32_t>(e % a.cols);
        int w;
        if constexpr (kSrc == ASCQ_I8) {
            w = static_cast<const int8_t*>(a.src)[e];
        } else {
            const uint32_t b = static_cast<const uint8_t*>(a.src)[e >> 1];
            const uint32_t nib = (e & 1) ? (b >> 4) : (b & 0xFu);
            w = static_cast<int>(nib ^ 8u) - 8;
        }
        float s = a.sscale, o = a.soffset;
        if (!a.per_tensor) {
            const size_t pi = a.transpose ? static_cast<size_t>(i) * a.groups + j / a.group_size
                                          : static_cast<size_t>(i / a.group_size) * a.cols + j;
            s = load1<kDst>(a.scale, pi);
            o = a.has_offset ? load1<kDst>(a.offset, pi) : 0.0f;
        }
        store1<kDst>(a.dst, e, antiquant_one<kDst>(static_cast<float>(w), s, o, a.has_offset != 0));
    }
}

// Fast path int8 -> half, [k, n] layout: bytes become halves through the exponent trick (0x6400 | (b ^ 0x80) is
// 1024 + b + 128, minus 1152 is b, both exact), then one rounded packed add of the offset and one rounded packed
// multiply by the scale: about 2.5 VALU operations per element.
template <bool kHasOffset>
__global__ __launch_bounds__(kThreads) void antiquant_i8_f16_fast_kernel(AntiQuantArgs a)
{
    // one lane = 8 columns: 8 bytes in, one 16-byte store out, so that every store instruction of a wavefront writes
    // 1 KiB of consecutive bytes.  The block size is chosen by the host so that the last block of a row is as full
    // as possible.
    const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) * 8u;
    if (j >= a.cols) {
        return;
    }
    constexpr int kRows = 2 * kRowsInFlight;
    const f16x2 k1152 = {static_cast<half_t>(1152.0f), static_cast<half_t>(1152.0f)};
    f16x2 s[4], o[4];
    uint32_t cached_group = 0xFFFFFFFFu;
    const int8_t* src = static_cast<const int8_t*>(a.src);
    uint16_t* dst = static_cast<uint16_t*>(a.dst);
    for (uint32_t r0 = blockIdx.y * kRows; r0 < a.rows; r0 += gridDim.y * kRows) {
        u32x2 raw[kRows];
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
            if (r0 + u < a.rows) {
                raw[u] = __builtin_nontemporal_load(
                    reinterpret_cast<const u32x2*>(src + static_cast<size_t>(r0 + u) * a.cols + j));
            }
        }
#pragma unroll
        for (int u = 0; u < kRows; ++u) {
            const uint32_t r = r0 + u;
            if (r >= a.rows) {
                break;
            }
            const uint32_t g = a.per_tensor ? 0u : r / a.group_size;
            if (g != cached_group) {
                cached_group = g;
                if (a.per_tensor) {
                    const half_t hs = static_cast<half_t>(a.sscale), ho = static_cast<half_t>(a.soffset);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        s[e] = f16x2{hs, hs};
                        o[e] = f16x2{ho, ho};
                    }
                } else {
                    const size_t pi = static_cast<size_t>(g) * a.cols + j;
                    const u32x4 s0 = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.scale) + pi);
#pragma unroll
                    for (int e = 0; e < 4; ++e) s[e] = h2_from_bits(s0[e]);
                    if constexpr (kHasOffset) {
                        const u32x4 o0 = *reinterpret_cast<const u32x4*>(static_cast<const uint16_t*>(a.offset) + pi);
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = h2_from_bits(o0[e]);
                    }
                }
            }
            u32x4 y;
#pragma unroll
            for (int d = 0; d < 2; ++d) {
                const uint32_t x = raw[u][d] ^ 0x80808080u;
                f16x2 lo = h2_from_bits(__builtin_amdgcn_perm(0x64646464u, x, 0x04010400u)) - k1152;  // bytes 0, 1
                f16x2 hi = h2_from_bits(__builtin_amdgcn_perm(0x64646464u, x, 0x04030402u)) - k1152;  // bytes 2, 3
                if constexpr (kHasOffset) {
                    lo = lo + o[2 * d];
                    hi = hi + o[2 * d + 1];
                }
                lo = s[2 * d] * lo;
                hi = s[2 * d + 1] * hi;
                uint32_t blo, bhi;
                __builtin_memcpy(&blo, &lo, 4);
                __builtin_memcpy(&bhi, &hi, 4);
                y[2 * d] = blo;
                y[2 * d + 1] = bhi;
            }
            __builtin_nontemporal_store(y, reinterpret_cast<u32x4*>(dst + static_cast<size_t>(r) * a.cols + j));
        }
    }
}

template <int kSrc, int kDst>
int launch_antiquant(const AntiQuantArgs& a, bool vec, hipStream_t st)
{
    if (vec) {
        // keep the rows of one lane inside as few parameter groups as possible: consecutive row groups per block
        const RowLaunch rl = row_launch(a.cols / 16, a.rows, kRowsInFlight);
        if constexpr (kSrc == ASCQ_I8 && kDst == ASCQ_F16) {
            if (!a.transpose) {
                const RowLaunch fl = row_launch(a.cols / 8, a.rows, 2 * kRowsInFlight);
                if (a.has_offset) {
                    antiquant_i8_f16_fast_kernel<true><<<fl.grid, fl.block, 0, st>>>(a);
                } else {
                    antiquant_i8_f16_fast_kernel<false><<<fl.grid, fl.block, 0, st>>>(a);
                }
                return launch_status("ascq_antiquant");
            }
        }
        antiquant_vec_kernel<kSrc, kDst><<<rl.grid, rl.block, 0, st>>>(a);
    } else {
        size_t total = static_cast<size_t>(a.rows) * a.cols;
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        antiquant_scalar_kernel<kSrc, kDst><<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(a);
    }
    return launch_status("ascq_antiquant");
}

bool ranges_overlap(const void* a, size_t abytes, const void* b, size_t bbytes)
{
    uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + bbytes && b0 < a0 + abytes;
}


// ============================================== AscendAntiQuant PER_TOKEN / PER_GROUP (one-byte sources)
struct AntiQuantPolicyArgs {
    void* dst;
    const uint8_t* src;
    const void* scale;
    const void* offset;
    uint32_t rows, n;
    int policy, along_n, has_offset, src_format;
    uint32_t group_size, params_per_row;
    float sscale, soffset;  // PER_TENSOR
};

// int8 / fp8_e4m3fn / fp8_e5m2 / hifloat8 byte -> fp32 (exact); the OCP 8-bit floats go through the hardware converters
__device__ __forceinline__ float decode_b8(uint32_t word, int byte, int fmt)
{
    const uint32_t b = (word >> (8 * byte)) & 0xFFu;
    if (fmt == ASCQ_QDST_I8) {
        return static_cast<float>(static_cast<int8_t>(b));
    }
    if (fmt == ASCQ_QDST_HIF8) {
        return hif8_to_f32(b);
    }
    return fmt == ASCQ_QDST_FP8_E5M2 ? __builtin_amdgcn_cvt_f32_bf8(static_cast<int>(b), 0)
                                     : __builtin_amdgcn_cvt_f32_fp8(static_cast<int>(b), 0);
}

template <int kPar>
__device__ __forceinline__ void aqp_params8(const AntiQuantPolicyArgs& a, const void* base, bool is_offset, uint32_t i,
                                            uint32_t j, float (&p)[8])
{
    if (a.policy == ASCQ_PER_GROUP && !a.along_n) {
        load8<kPar>(base, static_cast<size_t>(i / a.group_size) * a.n + j, p);
        return;
    }
    if (a.policy == ASCQ_PER_TENSOR) {
        const float s = is_offset ? a.soffset : a.sscale;
#pragma unroll
        for (int e = 0; e < 8; ++e) p[e] = s;
        return;
    }
    const float s = a.policy == ASCQ_PER_TOKEN
                        ? load1<kPar>(base, i)
                        : load1<kPar>(base, static_cast<size_t>(i) * a.params_per_row + j / a.group_size);
#pragma unroll
    for (int e = 0; e < 8; ++e) p[e] = s;
}

// fp32 -> destination with the reference's saturating cast for 16-bit outputs: infinity and everything beyond the
// largest finite value give that value, NaN gives +0
template <int kDst>
__device__ __forceinline__ float aqp_saturate(float v)
{
    if constexpr (kDst == ASCQ_F16) {
        return (v != v) ? 0.0f : fminf(fmaxf(v, -65504.0f), 65504.0f);
    } else if constexpr (kDst == ASCQ_BF16) {
        return (v != v) ? 0.0f : fminf(fmaxf(v, -3.3895313892515355e38f), 3.3895313892515355e38f);
    } else {
        return v;
    }
}

// One lane = 8 consecutive columns.  Requires n % 8 == 0, 8-byte aligned src, 16-byte aligned dst and parameters.
template <int kPar, int kCt, int kDst>
__global__ __launch_bounds__(kThreads) void antiquant_policy_vec_kernel(AntiQuantPolicyArgs a)
{
    const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) * 8u;
    if (j >= a.n) {
        return;
    }
    for (uint32_t r0 = blockIdx.y * kRowsInFlight; r0 < a.rows; r0 += gridDim.y * kRowsInFlight) {
        u32x2 raw[kRowsInFlight];
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            if (r0 + u < a.rows) {
                raw[u] = __builtin_nontemporal_load(
                    reinterpret_cast<const u32x2*>(a.src + static_cast<size_t>(r0 + u) * a.n + j));
            }
        }
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
            const uint32_t r = r0 + u;
            if (r >= a.rows) {
                break;
            }
            float s[8], o[8], v[8];
            aqp_params8<kPar>(a, a.scale, false, r, j, s);
            if (a.has_offset) {
                aqp_params8<kPar>(a, a.offset, true, r, j, o);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float t = decode_b8(raw[u][e >> 2], e & 3, a.src_format);  // exact in every compute type
                if (a.has_offset) {
                    t = Fmt<kCt>::add(t, Fmt<kCt>::cvt(o[e]));
                }
                t = Fmt<kCt>::mul(t, Fmt<kCt>::cvt(s[e]));
                v[e] = kCt == kDst ? t : aqp_saturate<kDst>(t);
            }
            store8<kDst, true>(a.dst, static_cast<size_t>(r) * a.n + j, v);
        }
    }
}

// Any shape / alignment: one element per lane.
template <int kPar, int kCt, int kDst>
__global__ __launch_bounds__(kThreads) void antiquant_policy_scalar_kernel(AntiQuantPolicyArgs a)
{
    const size_t total = static_cast<size_t>(a.rows) * a.n;
    for (size_t e = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; e < total;
         e += static_cast<size_t>(gridDim.x) * kThreads) {
        const uint32_t i = static_cast<uint32_t>(e / a.n), j = static_cast<uint32_t>(e % a.n);
        size_t pi;
        if (a.policy == ASCQ_PER_TOKEN) {
            pi = i;
        } else if (a.along_n) {
            pi = static_cast<size_t>(i) * a.params_per_row + j / a.group_size;
        } else {
            pi = static_cast<size_t>(i / a.group_size) * a.n + j;
        }
        const bool scalar = a.policy == ASCQ_PER_TENSOR;
        float t = decode_b8(a.src[e], 0, a.src_format);
        if (a.has_offset) {
            t = Fmt<kCt>::add(t, Fmt<kCt>::cvt(scalar ? a.soffset : load1<kPar>(a.offset, pi)));
        }
        t = Fmt<kCt>::mul(t, Fmt<kCt>::cvt(scalar ? a.sscale : load1<kPar>(a.scale, pi)));
        store1<kDst>(a.dst, e, kCt == kDst ? t : aqp_saturate<kDst>(t));
    }
}

// fp4 sources with fp8_e8m0 scales (PER_GROUP): one lane = 8 columns (4 source bytes, 16 bytes out).  The product of
// a 4-bit float and a power of two is exact in fp32 and in bfloat16 (infinity on overflow), so dst(bf16) is that
// product and dst(half) its saturating half-even cast.
__device__ __forceinline__ float fp4_code_to_f32(uint32_t code, bool e1m2)
{
    const uint32_t mag = code & 7u;
    float v;
    if (e1m2) {
        v = static_cast<float>(mag) * 0.25f;  // 0, 0.25 .. 1.75
    } else {
        // e2m1: 0, 0.5, then (1 + m / 2) * 2^(e - 1)
        const uint32_t e = mag >> 1, m = mag & 1u;
        v = e == 0u ? 0.5f * static_cast<float>(m)
                    : (1.0f + 0.5f * static_cast<float>(m)) * static_cast<float>(1u << (e - 1u));
    }
    return (code & 8u) ? -v : v;
}
__device__ __forceinline__ float e8m0_to_f32(uint32_t code)
{
    // 2^(code - 127): the code is the fp32 exponent field; 0 is 2^-127 (a subnormal), 255 is NaN
    const uint32_t bits = code == 0u ? 0x00400000u : (code == 255u ? 0x7FC00000u : code << 23);
    return __uint_as_float(bits);
}
template <int kDst>
__global__ __launch_bounds__(kThreads) void antiquant_fp4_kernel(AntiQuantPolicyArgs a)
{
    const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) * 8u;
    if (j >= a.n) {
        return;
    }
    const bool e1m2 = a.src_format == ASCQ_QDST_FP4_E1M2;
    const uint8_t* sc = static_cast<const uint8_t*>(a.scale);
    for (uint32_t r = blockIdx.y; r < a.rows; r += gridDim.y) {
        const uint32_t raw = __builtin_nontemporal_load(
            reinterpret_cast<const uint32_t*>(a.src + (static_cast<size_t>(r) * a.n + j) / 2u));
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const size_t pi = a.along_n ? static_cast<size_t>(r) * a.params_per_row + (j + e) / a.group_size
                                        : static_cast<size_t>(r / a.group_size) * a.n + j + e;
            const float p = fp4_code_to_f32((raw >> (4 * e)) & 15u, e1m2) * e8m0_to_f32(sc[pi]);
            v[e] = kDst == ASCQ_F16 ? aqp_saturate<ASCQ_F16>(p) : p;
        }
        store8<kDst, true>(a.dst, static_cast<size_t>(r) * a.n + j, v);
    }
}

template <int kPar, int kCt, int kDst>
int launch_antiquant_policy(const AntiQuantPolicyArgs& a, bool vec, hipStream_t st)
{
    if (vec) {
        const RowLaunch rl = row_launch(a.n / 8, a.rows, kRowsInFlight);
        antiquant_policy_vec_kernel<kPar, kCt, kDst><<<rl.grid, rl.block, 0, st>>>(a);
    } else {
        size_t blocks = (static_cast<size_t>(a.rows) * a.n + kThreads - 1) / kThreads;
        if (blocks > 65536) blocks = 65536;
        antiquant_policy_scalar_kernel<kPar, kCt, kDst><<<static_cast<uint32_t>(blocks), kThreads, 0, st>>>(a);
    }
    return launch_status("ascq_antiquant_policy");
}

}  // namespace
}  // namespace ascq

using namespace ascq;

// ------------------------------------------------------------------------------------------------ ascq_quant
// Checks mirror the reference's ASCENDC_ASSERT conditions
// (impl/adv_api/detail/quantization/quant/ascend_quant_common_impl.h:224-278, quant_check_common.h:84-120).
extern "C" int ascq_quant(const ascq_quant_desc* d, void* dst, const void* src, const void* scale, const void* offset,
                          void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_quant: desc is NULL");
    ASCQ_REQUIRE(dst != nullptr && src != nullptr, ASCQ_ENULL, "ascq_quant: dst/src is NULL");
    ASCQ_REQUIRE(d->policy != ASCQ_PER_CHANNEL_PER_GROUP && d->policy != ASCQ_PER_TOKEN_PER_GROUP, ASCQ_EUNSUPPORTED,
                 "ascq_quant: the combined policies PER_CHANNEL_PER_GROUP / PER_TOKEN_PER_GROUP are declared by the reference "
                 "but implemented by none of its operators");
    ASCQ_REQUIRE(d->policy >= ASCQ_PER_TENSOR && d->policy <= ASCQ_PER_GROUP, ASCQ_EINVAL,
                 "ascq_quant: unknown policy %d", d->policy);
    ASCQ_REQUIRE(d->src_dtype == ASCQ_F16 || d->src_dtype == ASCQ_BF16 || d->src_dtype == ASCQ_F32, ASCQ_EUNSUPPORTED,
                 "ascq_quant: src dtype %d is not half / bfloat16 / float", d->src_dtype);
    ASCQ_REQUIRE(d->compute >= ASCQ_COMPUTE_F16 && d->compute <= ASCQ_COMPUTE_F32, ASCQ_EINVAL,
                 "ascq_quant: unknown compute mode %d", d->compute);
    ASCQ_REQUIRE(d->round_mode >= ASCQ_CAST_NONE && d->round_mode <= ASCQ_CAST_TRUNC, ASCQ_EUNSUPPORTED,
                 "ascq_quant: round mode %d is not supported (CAST_ODD belongs to no quantisation operator; CAST_HYBRID, "
                 "for hifloat8 outputs, has no usable specification in the reference)", d->round_mode);
    ASCQ_REQUIRE(d->offset_kind >= ASCQ_OFFSET_NONE && d->offset_kind <= ASCQ_OFFSET_TENSOR, ASCQ_EINVAL,
                 "ascq_quant: unknown offset kind %d", d->offset_kind);
    ASCQ_REQUIRE(d->dst_format >= ASCQ_QDST_I8 && d->dst_format <= ASCQ_QDST_HIF8, ASCQ_EUNSUPPORTED,
                 "ascq_quant: destination format %d is not int8 / fp8_e4m3fn / fp8_e5m2 / fp4_e2m1 / fp4_e1m2 / hifloat8",
                 d->dst_format);
    const bool fp4 = d->dst_format == ASCQ_QDST_FP4_E2M1 || d->dst_format == ASCQ_QDST_FP4_E1M2;
    const bool hif8 = d->dst_format == ASCQ_QDST_HIF8;
    if (fp4) {
        // ref: AscendQuant.md table 4 (the fp4x2 rows), ascend_quant_per_group_3510_impl.h:1383-1385
        ASCQ_REQUIRE(d->policy == ASCQ_PER_GROUP && d->compute == ASCQ_COMPUTE_SCALE_T, ASCQ_EUNSUPPORTED,
                     "ascq_quant: fp4 destinations exist for AscendQuant PER_GROUP only");
        ASCQ_REQUIRE(d->src_dtype != ASCQ_F32, ASCQ_EUNSUPPORTED,
                     "ascq_quant: fp4 destinations take half / bfloat16 sources");
    }
    // ref: ascend_quant_3510_impl.h:69-111 ("pertensor process for int8/hif8 output": the half chain, then the cast)
    ASCQ_REQUIRE(d->dst_format == ASCQ_QDST_I8 || hif8 || d->compute != ASCQ_COMPUTE_F16, ASCQ_EUNSUPPORTED,
                 "ascq_quant: the fp16 contract (AscendQuant per tensor / per channel) has int8 and hifloat8 outputs only");
    const bool tensor_scale = d->policy != ASCQ_PER_TENSOR;
    int par = tensor_scale ? d->scale_dtype : ASCQ_F32;
    if (tensor_scale) {
        ASCQ_REQUIRE(scale != nullptr, ASCQ_ENULL, "ascq_quant: scale tensor is NULL");
        ASCQ_REQUIRE(par == ASCQ_F16 || par == ASCQ_BF16 || par == ASCQ_F32, ASCQ_EUNSUPPORTED,
                     "ascq_quant: scale dtype %d is not half / bfloat16 / float", par);
        ASCQ_REQUIRE(d->n > 0, ASCQ_EINVAL, "ascq_quant: n (scaleCount) must be greater than 0");
        ASCQ_REQUIRE(d->cal_count % d->n == 0, ASCQ_EINVAL,
                     "ascq_quant: calCount %u must be an integer multiple of n (scaleCount) %u", d->cal_count, d->n);
    } else {
        ASCQ_REQUIRE(d->offset_kind != ASCQ_OFFSET_TENSOR, ASCQ_EINVAL,
                     "ascq_quant: PER_TENSOR takes a scalar offset");
    }
    if (d->offset_kind == ASCQ_OFFSET_TENSOR) {
        ASCQ_REQUIRE(offset != nullptr, ASCQ_ENULL, "ascq_quant: offset tensor is NULL");
    }
    if (d->compute == ASCQ_COMPUTE_F16) {
        ASCQ_REQUIRE(d->policy == ASCQ_PER_TENSOR || d->policy == ASCQ_PER_CHANNEL, ASCQ_EUNSUPPORTED,
                     "ascq_quant: fp16 compute exists only for PER_TENSOR / PER_CHANNEL");
        ASCQ_REQUIRE(!tensor_scale || par == d->src_dtype, ASCQ_EUNSUPPORTED,
                     "ascq_quant: fp16 compute needs scale dtype == src dtype");
    } else if (tensor_scale) {
        const bool ok = (par == d->src_dtype) || (par == ASCQ_F32 && d->src_dtype != ASCQ_F32);
        ASCQ_REQUIRE(ok, ASCQ_EUNSUPPORTED, "ascq_quant: (src, scale) dtypes (%d, %d) are not a supported pair",
                     d->src_dtype, par);
    }
    uint32_t rows, n;
    uint32_t ppr = 0;
    if (!tensor_scale) {
        rows = 1;
        n = d->cal_count;
    } else {
        n = d->n;
        rows = d->cal_count / n;
        if (d->policy == ASCQ_PER_TOKEN || d->policy == ASCQ_PER_GROUP) {
            ASCQ_REQUIRE(static_cast<uint64_t>(d->m) * n >= d->cal_count, ASCQ_EINVAL,
                         "ascq_quant: calCount %u exceeds m*n = %u*%u", d->cal_count, d->m, n);
            ASCQ_REQUIRE((static_cast<uint64_t>(n) * dtype_size(d->src_dtype)) % 32 == 0, ASCQ_EALIGN,
                         "ascq_quant: a row of n=%u source elements must be a multiple of 32 bytes", n);
        }
        if (d->policy == ASCQ_PER_GROUP) {
            ASCQ_REQUIRE(d->group_size > 0 && d->group_size % 32 == 0, ASCQ_EINVAL,
                         "ascq_quant: groupSize %u must be a positive multiple of 32", d->group_size);
            ASCQ_REQUIRE(d->k_dim == 0 || d->k_dim == 1, ASCQ_EINVAL, "ascq_quant: kDim must be 0 or 1");
            ppr = (n + d->group_size - 1) / d->group_size;
        }
    }
    if (d->cal_count == 0) {
        return ASCQ_OK;
    }
    if (fp4) {
        ASCQ_REQUIRE(n % 8 == 0 && aligned16(src) && aligned16(scale) && (reinterpret_cast<uintptr_t>(dst) & 3u) == 0,
                     ASCQ_EALIGN, "ascq_quant: fp4 destinations need n %% 8 == 0, 16-byte aligned src / scale and a "
                                  "4-byte aligned dst");
    }
    ASCQ_REQUIRE(!ranges_overlap(dst, fp4 ? d->cal_count / 2u : d->cal_count, src,
                                 static_cast<size_t>(d->cal_count) * dtype_size(d->src_dtype)),
                 ASCQ_EINVAL, "ascq_quant: dst overlaps src (in-place operation is not supported on the GPU)");

    // the fp4 path of the reference is not given the offset at all
    const int offset_kind = fp4 ? static_cast<int>(ASCQ_OFFSET_NONE) : d->offset_kind;
    QuantArgs a{static_cast<int8_t*>(dst), src, scale, offset, rows, n, d->policy, offset_kind, d->k_dim,
                d->round_mode, d->scale, d->offset, d->group_size ? d->group_size : 1u, ppr, d->dst_format};
    bool vec = (n % 8 == 0) && aligned16(src) && ((reinterpret_cast<uintptr_t>(dst) & 7u) == 0 || fp4);
    if (tensor_scale) {
        vec = vec && aligned16(scale) && (offset_kind != ASCQ_OFFSET_TENSOR || aligned16(offset));
    }
    if (!tensor_scale && n > 8 * kThreads) {
        // a per-tensor call is a flat array: view it as rows of 2048 when that divides, so the launch is 2-D
        if (n % 2048 == 0) {
            a.rows = n / 2048;
            a.n = 2048;
        }
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int src_dt = d->src_dtype;
#define ASCQ_Q(S, P, C)                                            \
    if (src_dt == (S) && par == (P) && ct == (C)) {                \
        return launch_quant<S, P, C>(a, vec, st);                  \
    }
    // 8-bit float outputs are computed in fp32 whatever the parameter type
    const int ct = d->compute == ASCQ_COMPUTE_F16
                       ? ASCQ_F16
                       : ((d->compute == ASCQ_COMPUTE_F32 || (d->dst_format != ASCQ_QDST_I8 && !fp4 && !hif8)) ? ASCQ_F32 : par);
    if (!tensor_scale) {
        ASCQ_Q(ASCQ_F16, ASCQ_F32, ASCQ_F16)
        ASCQ_Q(ASCQ_BF16, ASCQ_F32, ASCQ_F16)
        ASCQ_Q(ASCQ_F32, ASCQ_F32, ASCQ_F16)
        ASCQ_Q(ASCQ_F16, ASCQ_F32, ASCQ_F32)
        ASCQ_Q(ASCQ_BF16, ASCQ_F32, ASCQ_F32)
        ASCQ_Q(ASCQ_F32, ASCQ_F32, ASCQ_F32)
    } else {
        ASCQ_Q(ASCQ_F16, ASCQ_F16, ASCQ_F16)
        ASCQ_Q(ASCQ_BF16, ASCQ_BF16, ASCQ_F16)
        ASCQ_Q(ASCQ_F32, ASCQ_F32, ASCQ_F16)
        ASCQ_Q(ASCQ_BF16, ASCQ_BF16, ASCQ_BF16)
        ASCQ_Q(ASCQ_F32, ASCQ_F32, ASCQ_F32)
        ASCQ_Q(ASCQ_F16, ASCQ_F32, ASCQ_F32)
        ASCQ_Q(ASCQ_BF16, ASCQ_F32, ASCQ_F32)
        ASCQ_Q(ASCQ_F16, ASCQ_F16, ASCQ_F32)
        ASCQ_Q(ASCQ_BF16, ASCQ_BF16, ASCQ_F32)
    }
#undef ASCQ_Q
    return fail(ASCQ_EUNSUPPORTED, "ascq_quant: no kernel for src %d, scale %d, compute %d", src_dt, par, d->compute);
}

extern "C" int ascq_dynamic_quant_per_token(int32_t src_dtype, uint32_t m, uint32_t n, void* q, void* tok_scale,
                                            const void* x, void* stream)
{
    ASCQ_REQUIRE(q != nullptr && tok_scale != nullptr && x != nullptr, ASCQ_ENULL,
                 "ascq_dynamic_quant_per_token: NULL tensor");
    ASCQ_REQUIRE(n > 0, ASCQ_EINVAL, "ascq_dynamic_quant_per_token: n must be greater than 0");
    if (m == 0) {
        return ASCQ_OK;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (src_dtype) {
        case ASCQ_F16: return launch_dynq<ASCQ_F16>(m, n, q, tok_scale, x, st);
        case ASCQ_BF16: return launch_dynq<ASCQ_BF16>(m, n, q, tok_scale, x, st);
        case ASCQ_F32: return launch_dynq<ASCQ_F32>(m, n, q, tok_scale, x, st);
        default: return fail(ASCQ_EUNSUPPORTED, "ascq_dynamic_quant_per_token: src dtype %d", src_dtype);
    }
}

// ---------------------------------------------------------------------------------------------- ascq_dequant
extern "C" uint32_t ascq_dequant_dst_stride(int32_t dst_dtype, uint32_t n)
{
    const uint32_t per_blk = (dst_dtype == ASCQ_F32) ? 8u : 16u;
    return (n + per_blk - 1) / per_blk * per_blk;
}

// Checks mirror impl/adv_api/detail/quantization/dequant/ascend_dequant_common_impl.h:80-155.
extern "C" int ascq_dequant(const ascq_dequant_desc* d, void* dst, const void* src, const void* scale, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_dequant: desc is NULL");
    ASCQ_REQUIRE(dst != nullptr && src != nullptr, ASCQ_ENULL, "ascq_dequant: dst/src is NULL");
    ASCQ_REQUIRE(d->policy != ASCQ_PER_CHANNEL_PER_GROUP && d->policy != ASCQ_PER_TOKEN_PER_GROUP, ASCQ_EUNSUPPORTED,
                 "ascq_dequant: the combined policies PER_CHANNEL_PER_GROUP / PER_TOKEN_PER_GROUP are declared by the reference "
                 "but implemented by none of its operators");
    ASCQ_REQUIRE(d->policy >= ASCQ_PER_TENSOR && d->policy <= ASCQ_PER_GROUP, ASCQ_EINVAL,
                 "ascq_dequant: unknown policy %d", d->policy);
    ASCQ_REQUIRE(d->dst_dtype == ASCQ_F16 || d->dst_dtype == ASCQ_BF16 || d->dst_dtype == ASCQ_F32,
                 ASCQ_EUNSUPPORTED, "ascq_dequant: dst dtype %d", d->dst_dtype);
    const bool legacy = d->policy <= ASCQ_PER_CHANNEL;
    if (legacy) {
        ASCQ_REQUIRE(d->src_dtype == ASCQ_I32, ASCQ_EUNSUPPORTED, "ascq_dequant: src must be int32");
        if (d->policy == ASCQ_PER_CHANNEL) {
            // deqScale dtype: uint64_t, float, bfloat16_t, bfloat16_t, float
            // dst      dtype: half    , float, float,      bfloat16_t, bfloat16_t
            const int s = d->scale_dtype, t = d->dst_dtype;
            const bool ok = (s == ASCQ_U64 && t == ASCQ_F16) || (s == ASCQ_F32 && t == ASCQ_F32) ||
                            (s == ASCQ_BF16 && t == ASCQ_F32) || (s == ASCQ_BF16 && t == ASCQ_BF16) ||
                            (s == ASCQ_F32 && t == ASCQ_BF16);
            ASCQ_REQUIRE(ok, ASCQ_EUNSUPPORTED,
                         "ascq_dequant: combination of deqScale dtype %d and dst dtype %d is not supported", s, t);
        } else {
            ASCQ_REQUIRE(d->dst_dtype != ASCQ_F16, ASCQ_EUNSUPPORTED,
                         "ascq_dequant: a scalar deqScale supports bfloat16 / float outputs only");
        }
    } else {
        ASCQ_REQUIRE(d->src_dtype == ASCQ_I32 || d->src_dtype == ASCQ_F32, ASCQ_EUNSUPPORTED,
                     "ascq_dequant: src must be int32 or float");
        ASCQ_REQUIRE(d->scale_dtype == ASCQ_F32 || d->scale_dtype == ASCQ_BF16 || d->scale_dtype == ASCQ_F16,
                     ASCQ_EUNSUPPORTED, "ascq_dequant: scale dtype %d", d->scale_dtype);
    }
    if (d->policy != ASCQ_PER_TENSOR) {
        ASCQ_REQUIRE(scale != nullptr, ASCQ_ENULL, "ascq_dequant: scale tensor is NULL");
    }
    ASCQ_REQUIRE(d->n > 0 && d->m > 0, ASCQ_EINVAL, "ascq_dequant: m and n must be greater than 0");
    ASCQ_REQUIRE((d->n * 4u) % 32 == 0, ASCQ_EALIGN, "ascq_dequant: a source row (n=%u int32) must be 32-byte aligned",
                 d->n);
    uint32_t m = d->m, n = d->n, cal = d->cal_count, ppr = 0;
    if (legacy) {
        ASCQ_REQUIRE(d->cal_count <= d->n, ASCQ_EINVAL, "ascq_dequant: calCount %u must not exceed n %u", d->cal_count,
                     d->n);
    } else {
        // the policy form counts elements: the first calCount / n rows are processed, every column of them scaled
        // (ref: impl/adv_api/detail/quantization/dequant/ascend_dequant_3510_impl.h:230, 272, 341, 397, 533, 601)
        ASCQ_REQUIRE(d->cal_count % d->n == 0, ASCQ_EINVAL,
                     "ascq_dequant: calCount %u must be an integer multiple of n %u", d->cal_count, d->n);
        ASCQ_REQUIRE(static_cast<uint64_t>(d->m) * d->n >= d->cal_count, ASCQ_EINVAL,
                     "ascq_dequant: calCount %u exceeds m*n = %u*%u", d->cal_count, d->m, d->n);
        m = d->cal_count / d->n;
        cal = n;
        if (m == 0) {
            return ASCQ_OK;
        }
    }
    if (legacy && d->mode == ASCQ_DEQUANT_WITH_SINGLE_ROW) {
        const uint32_t per_blk = (d->dst_dtype == ASCQ_F32) ? 8u : 16u;
        if (m == 1 && cal != 0 && cal % per_blk == 0 && n % cal == 0) {
            m = n / cal;
            n = cal;
        }
    }
    if (d->policy == ASCQ_PER_GROUP) {
        ASCQ_REQUIRE(d->group_size > 0 && d->group_size % 32 == 0, ASCQ_EINVAL,
                     "ascq_dequant: groupSize %u must be a positive multiple of 32", d->group_size);
        ASCQ_REQUIRE(d->k_dim == 0 || d->k_dim == 1, ASCQ_EINVAL, "ascq_dequant: kDim must be 0 or 1");
        ppr = (n + d->group_size - 1) / d->group_size;
    }
    const uint32_t stride = ascq_dequant_dst_stride(d->dst_dtype, n);
    ASCQ_REQUIRE(!ranges_overlap(dst, static_cast<size_t>(m) * stride * dtype_size(d->dst_dtype), src,
                                 static_cast<size_t>(m) * n * 4),
                 ASCQ_EINVAL, "ascq_dequant: dst overlaps src");
    DequantArgs a{dst, src, scale, m, n, cal, stride, d->policy, d->k_dim, d->scale, d->group_size ? d->group_size : 1u,
                  ppr};
    bool vec = (n % 8 == 0) && aligned16(src) && aligned16(dst) && (stride % 8 == 0);
    if (d->policy == ASCQ_PER_CHANNEL) {
        vec = vec && aligned16(scale);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int par = d->policy == ASCQ_PER_TENSOR ? ASCQ_F32 : d->scale_dtype;
    if (d->src_dtype == ASCQ_F32) {
        return dispatch_dequant_par<ASCQ_F32>(par, d->dst_dtype, a, vec, st);
    }
    return dispatch_dequant_par<ASCQ_I32>(par, d->dst_dtype, a, vec, st);
}

// -------------------------------------------------------------------------------------------- ascq_antiquant
// Checks mirror the reference's parameter rules (docs/zh/api/SIMD-API/高阶API/量化操作/AscendAntiQuant.md:325-328,
// impl/adv_api/tiling/quantization/ascend_antiquant_tiling_impl.cpp:52-68).
extern "C" int ascq_antiquant(const ascq_antiquant_desc* d, void* dst, const void* src, const void* offset,
                              const void* scale, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_antiquant: desc is NULL");
    ASCQ_REQUIRE(dst != nullptr && src != nullptr, ASCQ_ENULL, "ascq_antiquant: dst/src is NULL");
    ASCQ_REQUIRE(d->src_dtype == ASCQ_I8 || d->src_dtype == ASCQ_I4, ASCQ_EUNSUPPORTED,
                 "ascq_antiquant: src dtype %d is not int8 / int4", d->src_dtype);
    ASCQ_REQUIRE(d->dst_dtype == ASCQ_F16 || d->dst_dtype == ASCQ_BF16, ASCQ_EUNSUPPORTED,
                 "ascq_antiquant: dst dtype %d is not half / bfloat16", d->dst_dtype);
    ASCQ_REQUIRE(d->k > 0 && d->n > 0, ASCQ_EINVAL, "ascq_antiquant: k and n must be greater than 0");
    if (!d->per_tensor) {
        ASCQ_REQUIRE(scale != nullptr, ASCQ_ENULL, "ascq_antiquant: scale tensor is NULL");
        ASCQ_REQUIRE(!d->has_offset || offset != nullptr, ASCQ_ENULL, "ascq_antiquant: offset tensor is NULL");
    }
    const uint32_t rows = d->is_transpose ? d->n : d->k;
    const uint32_t cols = d->is_transpose ? d->k : d->n;
    uint32_t groups = d->is_transpose ? d->scale_width : d->scale_height;
    if (groups == 0) {
        groups = 1;
    }
    ASCQ_REQUIRE(d->k % groups == 0, ASCQ_EINVAL, "ascq_antiquant: k %u is not a multiple of the group count %u", d->k,
                 groups);
    if (d->has_offset && !d->per_tensor) {
        const uint32_t og = d->is_transpose ? d->offset_width : d->offset_height;
        ASCQ_REQUIRE(og == 0 || og == groups, ASCQ_EINVAL,
                     "ascq_antiquant: offset and scale shapes differ (%u vs %u groups)", og, groups);
    }
    if (d->is_transpose) {
        const uint32_t kbytes = d->src_dtype == ASCQ_I4 ? d->k / 2 : d->k;
        ASCQ_REQUIRE(kbytes % 32 == 0 && (d->src_dtype != ASCQ_I4 || d->k % 2 == 0), ASCQ_EALIGN,
                     "ascq_antiquant: with isTranspose the k axis must be 32-byte aligned");
    }
    if (d->src_dtype == ASCQ_I4) {
        ASCQ_REQUIRE(cols % 2 == 0, ASCQ_EINVAL, "ascq_antiquant: an int4 row must hold an even number of elements");
    }
    const size_t elems = static_cast<size_t>(rows) * cols;
    ASCQ_REQUIRE(!ranges_overlap(dst, elems * 2, src, d->src_dtype == ASCQ_I4 ? elems / 2 : elems), ASCQ_EINVAL,
                 "ascq_antiquant: dst overlaps src");
    AntiQuantArgs a{dst, src, offset, scale, rows, cols, groups, d->k / groups, d->is_transpose, d->has_offset,
                    d->per_tensor, d->scale, d->offset};
    if (d->per_tensor) {
        // scalars arrive as dstT values
        if (d->dst_dtype == ASCQ_F16) {
            a.sscale = static_cast<float>(static_cast<_Float16>(d->scale));
            a.soffset = static_cast<float>(static_cast<_Float16>(d->offset));
        } else {
            auto rb = [](float f) {
                uint32_t u;
                __builtin_memcpy(&u, &f, 4);
                u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
                __builtin_memcpy(&f, &u, 4);
                return f;
            };
            a.sscale = rb(d->scale);
            a.soffset = rb(d->offset);
        }
    }
    bool vec = (cols % 16 == 0) && aligned16(dst) &&
               ((reinterpret_cast<uintptr_t>(src) & (d->src_dtype == ASCQ_I4 ? 7u : 15u)) == 0);
    if (!d->per_tensor) {
        if (d->is_transpose) {
            vec = vec && (a.group_size % 16 == 0);
        } else {
            vec = vec && aligned16(scale) && (!d->has_offset || aligned16(offset));
        }
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (d->src_dtype == ASCQ_I8) {
        return d->dst_dtype == ASCQ_F16 ? launch_antiquant<ASCQ_I8, ASCQ_F16>(a, vec, st)
                                        : launch_antiquant<ASCQ_I8, ASCQ_BF16>(a, vec, st);
    }
    return d->dst_dtype == ASCQ_F16 ? launch_antiquant<ASCQ_I4, ASCQ_F16>(a, vec, st)
                                    : launch_antiquant<ASCQ_I4, ASCQ_BF16>(a, vec, st);
}

// ------------------------------------------------------------------------------------- ascq_antiquant_policy
// Checks mirror the reference's (impl/adv_api/detail/quantization/antiquant/ascend_antiquant_3510_impl.h:2176-2215).
extern "C" int ascq_antiquant_policy(const ascq_antiquant_policy_desc* d, void* dst, const void* src,
                                     const void* scale, const void* offset, void* stream)
{
    ASCQ_REQUIRE(d != nullptr, ASCQ_ENULL, "ascq_antiquant_policy: desc is NULL");
    const bool per_tensor = d->policy == ASCQ_PER_TENSOR, per_channel = d->policy == ASCQ_PER_CHANNEL;
    ASCQ_REQUIRE(dst != nullptr && src != nullptr && (per_tensor || scale != nullptr), ASCQ_ENULL,
                 "ascq_antiquant_policy: dst / src / scale is NULL");
    ASCQ_REQUIRE(!d->has_offset || per_tensor || offset != nullptr, ASCQ_ENULL,
                 "ascq_antiquant_policy: offset tensor is NULL");
    ASCQ_REQUIRE(d->policy != ASCQ_PER_CHANNEL_PER_GROUP && d->policy != ASCQ_PER_TOKEN_PER_GROUP, ASCQ_EUNSUPPORTED,
                 "ascq_antiquant_policy: the combined policies PER_CHANNEL_PER_GROUP / PER_TOKEN_PER_GROUP are declared by the reference "
                 "but implemented by none of its operators");
    ASCQ_REQUIRE(d->policy >= ASCQ_PER_TENSOR && d->policy <= ASCQ_PER_GROUP, ASCQ_EINVAL,
                 "ascq_antiquant_policy: unknown policy %d", d->policy);
    if (per_tensor || per_channel) {
        // ref: antiquantize_impl.h:42-45 (scale type == dst type, half or bfloat16), 70-110
        ASCQ_REQUIRE(d->compute == ASCQ_COMPUTE_F32, ASCQ_EUNSUPPORTED,
                     "ascq_antiquant_policy: PER_TENSOR / PER_CHANNEL exist for AntiQuantize (fp32 arithmetic) only");
        ASCQ_REQUIRE((d->dst_dtype == ASCQ_F16 || d->dst_dtype == ASCQ_BF16) && d->scale_dtype == d->dst_dtype,
                     ASCQ_EUNSUPPORTED,
                     "ascq_antiquant_policy: PER_TENSOR / PER_CHANNEL take half or bfloat16 parameters of the output's "
                     "type (scale dtype %d, dst dtype %d)", d->scale_dtype, d->dst_dtype);
    }
    ASCQ_REQUIRE(d->src_format >= ASCQ_QDST_I8 && d->src_format <= ASCQ_QDST_HIF8, ASCQ_EUNSUPPORTED,
                 "ascq_antiquant_policy: source format %d is not int8 / fp8_e4m3fn / fp8_e5m2 / fp4_e2m1 / fp4_e1m2 / "
                 "hifloat8", d->src_format);
    if (d->src_format == ASCQ_QDST_FP4_E2M1 || d->src_format == ASCQ_QDST_FP4_E1M2) {
        // ref: AscendAntiQuant.md table 3 (the fp4x2 rows), antiquantize_impl.h:53-58
        ASCQ_REQUIRE(d->policy == ASCQ_PER_GROUP, ASCQ_EUNSUPPORTED,
                     "ascq_antiquant_policy: fp4 sources exist for PER_GROUP only");
        ASCQ_REQUIRE(d->scale_dtype == ASCQ_E8M0 && (d->dst_dtype == ASCQ_F16 || d->dst_dtype == ASCQ_BF16),
                     ASCQ_EUNSUPPORTED,
                     "ascq_antiquant_policy: fp4 sources take fp8_e8m0 scales and give half or bfloat16 (scale dtype "
                     "%d, dst dtype %d)", d->scale_dtype, d->dst_dtype);
        ASCQ_REQUIRE(!d->has_offset, ASCQ_EUNSUPPORTED, "ascq_antiquant_policy: fp4 sources have no offset");
        ASCQ_REQUIRE(d->k_dim == 0 || d->k_dim == 1, ASCQ_EINVAL, "ascq_antiquant_policy: kDim must be 0 or 1");
        ASCQ_REQUIRE(d->group_size > 0 && d->group_size % 32 == 0, ASCQ_EINVAL,
                     "ascq_antiquant_policy: groupSize %u must be a positive multiple of 32", d->group_size);
        ASCQ_REQUIRE(d->n > 0 && d->n % 8 == 0, ASCQ_EALIGN, "ascq_antiquant_policy: fp4 rows need n %% 8 == 0 (n %u)",
                     d->n);
        ASCQ_REQUIRE(d->cal_count % d->n == 0 && static_cast<uint64_t>(d->m) * d->n >= d->cal_count, ASCQ_EINVAL,
                     "ascq_antiquant_policy: calCount %u must be a multiple of n %u and at most m*n", d->cal_count,
                     d->n);
        ASCQ_REQUIRE((reinterpret_cast<uintptr_t>(src) & 3u) == 0 && aligned16(dst), ASCQ_EALIGN,
                     "ascq_antiquant_policy: fp4 sources need a 4-byte aligned src and a 16-byte aligned dst");
        if (d->cal_count == 0) {
            return ASCQ_OK;
        }
        ASCQ_REQUIRE(!ranges_overlap(dst, static_cast<size_t>(d->cal_count) * 2u, src, d->cal_count / 2u), ASCQ_EINVAL,
                     "ascq_antiquant_policy: dst overlaps src");
        const int along = (d->k_dim == 1) != (d->is_transpose != 0) ? 1 : 0;
        AntiQuantPolicyArgs fa{dst, static_cast<const uint8_t*>(src), scale, nullptr, d->cal_count / d->n, d->n,
                               d->policy, along, 0, d->src_format, d->group_size,
                               (d->n + d->group_size - 1) / d->group_size, 0.0f, 0.0f};
        RowLaunch rl = row_launch(d->n / 8, fa.rows, 1);
        hipStream_t fst = static_cast<hipStream_t>(stream);
        if (d->dst_dtype == ASCQ_F16) {
            antiquant_fp4_kernel<ASCQ_F16><<<rl.grid, rl.block, 0, fst>>>(fa);
        } else {
            antiquant_fp4_kernel<ASCQ_BF16><<<rl.grid, rl.block, 0, fst>>>(fa);
        }
        return launch_status("ascq_antiquant_policy");
    }
    const int par = d->scale_dtype, dt = d->dst_dtype;
    ASCQ_REQUIRE(par == ASCQ_F16 || par == ASCQ_BF16 || par == ASCQ_F32, ASCQ_EUNSUPPORTED,
                 "ascq_antiquant_policy: scale dtype %d is not half / bfloat16 / float", par);
    ASCQ_REQUIRE(dt == ASCQ_F16 || dt == ASCQ_BF16 || dt == ASCQ_F32, ASCQ_EUNSUPPORTED,
                 "ascq_antiquant_policy: dst dtype %d is not half / bfloat16 / float", dt);
    ASCQ_REQUIRE(d->compute == ASCQ_COMPUTE_SCALE_T || d->compute == ASCQ_COMPUTE_F32, ASCQ_EINVAL,
                 "ascq_antiquant_policy: compute must be SCALE_T or F32");
    const int ct = d->compute == ASCQ_COMPUTE_F32 ? ASCQ_F32 : par;
    ASCQ_REQUIRE(ct == ASCQ_F32 || dt == ct, ASCQ_EUNSUPPORTED,
                 "ascq_antiquant_policy: with %s arithmetic the output has the same type (dst dtype %d)",
                 ct == ASCQ_F16 ? "half" : "bfloat16", dt);
    ASCQ_REQUIRE(d->n > 0, ASCQ_EINVAL, "ascq_antiquant_policy: n must be greater than 0");
    ASCQ_REQUIRE(d->cal_count % d->n == 0, ASCQ_EINVAL,
                 "ascq_antiquant_policy: calCount %u must be an integer multiple of n %u", d->cal_count, d->n);
    ASCQ_REQUIRE(static_cast<uint64_t>(d->m) * d->n >= d->cal_count, ASCQ_EINVAL,
                 "ascq_antiquant_policy: calCount %u exceeds m*n = %u*%u", d->cal_count, d->m, d->n);
    ASCQ_REQUIRE(d->n % 32 == 0, ASCQ_EALIGN, "ascq_antiquant_policy: a row of n=%u bytes must be a multiple of 32 bytes",
                 d->n);
    int along_n = 1;
    uint32_t ppr = 0;
    if (d->policy == ASCQ_PER_GROUP) {
        ASCQ_REQUIRE(d->k_dim == 0 || d->k_dim == 1, ASCQ_EINVAL, "ascq_antiquant_policy: kDim must be 0 or 1");
        ASCQ_REQUIRE(d->group_size > 0 && d->group_size % 32 == 0, ASCQ_EINVAL,
                     "ascq_antiquant_policy: groupSize %u must be a positive multiple of 32", d->group_size);
        along_n = (d->k_dim == 1) != (d->is_transpose != 0) ? 1 : 0;
        ppr = (d->n + d->group_size - 1) / d->group_size;
    }
    if (d->cal_count == 0) {
        return ASCQ_OK;
    }
    ASCQ_REQUIRE(!ranges_overlap(dst, static_cast<size_t>(d->cal_count) * dtype_size(dt), src, d->cal_count),
                 ASCQ_EINVAL, "ascq_antiquant_policy: dst overlaps src");
    AntiQuantPolicyArgs a{dst, static_cast<const uint8_t*>(src), scale, offset, d->cal_count / d->n, d->n, d->policy,
                          along_n, d->has_offset ? 1 : 0, d->src_format, d->group_size ? d->group_size : 1u, ppr,
                          0.0f, 0.0f};
    if (per_channel) {
        // one parameter row for every data row: a group along m that is never left
        a.policy = ASCQ_PER_GROUP;
        a.along_n = 0;
        a.group_size = 0xFFFFFFFFu;
    }
    if (per_tensor) {
        // the scalars arrive as values of the output type
        auto round_to = [&](float f) {
            if (dt == ASCQ_F16) {
                return static_cast<float>(static_cast<_Float16>(f));
            }
            uint32_t u;
            __builtin_memcpy(&u, &f, 4);
            u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
            __builtin_memcpy(&f, &u, 4);
            return f;
        };
        a.sscale = round_to(d->scale);
        a.soffset = round_to(d->offset);
    }
    const bool vec = (reinterpret_cast<uintptr_t>(src) & 7u) == 0 && aligned16(dst) &&
                     (per_tensor || (aligned16(scale) && (!d->has_offset || aligned16(offset))));
    hipStream_t st = static_cast<hipStream_t>(stream);
#define ASCQ_AQP(P, C, D)                                         \
    if (par == (P) && ct == (C) && dt == (D)) {                   \
        return launch_antiquant_policy<P, C, D>(a, vec, st);      \
    }
    ASCQ_AQP(ASCQ_F16, ASCQ_F16, ASCQ_F16)
    ASCQ_AQP(ASCQ_BF16, ASCQ_BF16, ASCQ_BF16)
    ASCQ_AQP(ASCQ_F32, ASCQ_F32, ASCQ_F32)
    ASCQ_AQP(ASCQ_F32, ASCQ_F32, ASCQ_F16)
    ASCQ_AQP(ASCQ_F32, ASCQ_F32, ASCQ_BF16)
    ASCQ_AQP(ASCQ_F16, ASCQ_F32, ASCQ_F32)
    ASCQ_AQP(ASCQ_F16, ASCQ_F32, ASCQ_F16)
    ASCQ_AQP(ASCQ_F16, ASCQ_F32, ASCQ_BF16)
    ASCQ_AQP(ASCQ_BF16, ASCQ_F32, ASCQ_F32)
    ASCQ_AQP(ASCQ_BF16, ASCQ_F32, ASCQ_F16)
    ASCQ_AQP(ASCQ_BF16, ASCQ_F32, ASCQ_BF16)
#undef ASCQ_AQP
    return fail(ASCQ_EUNSUPPORTED, "ascq_antiquant_policy: no kernel for scale %d, compute %d, dst %d", par, ct, dt);
}
