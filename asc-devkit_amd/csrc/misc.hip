// Error string, version, host-side "tiling" size queries, quant-parameter packing and the zero-fill kernel.
#include <algorithm>
#include <cstring>

#include "ascq_common.h"

namespace ascq {

static thread_local char g_error[512] = "";

static thread_local ascq_matmul_plan* g_plan = nullptr;

void plan_begin(ascq_matmul_plan* plan)
{
    std::memset(plan, 0, sizeof(*plan));
    plan->kernel = -1;
    g_plan = plan;
}
void plan_end() { g_plan = nullptr; }
bool plan_recording() { return g_plan != nullptr; }
bool plan_note(int kernel, uint32_t tile_m, uint32_t tile_n, uint32_t tile_k, uint32_t workgroups, uint32_t k_splits,
               uint32_t lds_bytes, size_t workspace_bytes)
{
    if (g_plan == nullptr) {
        return false;
    }
    if (g_plan->kernel < 0) {
        g_plan->kernel = kernel;
        g_plan->tile_m = tile_m;
        g_plan->tile_n = tile_n;
        g_plan->tile_k = tile_k;
        g_plan->workgroups = workgroups;
        g_plan->k_splits = k_splits;
        g_plan->lds_bytes = lds_bytes;
        g_plan->workspace_bytes = workspace_bytes;
    }
    g_plan->launches += 1;
    return true;
}
bool plan_note_extra(uint32_t narrow_tile_n, uint32_t narrow_workgroups)
{
    if (g_plan == nullptr) {
        return false;
    }
    g_plan->narrow_tile_n = narrow_tile_n;
    g_plan->narrow_workgroups = narrow_workgroups;
    return true;
}

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

namespace {
__global__ __launch_bounds__(256) void zero_fill_kernel(uint32_t* p, size_t words)
{
    for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < words;
         i += static_cast<size_t>(gridDim.x) * 256) {
        p[i] = 0u;
    }
}
// int8 [g][k][n] -> fractal [g][n / 32][k][32]: a workgroup moves 64 rows x 128 columns.  A wavefront reads 8 rows x
// 128 bytes (full lines) per instruction and writes, for each of the 4 column panels, the 8 rows x 32 bytes that are
// consecutive in the destination.
__global__ __launch_bounds__(256) void pack_nz_kernel(uint8_t* dst, const uint8_t* src, uint32_t k, uint32_t n)
{
    const uint32_t piece = threadIdx.x & 7u, r0 = threadIdx.x >> 3;
    const uint32_t col = blockIdx.x * 128u + piece * 16u;
    if (col >= n) {
        return;
    }
    const size_t plane = static_cast<size_t>(blockIdx.z) * k * n;
    const uint8_t* s = src + plane + col;
    uint8_t* d = dst + plane + static_cast<size_t>(col >> 5) * k * 32u + (col & 16u);
#pragma unroll
    for (uint32_t i = 0; i < 2u; ++i) {
        const uint32_t row = blockIdx.y * 64u + i * 32u + r0;
        if (row < k) {
            const uint4 v = *reinterpret_cast<const uint4*>(s + static_cast<size_t>(row) * n);
            *reinterpret_cast<uint4*>(d + static_cast<size_t>(row) * 32u) = v;
        }
    }
}
uint64_t shape_size(const uint32_t* shape, uint32_t ndim)
{
    uint64_t s = 1;
    for (uint32_t i = 0; i < ndim; ++i) s *= shape[i];
    return ndim ? s : 0;
}
}  // namespace
}  // namespace ascq

using namespace ascq;

extern "C" const char* ascq_last_error(void) { return g_error; }
extern "C" const char* ascq_version(void) { return "ascq 0.1 (gfx950)"; }

extern "C" int ascq_zero_fill(void* ptr, size_t bytes, void* stream)
{
    ASCQ_REQUIRE(ptr != nullptr || bytes == 0, ASCQ_ENULL, "ascq_zero_fill: ptr is NULL");
    ASCQ_REQUIRE(bytes % 4 == 0 && (reinterpret_cast<uintptr_t>(ptr) & 3u) == 0, ASCQ_EALIGN,
                 "ascq_zero_fill: pointer and size must be multiples of 4 bytes");
    if (bytes == 0) {
        return ASCQ_OK;
    }
    size_t words = bytes / 4;
    size_t blocks = std::min<size_t>((words + 255) / 256, 4096);
    zero_fill_kernel<<<static_cast<uint32_t>(blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<uint32_t*>(ptr), words);
    return launch_status("ascq_zero_fill");
}

// ref: examples/01_simd_cpp_api/05_best_practices/03_fusion_compute/quant_group_matmul_high_performance/scripts/
// gen_data.py:62-64 (weight.reshape([g, k/16, 16, n/32, 32]).transpose([0, 3, 1, 2, 4]))
extern "C" int ascq_pack_weight_nz(uint32_t groups, uint32_t k, uint32_t n, void* dst, const void* src, void* stream)
{
    ASCQ_REQUIRE(dst && src, ASCQ_ENULL, "ascq_pack_weight_nz: dst / src is NULL");
    ASCQ_REQUIRE(groups > 0 && k > 0 && n > 0, ASCQ_EINVAL, "ascq_pack_weight_nz: groups, k, n must be greater than 0");
    ASCQ_REQUIRE(k % 16 == 0 && n % 32 == 0, ASCQ_EINVAL,
                 "ascq_pack_weight_nz: the fractal layout needs k %% 16 == 0 and n %% 32 == 0 (k %u, n %u)", k, n);
    ASCQ_REQUIRE(groups <= 65535u && (k + 63u) / 64u <= 65535u, ASCQ_EUNSUPPORTED,
                 "ascq_pack_weight_nz: at most 65535 groups and k <= 4194240");
    ASCQ_REQUIRE(((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) == 0, ASCQ_EALIGN,
                 "ascq_pack_weight_nz: dst and src must be 16-byte aligned");
    ASCQ_REQUIRE(dst != src, ASCQ_EINVAL, "ascq_pack_weight_nz: dst and src must not be the same buffer");
    const dim3 grid((n + 127u) / 128u, (k + 63u) / 64u, groups);
    pack_nz_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(static_cast<uint8_t*>(dst),
                                                                      static_cast<const uint8_t*>(src), k, n);
    return launch_status("ascq_pack_weight_nz");
}

// Bit layout: docs/zh/api/SIMD-API/基础API/矩阵计算（ISASI）/矩阵计算的搬出/关键特性说明/随路量化.md (tables 1 and 2):
// [31:0] fp32 scale (the hardware reads [31:13]), [45:37] offset, [46] signed result.
extern "C" uint64_t ascq_pack_quant_param(float scale, int32_t offset9, int32_t is_signed)
{
    uint32_t bits;
    std::memcpy(&bits, &scale, 4);
    return static_cast<uint64_t>(bits) | (static_cast<uint64_t>(offset9 & 0x1FF) << 37) |
           (static_cast<uint64_t>(is_signed ? 1 : 0) << 46);
}

// ref: impl/adv_api/tiling/quantization/ascend_quant_tiling_impl.cpp:31-68
extern "C" int ascq_get_ascend_quant_max_min_tmp_size(const uint32_t* shape, uint32_t ndim, uint32_t type_size,
                                                      uint32_t* max_value, uint32_t* min_value)
{
    ASCQ_REQUIRE(shape && max_value && min_value, ASCQ_ENULL, "GetAscendQuantMaxMinTmpSize: NULL argument");
    // Like the reference, a failed check is reported but the sizes are still produced.
    const uint64_t size = shape_size(shape, ndim);
    const uint32_t two_repeats = 2u * 256u;
    uint32_t mx = std::max<uint32_t>(static_cast<uint32_t>(size) * 2u, two_repeats);
    *max_value = (mx + 31u) / 32u * 32u;
    *min_value = two_repeats;
    ASCQ_REQUIRE(size > 0, ASCQ_EINVAL, "[AscendQuant][GetAscendQuantMaxMinTmpSize] Input Shape size must be greater than 0.");
    ASCQ_REQUIRE(size * type_size % 32 == 0, ASCQ_EALIGN,
                 "[AscendQuant][GetAscendQuantMaxMinTmpSize] Input Shape size must be 32B aligned!.");
    ASCQ_REQUIRE(type_size == 2 || type_size == 4, ASCQ_EUNSUPPORTED,
                 "[AscendQuant][GetAscendQuantMaxMinTmpSize] Type size %u is unsupported!", type_size);
    return ASCQ_OK;
}

// ref: impl/adv_api/tiling/quantization/ascend_dequant_tiling_impl.cpp:31-118
extern "C" int ascq_get_ascend_dequant_max_min_tmp_size(const uint32_t* shape, uint32_t ndim, uint32_t type_size,
                                                        uint32_t* max_value, uint32_t* min_value)
{
    ASCQ_REQUIRE(shape && max_value && min_value, ASCQ_ENULL, "GetAscendDequantMaxMinTmpSize: NULL argument");
    ASCQ_REQUIRE(ndim == 1 || ndim == 2, ASCQ_EINVAL,
                 "[AscendDequant][GetAscendDequantMaxMinTmpSize] SrcShape dim %u is unsupported, must be 1 or 2!", ndim);
    const uint32_t outer = ndim == 2 ? shape[0] : 1u;
    const uint32_t inner = ndim == 2 ? shape[1] : shape[0];
    const uint32_t deq_scale = inner + 8u;  // covers a bf16 deqScale padded to 32 bytes
    *max_value = (64u + outer * inner + deq_scale) * 4u;
    *min_value = (64u + inner + deq_scale) * 4u;
    // Like the reference, a failed check is reported but the sizes are still produced.
    ASCQ_REQUIRE(shape_size(shape, ndim) > 0, ASCQ_EINVAL,
                 "[AscendDequant][GetAscendDequantMaxMinTmpSize] Input Shape size must be greater than 0.");
    ASCQ_REQUIRE(type_size == 4, ASCQ_EUNSUPPORTED,
                 "[AscendDequant][GetAscendDequantMaxMinTmpSize] Type size %u is unsupported!", type_size);
    return ASCQ_OK;
}

// ref: impl/adv_api/tiling/quantization/ascend_antiquant_tiling_impl.cpp:70-150 (int8 / int4 sources)
extern "C" int ascq_get_ascend_antiquant_max_min_tmp_size(const uint32_t* src_shape, uint32_t src_ndim,
                                                          const uint32_t* scale_shape, uint32_t scale_ndim,
                                                          int32_t is_transpose, int32_t input_dtype,
                                                          int32_t output_dtype, uint32_t* max_value,
                                                          uint32_t* min_value)
{
    ASCQ_REQUIRE(src_shape && scale_shape && max_value && min_value, ASCQ_ENULL,
                 "GetAscendAntiQuantMaxMinTmpSize: NULL argument");
    ASCQ_REQUIRE(src_ndim == 2, ASCQ_EINVAL, "[AscendAntiQuant] srcShape must be 2-dimensional");
    const uint64_t src_size = shape_size(src_shape, src_ndim);
    ASCQ_REQUIRE(src_size > 0, ASCQ_EINVAL,
                 "[AscendAntiQuant][GetAscendAntiQuantMaxMinTmpSize] Input Shape size must be greater than 0.");
    ASCQ_REQUIRE(input_dtype == ASCQ_I8 || input_dtype == ASCQ_I4, ASCQ_EUNSUPPORTED,
                 "[AscendAntiQuant] input dtype %d", input_dtype);
    if (output_dtype == ASCQ_F16) {
        *max_value = 0;
        *min_value = 0;
        return ASCQ_OK;
    }
    const uint32_t scale_size = static_cast<uint32_t>(std::max<uint64_t>(shape_size(scale_shape, scale_ndim), 1));
    const bool per_channel = scale_size != 1;
    const uint32_t k = src_shape[0];
    const uint32_t transposed = 80u * scale_size * 4u;  // (8 + 8 + 64) * N fp32
    const uint32_t not_transposed = scale_size * 2u * 4u + 64u * k * 4u;
    if (is_transpose && per_channel) {
        *max_value = transposed;
    } else if (!is_transpose && per_channel) {
        *max_value = not_transposed;
    } else {
        *max_value = static_cast<uint32_t>(src_size) * 4u;
    }
    if (!per_channel) {
        *min_value = 1024u;
    } else {
        *min_value = is_transpose ? transposed : not_transposed;
    }
    return ASCQ_OK;
}

// The "factor" queries: a temporary buffer of maxLiveNodeCount * (bytes of the data processed at once) + extraBuf bytes
// serves the operator; host code that carves one shared buffer for several operators sizes it from them.
// ref: impl/adv_api/tiling/quantization/ascend_quant_tiling_impl.cpp:57-61 (GetAscendQuantTmpBufferFactorSize; the
// Quantize form, quantize_tiling_impl.cpp, answers the same)
extern "C" int ascq_get_ascend_quant_tmp_buffer_factor_size(uint32_t* max_live_node_count, uint32_t* extra_buf)
{
    ASCQ_REQUIRE(max_live_node_count && extra_buf, ASCQ_ENULL, "GetAscendQuantTmpBufferFactorSize: NULL argument");
    *max_live_node_count = 2u;
    *extra_buf = 0u;
    return ASCQ_OK;
}

// ref: impl/adv_api/tiling/quantization/ascend_dequant_tiling_impl.cpp:67-81
extern "C" int ascq_get_ascend_dequant_tmp_buffer_factor_size(const uint32_t* shape, uint32_t ndim,
                                                              uint32_t* max_live_node_count, uint32_t* extra_buf)
{
    ASCQ_REQUIRE(max_live_node_count && extra_buf && (shape || ndim == 0), ASCQ_ENULL,
                 "GetAscendDequantTmpBufferFactorSize: NULL argument");
    *extra_buf = 8u + 64u;  // floats per 32-byte block + floats per 256-byte repeat
    if (ndim == 2) {
        *extra_buf += shape[1];
        *max_live_node_count = 1u;
    } else if (ndim == 1) {
        *max_live_node_count = 2u;
    } else {  // the reference answers any other rank with zeros
        *extra_buf = 0u;
        *max_live_node_count = 0u;
    }
    return ASCQ_OK;
}

// ref: impl/adv_api/tiling/quantization/ascend_antiquant_tiling_impl.cpp:145-169 (int8 / int4 and the 4-bit float sources)
extern "C" int ascq_get_ascend_antiquant_tmp_buffer_factor_size(const uint32_t* src_shape, uint32_t src_ndim,
                                                                const uint32_t* scale_shape, uint32_t scale_ndim,
                                                                int32_t is_transpose, int32_t input_format,
                                                                int32_t output_dtype, uint32_t* max_live_node_count,
                                                                uint32_t* extra_buf)
{
    ASCQ_REQUIRE(src_shape && scale_shape && max_live_node_count && extra_buf, ASCQ_ENULL,
                 "GetAscendAntiQuantTmpBufferFactorSize: NULL argument");
    ASCQ_REQUIRE(src_ndim >= 1, ASCQ_EINVAL, "[AscendAntiQuant] srcShape has no dimension");
    *extra_buf = 0u;
    *max_live_node_count = 0u;
    const uint32_t scale_size = static_cast<uint32_t>(std::max<uint64_t>(shape_size(scale_shape, scale_ndim), 1));
    const bool per_channel = scale_size != 1;
    if (input_format == ASCQ_QDST_FP4_E2M1 || input_format == ASCQ_QDST_FP4_E1M2) {
        if (is_transpose) {
            *extra_buf = (scale_size + 31u) / 32u * 32u * 2u;
        }
    } else if (output_dtype == ASCQ_F16) {
        // nothing
    } else if (is_transpose && per_channel) {
        *extra_buf = 80u * scale_size * 4u;
    } else if (!per_channel) {
        *max_live_node_count = 1u;
    } else {
        *extra_buf = scale_size * 2u * 4u + 64u * src_shape[0] * 4u;
    }
    return ASCQ_OK;
}
