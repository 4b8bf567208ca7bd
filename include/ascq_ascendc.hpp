// C++ host-side mirror of the reference's operator surface for the quantized-inference path, on top of the C ABI in
// ascq.h.  The reference's operators are `AscendC::` function templates called inside a device kernel on on-chip
// `LocalTensor<T>` views; here the same names, template parameters and argument order act on `DeviceTensor<T>` views
// of HBM buffers and enqueue the fused gfx950 kernel on a HIP stream.
//
//   reference (include/adv_api/quantization/ascend_quant.h:63-762)       this header
//   AscendC::AscendQuant<T>(dst, src, tmp, scale, offset, calCount)      ascq::AscendQuant<T>(dst, src, scale, offset, calCount, stream)
//   AscendC::AscendDequant<dstT, scaleT, mode>(dst, src, deqScale, tmp, params)   ascq::AscendDequant<dstT, scaleT, mode>(dst, src, deqScale, params, stream)
//   AscendC::AscendAntiQuant<In, Out, isTranspose>(dst, src, offset, scale, tmp, k, shapeInfo)   ascq::AscendAntiQuant<...>(dst, src, offset, scale, k, shapeInfo, stream)
//   AscendC::Matmul<...> mm; mm.SetTensorA/B, SetBias, SetQuantScalar/Vector, IterateAll (include/adv_api/matmul/matmul.h:175-185)   ascq::Matmul
//
// Differences a caller sees: there is no `sharedTmpBuffer` argument (the kernels need none); a trailing `stream`
// argument (a hipStream_t as void*, nullptr = default stream) is added; failed argument checks throw `ascq::Error`
// carrying the C ABI's status code and message instead of the reference's log-and-abort in CPU-debug builds.
#ifndef ASCQ_ASCENDC_HPP
#define ASCQ_ASCENDC_HPP

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

#include "ascq.h"

namespace ascq {

class Error : public std::runtime_error {
public:
    Error(int status, const char* what) : std::runtime_error(what ? what : ""), status_(status) {}
    int status() const { return status_; }

private:
    int status_;
};

inline void Check(int status)
{
    if (status != ASCQ_OK) {
        throw Error(status, ascq_last_error());
    }
}

// Storage-only element types: the host never does arithmetic on them.
struct half {
    uint16_t bits;
};
struct bfloat16_t {
    uint16_t bits;
};
struct int4b_t {  // two values per byte, even element in the low nibble
    uint8_t pair;
};
struct fp8_e4m3fn_t {
    uint8_t bits;
};
struct fp8_e5m2_t {
    uint8_t bits;
};
struct hifloat8_t {  // see ASCQ_QDST_HIF8 for the encoding
    uint8_t bits;
};
struct fp8_e8m0_t {  // a power of two: 2^(bits - 127); the scales of the fp4 sources of AscendAntiQuant
    uint8_t bits;
};
struct fp4x2_e2m1_t {  // two 4-bit floats per byte, even element in the low nibble
    uint8_t pair;
};
struct fp4x2_e1m2_t {
    uint8_t pair;
};

// destination types of AscendQuant
template <typename T>
struct QuantDstOf;
template <>
struct QuantDstOf<int8_t> {
    static constexpr int32_t value = ASCQ_QDST_I8;
};
template <>
struct QuantDstOf<fp8_e4m3fn_t> {
    static constexpr int32_t value = ASCQ_QDST_FP8_E4M3FN;
};
template <>
struct QuantDstOf<fp8_e5m2_t> {
    static constexpr int32_t value = ASCQ_QDST_FP8_E5M2;
};
template <>
struct QuantDstOf<hifloat8_t> {
    static constexpr int32_t value = ASCQ_QDST_HIF8;
};
template <>
struct QuantDstOf<fp4x2_e2m1_t> {  // AscendQuant PER_GROUP only
    static constexpr int32_t value = ASCQ_QDST_FP4_E2M1;
};
template <>
struct QuantDstOf<fp4x2_e1m2_t> {
    static constexpr int32_t value = ASCQ_QDST_FP4_E1M2;
};

template <typename T>
struct DTypeOf;
template <>
struct DTypeOf<half> {
    static constexpr int32_t value = ASCQ_F16;
};
template <>
struct DTypeOf<bfloat16_t> {
    static constexpr int32_t value = ASCQ_BF16;
};
template <>
struct DTypeOf<float> {
    static constexpr int32_t value = ASCQ_F32;
};
template <>
struct DTypeOf<int8_t> {
    static constexpr int32_t value = ASCQ_I8;
};
template <>
struct DTypeOf<int4b_t> {
    static constexpr int32_t value = ASCQ_I4;
};
template <>
struct DTypeOf<int32_t> {
    static constexpr int32_t value = ASCQ_I32;
};
template <>
struct DTypeOf<uint64_t> {
    static constexpr int32_t value = ASCQ_U64;
};
template <>
struct DTypeOf<fp8_e8m0_t> {
    static constexpr int32_t value = ASCQ_E8M0;
};

// View of a caller-owned device buffer: the counterpart of LocalTensor / GlobalTensor.  `size` counts elements
// (for int4b_t: values, two per byte).
template <typename T>
class DeviceTensor {
public:
    DeviceTensor() = default;
    DeviceTensor(T* data, uint32_t size) : data_(data), size_(size) {}
    T* GetPhyAddr() const { return data_; }
    uint32_t GetSize() const { return size_; }

private:
    T* data_ = nullptr;
    uint32_t size_ = 0;
};

// ref: include/adv_api/quantization/ascend_quant_utils.h:31-87
enum class RoundMode : int32_t { CAST_NONE = 0, CAST_RINT, CAST_FLOOR, CAST_CEIL, CAST_ROUND, CAST_TRUNC, CAST_ODD, CAST_HYBRID };
// ref: include/adv_api/quantization/ascend_quant_utils.h:73-80 (same members, same values; the two combined policies are
// declared there and implemented by none of the reference's operators: ascq_quant answers ASCQ_EUNSUPPORTED)
enum class AscendQuantPolicy : int32_t { PER_TENSOR, PER_CHANNEL, PER_TOKEN, PER_GROUP, PER_CHANNEL_PER_GROUP, PER_TOKEN_PER_GROUP };
struct AscendQuantConfig {
    bool hasOffset = false;
    int32_t kDim = 1;
    RoundMode roundMode = RoundMode::CAST_RINT;
};
struct AscendQuantParam {
    uint32_t m;
    uint32_t n;
    uint32_t calCount;
    uint32_t groupSize = 0;
};

// Per tensor (ref: ascend_quant.h:63-139).
template <typename T>
void AscendQuant(const DeviceTensor<int8_t>& dstTensor, const DeviceTensor<T>& srcTensor, float scale, float offset,
                 uint32_t calCount, void* stream = nullptr)
{
    ascq_quant_desc d{};
    d.policy = ASCQ_PER_TENSOR;
    d.src_dtype = d.scale_dtype = DTypeOf<T>::value;
    d.compute = ASCQ_COMPUTE_F16;
    d.round_mode = ASCQ_CAST_RINT;
    d.offset_kind = ASCQ_OFFSET_SCALAR;
    d.scale = scale;
    d.offset = offset;
    d.m = 1;
    d.n = d.cal_count = calCount;
    Check(ascq_quant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), nullptr, nullptr, stream));
}

template <typename T>
void AscendQuant(const DeviceTensor<int8_t>& dstTensor, const DeviceTensor<T>& srcTensor, float scale, float offset,
                 void* stream = nullptr)
{
    AscendQuant<T>(dstTensor, srcTensor, scale, offset, srcTensor.GetSize(), stream);
}

// Per channel, scalar offset (ref: ascend_quant.h:159-232); `offset` is given as float and rounded once to T.
template <typename T>
void AscendQuant(const DeviceTensor<int8_t>& dstTensor, const DeviceTensor<T>& srcTensor,
                 const DeviceTensor<T>& scaleTensor, float offset, uint32_t scaleCount, uint32_t calCount,
                 void* stream = nullptr)
{
    ascq_quant_desc d{};
    d.policy = ASCQ_PER_CHANNEL;
    d.src_dtype = d.scale_dtype = DTypeOf<T>::value;
    d.compute = ASCQ_COMPUTE_F16;
    d.round_mode = ASCQ_CAST_RINT;
    d.offset_kind = ASCQ_OFFSET_SCALAR;
    d.offset = offset;
    d.n = scaleCount;
    d.m = scaleCount ? calCount / scaleCount : 0;
    d.cal_count = calCount;
    Check(ascq_quant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scaleTensor.GetPhyAddr(), nullptr, stream));
}

// Per channel, offset tensor (ref: ascend_quant.h:234-347).
template <typename T>
void AscendQuant(const DeviceTensor<int8_t>& dstTensor, const DeviceTensor<T>& srcTensor,
                 const DeviceTensor<T>& scaleTensor, const DeviceTensor<T>& offsetTensor, uint32_t scaleCount,
                 uint32_t offsetCount, uint32_t calCount, void* stream = nullptr)
{
    if (scaleCount != offsetCount) {
        throw Error(ASCQ_EINVAL, "AscendQuant: scaleCount must equal offsetCount");
    }
    ascq_quant_desc d{};
    d.policy = ASCQ_PER_CHANNEL;
    d.src_dtype = d.scale_dtype = DTypeOf<T>::value;
    d.compute = ASCQ_COMPUTE_F16;
    d.round_mode = ASCQ_CAST_RINT;
    d.offset_kind = ASCQ_OFFSET_TENSOR;
    d.n = scaleCount;
    d.m = scaleCount ? calCount / scaleCount : 0;
    d.cal_count = calCount;
    Check(ascq_quant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scaleTensor.GetPhyAddr(),
                     offsetTensor.GetPhyAddr(), stream));
}

// PER_TOKEN / PER_GROUP (ref: ascend_quant.h:667-762): dstT int8_t with the arithmetic in scaleT, or fp8_e4m3fn_t /
// fp8_e5m2_t with fp32 arithmetic.  The reference passes config and policy as template arguments; they are ordinary
// arguments here.
template <typename dstT, typename srcT, typename scaleT>
void AscendQuant(const DeviceTensor<dstT>& dstTensor, const DeviceTensor<srcT>& srcTensor,
                 const DeviceTensor<scaleT>& scaleTensor, const DeviceTensor<scaleT>& offsetTensor,
                 const AscendQuantParam& para, const AscendQuantConfig& config, AscendQuantPolicy policy,
                 void* stream = nullptr)
{
    ascq_quant_desc d{};
    d.policy = static_cast<int32_t>(policy);
    d.src_dtype = DTypeOf<srcT>::value;
    d.scale_dtype = DTypeOf<scaleT>::value;
    d.compute = ASCQ_COMPUTE_SCALE_T;
    d.round_mode = static_cast<int32_t>(config.roundMode);
    d.offset_kind = config.hasOffset ? ASCQ_OFFSET_TENSOR : ASCQ_OFFSET_NONE;
    d.k_dim = config.kDim;
    d.m = para.m;
    d.n = para.n;
    d.cal_count = para.calCount;
    d.group_size = para.groupSize;
    d.dst_format = QuantDstOf<dstT>::value;
    Check(ascq_quant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scaleTensor.GetPhyAddr(),
                     config.hasOffset ? offsetTensor.GetPhyAddr() : nullptr, stream));
}

// ref: include/adv_api/quantization/ascend_dequant_utils.h:26-30, impl/basic_api/utils/kernel_utils_mode.h:181-184
struct DequantParams {
    uint32_t m;
    uint32_t n;
    uint32_t calCount;
};
enum class DeQuantMode : int32_t { DEQUANT_WITH_SINGLE_ROW = 0, DEQUANT_WITH_MULTI_ROW = 1 };

// Tensor scale (ref: ascend_dequant.h:58-175).  dst rows are ascq_dequant_dst_stride(dstT, n) elements apart.
template <typename dstT, typename scaleT, DeQuantMode mode = DeQuantMode::DEQUANT_WITH_SINGLE_ROW>
void AscendDequant(const DeviceTensor<dstT>& dstTensor, const DeviceTensor<int32_t>& srcTensor,
                   const DeviceTensor<scaleT>& deqScale, DequantParams params, void* stream = nullptr)
{
    ascq_dequant_desc d{};
    d.policy = ASCQ_PER_CHANNEL;
    d.src_dtype = ASCQ_I32;
    d.scale_dtype = DTypeOf<scaleT>::value;
    d.dst_dtype = DTypeOf<dstT>::value;
    d.mode = static_cast<int32_t>(mode);
    d.m = params.m;
    d.n = params.n;
    d.cal_count = params.calCount;
    Check(ascq_dequant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), deqScale.GetPhyAddr(), stream));
}

// Scalar scale (ref: ascend_dequant.h:205-281).
template <typename dstT, DeQuantMode mode = DeQuantMode::DEQUANT_WITH_SINGLE_ROW>
void AscendDequant(const DeviceTensor<dstT>& dstTensor, const DeviceTensor<int32_t>& srcTensor, float deqScale,
                   DequantParams params, void* stream = nullptr)
{
    ascq_dequant_desc d{};
    d.policy = ASCQ_PER_TENSOR;
    d.src_dtype = ASCQ_I32;
    d.scale_dtype = ASCQ_F32;
    d.dst_dtype = DTypeOf<dstT>::value;
    d.mode = static_cast<int32_t>(mode);
    d.scale = deqScale;
    d.m = params.m;
    d.n = params.n;
    d.cal_count = params.calCount;
    Check(ascq_dequant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), nullptr, stream));
}

// AscendAntiQuant<dstT, srcT, scaleT, config, policy> for PER_TOKEN / PER_GROUP (ref: ascend_antiquant.h, the
// AscendAntiQuantParam overloads; ascend_antiquant_common.h:45-65): srcT int8_t / fp8_e4m3fn_t / fp8_e5m2_t, the
// arithmetic in scaleT.  config and policy are ordinary arguments here.
struct AscendAntiQuantConfig {
    bool hasOffset = false;
    bool isTranspose = false;
    int32_t kDim = 1;
};
struct AscendAntiQuantParam {
    uint32_t m;
    uint32_t n;
    uint32_t calCount;
    uint32_t groupSize = 0;
};
enum class AscendAntiQuantPolicy : int32_t { PER_TENSOR, PER_CHANNEL, PER_TOKEN, PER_GROUP };

template <typename dstT, typename srcT, typename scaleT>
void AscendAntiQuant(const DeviceTensor<dstT>& dstTensor, const DeviceTensor<srcT>& srcTensor,
                     const DeviceTensor<scaleT>& scaleTensor, const DeviceTensor<scaleT>& offsetTensor,
                     const AscendAntiQuantParam& para, const AscendAntiQuantConfig& config,
                     AscendAntiQuantPolicy policy, void* stream = nullptr)
{
    ascq_antiquant_policy_desc d{};
    d.policy = static_cast<int32_t>(policy);
    d.src_format = QuantDstOf<srcT>::value;
    d.scale_dtype = DTypeOf<scaleT>::value;
    d.dst_dtype = DTypeOf<dstT>::value;
    d.compute = ASCQ_COMPUTE_SCALE_T;
    d.has_offset = config.hasOffset ? 1 : 0;
    d.is_transpose = config.isTranspose ? 1 : 0;
    d.k_dim = config.kDim;
    d.m = para.m;
    d.n = para.n;
    d.cal_count = para.calCount;
    d.group_size = para.groupSize;
    Check(ascq_antiquant_policy(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scaleTensor.GetPhyAddr(),
                                config.hasOffset ? offsetTensor.GetPhyAddr() : nullptr, stream));
}

// ---------------------------------------------------------------------------------------------------------------
// AscendDequant<dstT, srcT, scaleT, config, policy> for PER_TOKEN / PER_GROUP (ref: ascend_dequant.h:284-305,
// ascend_dequant_utils.h:32-44); srcT int32_t or float; the offset tensor is accepted and unused, as in the reference.
struct AscendDeQuantConfig {
    bool hasOffset = false;
    int32_t kDim = 1;
};
// ref: include/adv_api/quantization/ascend_dequant_utils.h:37 (same members, same values: PER_TOKEN is 0 here)
enum class AscendDeQuantPolicy : int32_t { PER_TOKEN, PER_GROUP, PER_CHANNEL_PER_GROUP, PER_TOKEN_PER_GROUP };
inline int32_t ToAscqPolicy(AscendDeQuantPolicy p)
{
    switch (p) {
        case AscendDeQuantPolicy::PER_TOKEN: return ASCQ_PER_TOKEN;
        case AscendDeQuantPolicy::PER_GROUP: return ASCQ_PER_GROUP;
        case AscendDeQuantPolicy::PER_CHANNEL_PER_GROUP: return ASCQ_PER_CHANNEL_PER_GROUP;  // rejected by ascq_dequant
        default: return ASCQ_PER_TOKEN_PER_GROUP;                                            // likewise
    }
}
struct AscendDeQuantParam {
    uint32_t m;
    uint32_t n;
    uint32_t calCount;
    uint32_t groupSize = 0;
};
template <typename dstT, typename srcT, typename scaleT>
void AscendDequant(const DeviceTensor<dstT>& dstTensor, const DeviceTensor<srcT>& srcTensor,
                   const DeviceTensor<scaleT>& scaleTensor, const DeviceTensor<scaleT>& /*offsetTensor*/,
                   const AscendDeQuantParam& para, const AscendDeQuantConfig& config, AscendDeQuantPolicy policy,
                   void* stream = nullptr)
{
    ascq_dequant_desc d{};
    d.policy = ToAscqPolicy(policy);
    d.src_dtype = DTypeOf<srcT>::value;
    d.scale_dtype = DTypeOf<scaleT>::value;
    d.dst_dtype = DTypeOf<dstT>::value;
    d.mode = ASCQ_DEQUANT_WITH_MULTI_ROW;
    d.k_dim = config.kDim;
    d.m = para.m;
    d.n = para.n;
    d.cal_count = para.calCount;
    d.group_size = para.groupSize;
    Check(ascq_dequant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scaleTensor.GetPhyAddr(), stream));
}

// ---------------------------------------------------------------------------------------------------------------
// The unified surface: Quantize / Dequantize / AntiQuantize, one config type each with the policy inside
// (ref: include/adv_api/quantization/quantize.h:53-90, quantize_utils.h:32-45; dequantize.h:57-91,
// impl/adv_api/detail/quantization/dequantize/dequantize_common.h:26-45; antiquantize.h:59-95,
// .../antiquantize/antiquantize_common.h:26-45).  The reference passes the config as a template argument; it is an
// ordinary argument here.  Tensor parameters for every policy but PER_TENSOR, which takes scalars.
enum class QuantizePolicy : int32_t { PER_TENSOR, PER_CHANNEL, PER_TOKEN, PER_GROUP };
struct QuantizeConfig {
    QuantizePolicy policy;
    bool hasOffset;
    RoundMode roundMode = RoundMode::CAST_RINT;
    int32_t kDim = 1;
};
struct QuantizeParams {
    uint32_t m;
    uint32_t n;
    uint32_t groupSize = 0;
};
// Always fp32 arithmetic (ref: impl/adv_api/detail/quantization/quantize/quantize_impl.h:641-968).
template <typename DstT, typename SrcT, typename ScaleT>
void Quantize(const DeviceTensor<DstT>& dstTensor, const DeviceTensor<SrcT>& srcTensor,
              const DeviceTensor<ScaleT>& scale, const DeviceTensor<ScaleT>& offset, const QuantizeParams& params,
              const QuantizeConfig& config, void* stream = nullptr)
{
    ascq_quant_desc d{};
    d.policy = static_cast<int32_t>(config.policy);
    d.src_dtype = DTypeOf<SrcT>::value;
    d.scale_dtype = DTypeOf<ScaleT>::value;
    d.compute = ASCQ_COMPUTE_F32;
    d.round_mode = static_cast<int32_t>(config.roundMode);
    d.offset_kind = config.hasOffset ? ASCQ_OFFSET_TENSOR : ASCQ_OFFSET_NONE;
    d.k_dim = config.kDim;
    d.m = params.m;
    d.n = params.n;
    d.cal_count = params.m * params.n;
    d.group_size = params.groupSize;
    d.dst_format = QuantDstOf<DstT>::value;
    Check(ascq_quant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scale.GetPhyAddr(),
                     config.hasOffset ? offset.GetPhyAddr() : nullptr, stream));
}
template <typename DstT, typename SrcT>
void Quantize(const DeviceTensor<DstT>& dstTensor, const DeviceTensor<SrcT>& srcTensor, float scale, float offset,
              const QuantizeParams& params, const QuantizeConfig& config, void* stream = nullptr)
{
    ascq_quant_desc d{};
    d.policy = ASCQ_PER_TENSOR;
    d.src_dtype = DTypeOf<SrcT>::value;
    d.scale_dtype = DTypeOf<SrcT>::value;
    d.compute = ASCQ_COMPUTE_F32;
    d.round_mode = static_cast<int32_t>(config.roundMode);
    d.offset_kind = config.hasOffset ? ASCQ_OFFSET_SCALAR : ASCQ_OFFSET_NONE;
    d.scale = scale;
    d.offset = offset;
    d.m = params.m;
    d.n = params.n;
    d.cal_count = params.m * params.n;
    d.dst_format = QuantDstOf<DstT>::value;
    Check(ascq_quant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), nullptr, nullptr, stream));
}

enum class DequantizePolicy : int32_t { PER_TENSOR, PER_CHANNEL, PER_TOKEN, PER_GROUP };
struct DequantizeConfig {
    DequantizePolicy policy;
    bool hasOffset = false;  // not supported by the reference either
    int32_t kDim = 1;
};
struct DequantizeParams {
    uint32_t m;
    uint32_t n;
    uint32_t groupSize = 0;
};
// PER_CHANNEL is AscendDequant in DEQUANT_WITH_MULTI_ROW mode on {m, n, n}; PER_TOKEN / PER_GROUP the policy form
// (ref: impl/adv_api/detail/quantization/dequantize/dequantize_impl.h:117-196).
template <typename DstT, typename SrcT, typename ScaleT>
void Dequantize(const DeviceTensor<DstT>& dstTensor, const DeviceTensor<SrcT>& srcTensor,
                const DeviceTensor<ScaleT>& scale, const DeviceTensor<ScaleT>& /*offset*/,
                const DequantizeParams& params, const DequantizeConfig& config, void* stream = nullptr)
{
    ascq_dequant_desc d{};
    d.policy = static_cast<int32_t>(config.policy);
    d.src_dtype = DTypeOf<SrcT>::value;
    d.scale_dtype = DTypeOf<ScaleT>::value;
    d.dst_dtype = DTypeOf<DstT>::value;
    d.mode = ASCQ_DEQUANT_WITH_MULTI_ROW;
    d.k_dim = config.kDim;
    d.m = params.m;
    d.n = params.n;
    d.cal_count = config.policy == DequantizePolicy::PER_CHANNEL ? params.n : params.m * params.n;
    d.group_size = params.groupSize;
    Check(ascq_dequant(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scale.GetPhyAddr(), stream));
}
// PER_TENSOR (ref: dequantize_impl.h:94-115)
template <typename DstT>
void Dequantize(const DeviceTensor<DstT>& dstTensor, const DeviceTensor<int32_t>& srcTensor, float scale,
                float /*offset*/, const DequantizeParams& params, const DequantizeConfig& /*config*/,
                void* stream = nullptr)
{
    AscendDequant<DstT, DeQuantMode::DEQUANT_WITH_MULTI_ROW>(dstTensor, srcTensor, scale,
                                                            DequantParams{params.m, params.n, params.n}, stream);
}

enum class AntiQuantizePolicy : int32_t { PER_TENSOR, PER_CHANNEL, PER_TOKEN, PER_GROUP };
struct AntiQuantizeConfig {
    AntiQuantizePolicy policy;
    bool hasOffset;
    int32_t kDim = 1;
};
struct AntiQuantizeParams {
    uint32_t m;
    uint32_t n;
    uint32_t groupSize = 0;
};
// fp32 arithmetic whatever the parameter type; SrcT int8_t / fp8_e4m3fn_t / fp8_e5m2_t; PER_CHANNEL takes parameters
// [n] of the output's type (ref: impl/adv_api/detail/quantization/antiquantize/antiquantize_impl.h:36-135,
// antiquantize_3510_impl.h:200-362).
template <typename DstT, typename SrcT, typename ScaleT>
void AntiQuantize(const DeviceTensor<DstT>& dstTensor, const DeviceTensor<SrcT>& srcTensor,
                  const DeviceTensor<ScaleT>& scale, const DeviceTensor<ScaleT>& offset,
                  const AntiQuantizeParams& params, const AntiQuantizeConfig& config, void* stream = nullptr)
{
    ascq_antiquant_policy_desc d{};
    d.policy = static_cast<int32_t>(config.policy);
    d.src_format = QuantDstOf<SrcT>::value;
    d.scale_dtype = DTypeOf<ScaleT>::value;
    d.dst_dtype = DTypeOf<DstT>::value;
    d.compute = ASCQ_COMPUTE_F32;
    d.has_offset = config.hasOffset ? 1 : 0;
    d.k_dim = config.kDim;
    d.m = params.m;
    d.n = params.n;
    d.cal_count = params.m * params.n;
    d.group_size = params.groupSize;
    Check(ascq_antiquant_policy(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), scale.GetPhyAddr(),
                                config.hasOffset ? offset.GetPhyAddr() : nullptr, stream));
}
// PER_TENSOR: the scalars are values of the output's type (ref: antiquantize_3510_impl.h:253-302).
template <typename DstT, typename SrcT>
void AntiQuantize(const DeviceTensor<DstT>& dstTensor, const DeviceTensor<SrcT>& srcTensor, float scale, float offset,
                  const AntiQuantizeParams& params, const AntiQuantizeConfig& config, void* stream = nullptr)
{
    ascq_antiquant_policy_desc d{};
    d.policy = ASCQ_PER_TENSOR;
    d.src_format = QuantDstOf<SrcT>::value;
    d.scale_dtype = DTypeOf<DstT>::value;
    d.dst_dtype = DTypeOf<DstT>::value;
    d.compute = ASCQ_COMPUTE_F32;
    d.has_offset = config.hasOffset ? 1 : 0;
    d.m = params.m;
    d.n = params.n;
    d.cal_count = params.m * params.n;
    d.scale = scale;
    d.offset = offset;
    Check(ascq_antiquant_policy(&d, dstTensor.GetPhyAddr(), srcTensor.GetPhyAddr(), nullptr, nullptr, stream));
}

// ref: include/adv_api/quantization/ascend_antiquant_utils.h:27-32
struct AntiQuantShapeInfo {
    uint32_t offsetHeight{0};
    uint32_t offsetWidth{0};
    uint32_t scaleHeight{0};
    uint32_t scaleWidth{0};
};

// Offset and scale tensors (ref: ascend_antiquant.h:46-134).  src is [k, n] (or [n, k] when isTranspose); n is derived
// from the source size as the reference derives it from the tensor's shape.
template <typename InputDataType, typename OutputDataType, bool isTranspose>
void AscendAntiQuant(const DeviceTensor<OutputDataType>& dst, const DeviceTensor<InputDataType>& src,
                     const DeviceTensor<OutputDataType>& offset, const DeviceTensor<OutputDataType>& scale, uint32_t k,
                     const AntiQuantShapeInfo& shapeInfo = {}, void* stream = nullptr)
{
    ascq_antiquant_desc d{};
    d.src_dtype = DTypeOf<InputDataType>::value;
    d.dst_dtype = DTypeOf<OutputDataType>::value;
    d.is_transpose = isTranspose ? 1 : 0;
    d.has_offset = 1;
    d.k = k;
    d.n = k ? src.GetSize() / k : 0;
    d.offset_height = shapeInfo.offsetHeight;
    d.offset_width = shapeInfo.offsetWidth;
    d.scale_height = shapeInfo.scaleHeight;
    d.scale_width = shapeInfo.scaleWidth;
    Check(ascq_antiquant(&d, dst.GetPhyAddr(), src.GetPhyAddr(), offset.GetPhyAddr(), scale.GetPhyAddr(), stream));
}

// Scale only (ref: ascend_antiquant.h:136-210).
template <typename InputDataType, typename OutputDataType, bool isTranspose>
void AscendAntiQuant(const DeviceTensor<OutputDataType>& dst, const DeviceTensor<InputDataType>& src,
                     const DeviceTensor<OutputDataType>& scale, uint32_t k, const AntiQuantShapeInfo& shapeInfo = {},
                     void* stream = nullptr)
{
    ascq_antiquant_desc d{};
    d.src_dtype = DTypeOf<InputDataType>::value;
    d.dst_dtype = DTypeOf<OutputDataType>::value;
    d.is_transpose = isTranspose ? 1 : 0;
    d.has_offset = 0;
    d.k = k;
    d.n = k ? src.GetSize() / k : 0;
    d.scale_height = shapeInfo.scaleHeight;
    d.scale_width = shapeInfo.scaleWidth;
    Check(ascq_antiquant(&d, dst.GetPhyAddr(), src.GetPhyAddr(), nullptr, scale.GetPhyAddr(), stream));
}

// Scalar offset and scale (ref: ascend_antiquant.h:211-262); the scalars are given as float and rounded once to
// OutputDataType.
template <typename InputDataType, typename OutputDataType, bool isTranspose>
void AscendAntiQuant(const DeviceTensor<OutputDataType>& dst, const DeviceTensor<InputDataType>& src, float offset,
                     float scale, uint32_t k, void* stream = nullptr)
{
    ascq_antiquant_desc d{};
    d.src_dtype = DTypeOf<InputDataType>::value;
    d.dst_dtype = DTypeOf<OutputDataType>::value;
    d.is_transpose = isTranspose ? 1 : 0;
    d.has_offset = 1;
    d.per_tensor = 1;
    d.scale = scale;
    d.offset = offset;
    d.k = k;
    d.n = k ? src.GetSize() / k : 0;
    Check(ascq_antiquant(&d, dst.GetPhyAddr(), src.GetPhyAddr(), nullptr, nullptr, stream));
}

// Memory layout of a matrix operand, as the CubeFormat argument of the reference's MatmulType.
enum class CubeFormat : int32_t { ND = 0, NZ = 1 };

// The int8 Matmul object with the quant epilogue (ref: include/adv_api/matmul/matmul.h:138-185; the quant parameters
// are consumed at copy-out, impl/adv_api/detail/matmul/stage/copy_cube_out/quant/quant_processor_fixpipe.h:74-222).
// CType selects the output: int32_t (no quant), half / bfloat16_t / float / int8_t (quant epilogue).

// ABType: int8_t, or int4b_t for Matmul<int4b_t, int4b_t, C> (both operands two values per byte; the workspace is
// then mandatory, no transposed A, ND only;
// ref: examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_int4/matmul_int4.asc:52-58).
template <typename CType, typename ABType = int8_t>
class Matmul {
    static_assert(std::is_same<ABType, int8_t>::value || std::is_same<ABType, int4b_t>::value,
                  "Matmul: A and B are int8_t or int4b_t");
    static constexpr bool kInt4 = std::is_same<ABType, int4b_t>::value;

public:
    Matmul(uint32_t m, uint32_t n, uint32_t k)
    {
        desc_ = ascq_matmul_desc{};
        desc_.m = m;
        desc_.n = n;
        desc_.k = k;
        desc_.out_dtype = DTypeOf<CType>::value;
        desc_.quant_mode = ASCQ_MM_QUANT_NONE;
    }
    void SetTensorA(const DeviceTensor<ABType>& a, bool isTransposeA = false)
    {
        a_ = a.GetPhyAddr();
        desc_.trans_a = isTransposeA ? 1 : 0;
    }
    // format: the CubeFormat of the reference's MatmulType for B (ND, or the fractal NZ layout [n/32][k/16][16][32])
    void SetTensorB(const DeviceTensor<ABType>& b, bool isTransposeB = false, CubeFormat format = CubeFormat::ND)
    {
        b_ = b.GetPhyAddr();
        desc_.trans_b = isTransposeB ? 1 : 0;
        desc_.b_format = format == CubeFormat::NZ ? ASCQ_MM_B_NZ : ASCQ_MM_B_ND;
    }
    // B in the layout of ascq_pack_weight_w8 (PackWeightInt8 below), packed once per weight matrix: IterateAll then
    // runs the one-launch decode kernel (up to 16 rows per pass over the weights), with the results of SetTensorB's
    // matmul bit for bit.  No counterpart in the reference (the analogue of its offline ND -> NZ packing).
    void SetTensorBPacked(const void* packed)
    {
        static_assert(!kInt4, "packed weights are int8");
        b_ = packed;
        packed_ = true;
        desc_.trans_b = 0;
        desc_.b_format = ASCQ_MM_B_ND;
    }
    // int32 bias: the accumulator's initial value, as in the reference.
    void SetBias(const DeviceTensor<int32_t>& bias)
    {
        bias_ = bias.GetPhyAddr();
        desc_.bias_kind = ASCQ_MM_BIAS_I32_PRE;
    }
    // fp32 / bf16 bias added after dequantisation (not a reference combination; used by LLM linears).
    void SetBias(const DeviceTensor<float>& bias)
    {
        bias_ = bias.GetPhyAddr();
        desc_.bias_kind = ASCQ_MM_BIAS_F32_POST;
    }
    void SetBias(const DeviceTensor<bfloat16_t>& bias)
    {
        bias_ = bias.GetPhyAddr();
        desc_.bias_kind = ASCQ_MM_BIAS_BF16_POST;
    }
    void DisableBias()
    {
        bias_ = nullptr;
        desc_.bias_kind = ASCQ_MM_BIAS_NONE;
    }
    void SetQuantScalar(uint64_t quantScalar)
    {
        desc_.quant_mode = ASCQ_MM_QUANT_SCALAR;
        desc_.scale_format = ASCQ_MM_SCALE_U64;
        desc_.quant_scalar = quantScalar;
    }
    void SetQuantVector(const DeviceTensor<uint64_t>& quantTensor)
    {
        desc_.quant_mode = ASCQ_MM_QUANT_VECTOR;
        desc_.scale_format = ASCQ_MM_SCALE_U64;
        quant_ = quantTensor.GetPhyAddr();
    }
    // Plain fp32 per-channel scales (all 23 mantissa bits), optionally with per-token scales.
    void SetQuantVector(const DeviceTensor<float>& scaleTensor)
    {
        desc_.quant_mode = ASCQ_MM_QUANT_VECTOR;
        desc_.scale_format = ASCQ_MM_SCALE_F32;
        quant_ = scaleTensor.GetPhyAddr();
    }
    void SetTokenScale(const DeviceTensor<float>& tokScale)
    {
        tok_ = tokScale.GetPhyAddr();
        desc_.has_tok_scale = 1;
    }
    // Fused activation of the dequantised result (no reference counterpart on the Matmul object: the reference applies
    // FasterGelu / SwiGLU as separate vector operators, gelu_impl.h:140-143, swiglu_common_impl.h:154-190).
    // ASCQ_MM_ACT_SWIGLU: columns 2j / 2j + 1 of the product are src0 / src1 and C is [m, n / 2].
    void SetActivation(ascq_mm_activation activation, float beta = 1.0f)
    {
        desc_.activation = activation;
        desc_.act_beta = beta;
    }
    void SetWorkspace(void* workspace, size_t bytes)
    {
        workspace_ = workspace;
        workspace_bytes_ = bytes;
    }
    size_t GetWorkspaceSize() const
    {
        size_t bytes = 0;
        Check(kInt4 ? ascq_matmul_w4a4_workspace_size(&desc_, &bytes)
                    : ascq_matmul_w8a8_workspace_size(&desc_, &bytes));
        return bytes;
    }
    void IterateAll(const DeviceTensor<CType>& c, void* stream = nullptr)
    {
        if (packed_) {
            Check(ascq_matmul_w8a8_packed(&desc_, c.GetPhyAddr(), a_, b_, bias_, quant_, tok_, stream));
            return;
        }
        Check((kInt4 ? ascq_matmul_w4a4 : ascq_matmul_w8a8)(&desc_, c.GetPhyAddr(), a_, b_, bias_, quant_, tok_,
                                                            workspace_, workspace_bytes_, stream));
    }
    // The plan IterateAll(c) would follow; nothing is launched.  The counterpart of the reference's host-side
    // TCubeTiling (include/adv_api/matmul/matmul_tilingdata.h:21-72).
    ascq_matmul_plan GetPlan(const DeviceTensor<CType>& c) const
    {
        static_assert(!kInt4, "the plan query describes the int8 matmul");
        ascq_matmul_plan plan;
        Check(ascq_matmul_w8a8_plan(&desc_, c.GetPhyAddr(), a_, b_, bias_, quant_, tok_, workspace_, workspace_bytes_,
                                    &plan));
        return plan;
    }
    const ascq_matmul_desc& Desc() const { return desc_; }

private:
    ascq_matmul_desc desc_;
    const void* a_ = nullptr;
    const void* b_ = nullptr;
    const void* bias_ = nullptr;
    const void* quant_ = nullptr;
    const void* tok_ = nullptr;
    void* workspace_ = nullptr;
    size_t workspace_bytes_ = 0;
    bool packed_ = false;
};

// Bytes of, and the packing into, the decode layout of int8 weights (b: [k, n], or [n, k] with isTransposeB).
inline size_t PackWeightInt8Size(uint32_t k, uint32_t n)
{
    size_t bytes = 0;
    Check(ascq_pack_weight_w8_size(k, n, &bytes));
    return bytes;
}
inline void PackWeightInt8(const DeviceTensor<int8_t>& b, void* packed, uint32_t k, uint32_t n, bool isTransposeB = false,
                           void* stream = nullptr)
{
    Check(ascq_pack_weight_w8(b.GetPhyAddr(), packed, k, n, isTransposeB ? 1 : 0, stream));
}

// Matmul with A half and B int8 de-quantised on the way in (MatmulType<.., half> x MatmulType<.., int8_t>).
// ref: include/adv_api/matmul/matmul.h:161-168 (SetAntiQuantScalar / SetAntiQuantVector); hasAntiQuantOffset is the
// MatmulConfig field of that name.  CType: half or float.
template <typename CType, bool hasAntiQuantOffset = true>
class AntiQuantMatmul {
public:
    AntiQuantMatmul(uint32_t m, uint32_t n, uint32_t k)
    {
        desc_ = ascq_w8a16_desc{};
        desc_.m = m;
        desc_.n = n;
        desc_.k = k;
        desc_.has_offset = hasAntiQuantOffset ? 1 : 0;
        desc_.out_dtype = DTypeOf<CType>::value;
    }
    void SetTensorA(const DeviceTensor<half>& a) { a_ = a.GetPhyAddr(); }
    // isTransposeB: b is [n, k] (ref: include/adv_api/matmul/matmul.h:129)
    void SetTensorB(const DeviceTensor<int8_t>& b, bool isTransposeB = false)
    {
        b_ = b.GetPhyAddr();
        desc_.trans_b = isTransposeB ? 1 : 0;
    }
    void SetAntiQuantScalar(float offsetScalar, float scaleScalar)
    {
        desc_.per_tensor = 1;
        desc_.offset = offsetScalar;
        desc_.scale = scaleScalar;
    }
    void SetAntiQuantVector(const DeviceTensor<half>& offsetTensor, const DeviceTensor<half>& scaleTensor)
    {
        desc_.per_tensor = 0;
        offset_ = offsetTensor.GetPhyAddr();
        scale_ = scaleTensor.GetPhyAddr();
    }
    void SetWorkspace(void* workspace, size_t bytes)
    {
        workspace_ = workspace;
        workspace_bytes_ = bytes;
    }
    size_t GetWorkspaceSize() const
    {
        size_t bytes = 0;
        Check(ascq_matmul_w8a16_workspace_size(&desc_, &bytes));
        return bytes;
    }
    void IterateAll(const DeviceTensor<CType>& c, void* stream = nullptr)
    {
        Check(ascq_matmul_w8a16(&desc_, c.GetPhyAddr(), a_, b_, offset_, scale_, workspace_, workspace_bytes_,
                                stream));
    }
    const ascq_w8a16_desc& Desc() const { return desc_; }

private:
    ascq_w8a16_desc desc_;
    const void* a_ = nullptr;
    const void* b_ = nullptr;
    const void* offset_ = nullptr;
    const void* scale_ = nullptr;
    void* workspace_ = nullptr;
    size_t workspace_bytes_ = 0;
};

}  // namespace ascq

#endif  // ASCQ_ASCENDC_HPP
