"""Operator interface of the asc-devkit quantization path on torch device tensors, bound to libascq over its C ABI.

Names and argument meaning follow the reference's `AscendC::` functions (citations below are files of the reference
tree); a tensor argument is a CUDA/HIP torch tensor whose storage is handed to the library as a raw device pointer.
torch only provides device memory and the current stream.  Every function raises `AscqError` when the library
rejects the call; nothing here computes on the CPU.
"""
import ctypes as C
from dataclasses import dataclass

import torch

from . import _abi as abi
from ._abi import AscqError, check, load_library  # noqa: F401

_DT = {torch.float16: abi.F16, torch.bfloat16: abi.BF16, torch.float32: abi.F32, torch.int8: abi.I8,
       torch.int32: abi.I32, torch.int64: abi.U64, torch.uint8: abi.I4}
if hasattr(torch, "uint64"):
    _DT[torch.uint64] = abi.U64
_QDST = {torch.int8: abi.QDST_I8, torch.float8_e4m3fn: abi.QDST_FP8_E4M3FN, torch.float8_e5m2: abi.QDST_FP8_E5M2}
_TORCH = {abi.F16: torch.float16, abi.BF16: torch.bfloat16, abi.F32: torch.float32, abi.I8: torch.int8,
          abi.I32: torch.int32}


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("ascq operators take device tensors")
    if not t.is_contiguous():
        raise ValueError("ascq operators take contiguous tensors")
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dt(t):
    return _DT[t.dtype]


# ------------------------------------------------------------------------------------------------ AscendQuant
@dataclass
class AscendQuantConfig:
    """ref: include/adv_api/quantization/ascend_quant_utils.h:31-71"""
    has_offset: bool = False
    k_dim: int = 1
    round_mode: int = abi.CAST_RINT


@dataclass
class AscendQuantParam:
    """ref: include/adv_api/quantization/ascend_quant_utils.h:82-87"""
    m: int
    n: int
    cal_count: int
    group_size: int = 0


def _quant(desc, dst, src, scale, offset):
    check(load_library().ascq_quant(C.byref(desc), _ptr(dst), _ptr(src), _ptr(scale), _ptr(offset), _stream()))
    return dst


def ascend_quant(dst, src, scale, offset, cal_count=None, scale_count=None, offset_count=None, dst_format=None):
    """AscendQuant<T>(dst, src, scale, offset, [scaleCount, offsetCount,] calCount): per-tensor when `scale` is a
    float, per-channel when it is a tensor (offset: float or tensor).  Every intermediate is fp16.
    dst_format=abi.QDST_HIF8: dst is a uint8 tensor of hifloat8 codes (the half chain, then the cast that rounds ties
    away from zero: ascend_quant_3510_impl.h:82-111).
    ref: include/adv_api/quantization/ascend_quant.h:63-347."""
    cal = src.numel() if cal_count is None else cal_count
    d = abi.QuantDesc(src_dtype=_dt(src), compute=abi.COMPUTE_F16, round_mode=abi.CAST_RINT, k_dim=1, cal_count=cal,
                      dst_format=abi.QDST_I8 if dst_format is None else dst_format)
    if torch.is_tensor(scale):
        n = scale.numel() if scale_count is None else scale_count
        d.policy, d.scale_dtype, d.n = abi.PER_CHANNEL, _dt(scale), n
        if torch.is_tensor(offset):
            oc = offset.numel() if offset_count is None else offset_count
            if oc != n:
                raise AscqError(abi.EINVAL, f"scaleCount {n} must equal offsetCount {oc}")
            d.offset_kind = abi.OFFSET_TENSOR
            return _quant(d, dst, src, scale, offset)
        d.offset_kind, d.offset = abi.OFFSET_SCALAR, float(offset)
        return _quant(d, dst, src, scale, None)
    d.policy, d.scale_dtype = abi.PER_TENSOR, _dt(src)
    d.scale, d.offset, d.offset_kind = float(scale), float(offset), abi.OFFSET_SCALAR
    return _quant(d, dst, src, None, None)


def _policy_quant(compute, dst, src, scale, offset, para, policy, config, dst_format=None):
    d = abi.QuantDesc(policy=policy, src_dtype=_dt(src), compute=compute, round_mode=config.round_mode,
                      k_dim=config.k_dim, m=para.m, n=para.n, cal_count=para.cal_count, group_size=para.group_size,
                      dst_format=_QDST[dst.dtype] if dst_format is None else dst_format)
    if policy == abi.PER_TENSOR:
        d.scale, d.scale_dtype = float(scale), _dt(src)
        scale = None
    else:
        d.scale_dtype = _dt(scale)
    if not config.has_offset:
        d.offset_kind, offset = abi.OFFSET_NONE, None
    elif torch.is_tensor(offset):
        d.offset_kind = abi.OFFSET_TENSOR
    else:
        d.offset_kind, d.offset, offset = abi.OFFSET_SCALAR, float(offset), None
    return _quant(d, dst, src, scale, offset)


def ascend_quant_policy(dst, src, scale, offset, para, policy, config=AscendQuantConfig(), dst_format=None):
    """AscendQuant<dstT, srcT, scaleT, config, policy>(dst, src, scale, offset, para) for PER_TOKEN / PER_GROUP:
    arithmetic in the scale's dtype for an int8 dst, in fp32 for a torch.float8_e4m3fn / float8_e5m2 dst.
    dst_format=abi.QDST_FP4_E2M1 / QDST_FP4_E1M2 (PER_GROUP only): dst is a uint8 tensor of cal_count / 2 bytes, two
    4-bit floats per byte with the even element in the low nibble (fp4x2_e2m1_t / fp4x2_e1m2_t).
    dst_format=abi.QDST_HIF8: dst is a uint8 tensor of hifloat8 codes; arithmetic in the scale's dtype as for int8,
    config.round_mode CAST_ROUND (CAST_HYBRID is refused).
    ref: include/adv_api/quantization/ascend_quant.h:667-762."""
    return _policy_quant(abi.COMPUTE_SCALE_T, dst, src, scale, offset, para, policy, config, dst_format)


def quantize(dst, src, scale, offset, para, policy, config=AscendQuantConfig(), dst_format=None):
    """Quantize<config>(dst, src, scale, offset, params): always fp32 arithmetic, any policy; dst_format=abi.QDST_HIF8
    for hifloat8 codes in a uint8 dst.
    ref: include/adv_api/quantization/quantize.h, impl/adv_api/detail/quantization/quantize/quantize_impl.h:923-968."""
    return _policy_quant(abi.COMPUTE_F32, dst, src, scale, offset, para, policy, config, dst_format)


def dynamic_quant_per_token(x, q=None, tok_scale=None):
    """Row abs-max -> scale = amax/127 -> AscendQuant PER_TOKEN with 127/amax, in one kernel."""
    m, n = x.shape
    q = torch.empty((m, n), dtype=torch.int8, device=x.device) if q is None else q
    tok_scale = torch.empty(m, dtype=torch.float32, device=x.device) if tok_scale is None else tok_scale
    check(load_library().ascq_dynamic_quant_per_token(_dt(x), m, n, _ptr(q), _ptr(tok_scale), _ptr(x), _stream()))
    return q, tok_scale


# ---------------------------------------------------------------------------------------------- AscendDequant
@dataclass
class DequantParams:
    """ref: include/adv_api/quantization/ascend_dequant_utils.h:26-30"""
    m: int
    n: int
    cal_count: int


def dequant_dst_stride(dst_dtype, n):
    return load_library().ascq_dequant_dst_stride(_DT[dst_dtype], n)


def ascend_dequant(dst, src, deq_scale, params, mode=abi.DEQUANT_WITH_SINGLE_ROW, scale_dtype=None):
    """AscendDequant<dstT, scaleT, mode>(dst, src, deqScale, {m, n, calCount}); deqScale is a tensor (float32,
    bfloat16, or uint64 passed as an int64 tensor) or a float.  ref: include/adv_api/quantization/ascend_dequant.h:58-281."""
    d = abi.DequantDesc(src_dtype=_dt(src), dst_dtype=_dt(dst), mode=mode, m=params.m, n=params.n,
                        cal_count=params.cal_count)
    if torch.is_tensor(deq_scale):
        d.policy = abi.PER_CHANNEL
        d.scale_dtype = _dt(deq_scale) if scale_dtype is None else scale_dtype
    else:
        d.policy, d.scale, d.scale_dtype = abi.PER_TENSOR, float(deq_scale), abi.F32
        deq_scale = None
    check(load_library().ascq_dequant(C.byref(d), _ptr(dst), _ptr(src), _ptr(deq_scale), _stream()))
    return dst


class AscendDeQuantPolicy:
    """ref: include/adv_api/quantization/ascend_dequant_utils.h:37 (same members, same values)"""
    PER_TOKEN, PER_GROUP, PER_CHANNEL_PER_GROUP, PER_TOKEN_PER_GROUP = range(4)
    TO_ABI = {0: abi.PER_TOKEN, 1: abi.PER_GROUP, 2: abi.PER_CHANNEL_PER_GROUP, 3: abi.PER_TOKEN_PER_GROUP}


def ascend_dequant_policy(dst, src, scale, para, policy, k_dim=1):
    """AscendDequant<dstT, srcT, scaleT, config, policy> for PER_TOKEN / PER_GROUP; `policy` is an ascq policy value
    (abi.PER_TOKEN ...); AscendDeQuantPolicy.TO_ABI maps the reference's own enumerators.  The two combined policies the
    reference declares are answered with ASCQ_EUNSUPPORTED.
    ref: include/adv_api/quantization/ascend_dequant.h:284-305."""
    d = abi.DequantDesc(policy=policy, src_dtype=_dt(src), scale_dtype=_dt(scale), dst_dtype=_dt(dst),
                        mode=abi.DEQUANT_WITH_MULTI_ROW, k_dim=k_dim, m=para.m, n=para.n, cal_count=para.cal_count,
                        group_size=para.group_size)
    check(load_library().ascq_dequant(C.byref(d), _ptr(dst), _ptr(src), _ptr(scale), _stream()))
    return dst


# -------------------------------------------------------------------------------------------- AscendAntiQuant
@dataclass
class AntiQuantShapeInfo:
    """ref: include/adv_api/quantization/ascend_antiquant_utils.h:27-32"""
    offset_height: int = 0
    offset_width: int = 0
    scale_height: int = 0
    scale_width: int = 0


def ascend_antiquant(dst, src, offset, scale, k, shape_info=AntiQuantShapeInfo(), is_transpose=False, int4=False):
    """AscendAntiQuant<SrcT, DstT, isTranspose>(dst, src, offset, scale, k, shapeInfo).  `offset` may be None (the
    scale-only overloads); `scale` / `offset` floats select the per-tensor overloads.  `src` is int8, or uint8 holding
    packed int4 when int4=True.  ref: include/adv_api/quantization/ascend_antiquant.h:50-199."""
    elems = dst.numel()
    d = abi.AntiQuantDesc(src_dtype=abi.I4 if int4 else abi.I8, dst_dtype=_dt(dst), is_transpose=int(is_transpose),
                          has_offset=int(offset is not None), k=k, n=elems // k,
                          offset_height=shape_info.offset_height, offset_width=shape_info.offset_width,
                          scale_height=shape_info.scale_height, scale_width=shape_info.scale_width)
    if not torch.is_tensor(scale):
        d.per_tensor, d.scale, d.offset = 1, float(scale), float(offset or 0.0)
        scale = offset = None
    check(load_library().ascq_antiquant(C.byref(d), _ptr(dst), _ptr(src), _ptr(offset), _ptr(scale), _stream()))
    return dst


@dataclass
class AscendAntiQuantConfig:
    """ref: include/adv_api/quantization/ascend_antiquant_common.h:45-65"""
    has_offset: bool = False
    is_transpose: bool = False
    k_dim: int = 1


@dataclass
class AscendAntiQuantParam:
    m: int
    n: int
    cal_count: int
    group_size: int = 0


def _antiquant_policy(compute, dst, src, scale, offset, para, policy, config, src_format=None):
    d = abi.AntiQuantPolicyDesc(policy=policy, src_format=_QDST[src.dtype] if src_format is None else src_format,
                                dst_dtype=_dt(dst),
                                compute=compute, has_offset=int(config.has_offset),
                                is_transpose=int(config.is_transpose), k_dim=config.k_dim, m=para.m, n=para.n,
                                cal_count=para.cal_count, group_size=para.group_size)
    if policy == abi.PER_TENSOR:
        d.scale_dtype, d.scale, d.offset = _dt(dst), float(scale), float(offset) if config.has_offset else 0.0
        scale = offset = None
    elif d.src_format in (abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2):
        d.scale_dtype = abi.E8M0        # one byte per group: 2^(code - 127)
    else:
        d.scale_dtype = _dt(scale)
    check(load_library().ascq_antiquant_policy(C.byref(d), _ptr(dst), _ptr(src), _ptr(scale),
                                               _ptr(offset) if config.has_offset else None, _stream()))
    return dst


def ascend_antiquant_policy(dst, src, scale, offset, para, policy, config=AscendAntiQuantConfig(), src_format=None):
    """AscendAntiQuant<dstT, srcT, scaleT, config, policy>(dst, src, scale, offset, para) for PER_TOKEN / PER_GROUP:
    src int8 / torch.float8_e4m3fn / torch.float8_e5m2 [m, n], arithmetic in the scale's dtype.
    src_format=abi.QDST_FP4_E2M1 / QDST_FP4_E1M2 (PER_GROUP, no offset): src is a uint8 tensor [m, n / 2] holding two
    4-bit floats per byte (fp4x2_e2m1_t / fp4x2_e1m2_t), scale a uint8 tensor of fp8_e8m0 codes, dst half / bfloat16.
    ref: impl/adv_api/detail/quantization/antiquant/ascend_antiquant_3510_impl.h:1727-1779, 2166-2222."""
    return _antiquant_policy(abi.COMPUTE_SCALE_T, dst, src, scale, offset, para, policy, config, src_format)


def antiquantize(dst, src, scale, offset, para, policy, config=AscendAntiQuantConfig(), src_format=None):
    """AntiQuantize<config>(dst, src, scale, offset, params): fp32 arithmetic whatever the parameter type, any policy.
    PER_TENSOR takes Python floats (values of the output's type), PER_CHANNEL tensors [n] of the output's type.
    src_format=abi.QDST_HIF8: src is a uint8 tensor of hifloat8 codes.
    ref: include/adv_api/quantization/antiquantize.h:59-95, impl/adv_api/detail/quantization/antiquantize/
    antiquantize_impl.h:36-135."""
    return _antiquant_policy(abi.COMPUTE_F32, dst, src, scale, offset, para, policy, config, src_format)


def dequantize(dst, src, scale, para, policy, k_dim=1):
    """Dequantize<config>(dst, src, scale, offset, params) (the offset is not supported by the reference either):
    PER_TENSOR (scale a Python float) and PER_CHANNEL are AscendDequant in DEQUANT_WITH_MULTI_ROW mode on {m, n, n},
    PER_TOKEN / PER_GROUP the policy form.  `para` has m, n (and group_size for PER_GROUP).
    ref: impl/adv_api/detail/quantization/dequantize/dequantize_impl.h:94-196."""
    if policy in (abi.PER_TENSOR, abi.PER_CHANNEL):
        return ascend_dequant(dst, src, scale, DequantParams(m=para.m, n=para.n, cal_count=para.n),
                              mode=abi.DEQUANT_WITH_MULTI_ROW)
    p = AscendQuantParam(m=para.m, n=para.n, cal_count=para.m * para.n, group_size=getattr(para, "group_size", 0))
    return ascend_dequant_policy(dst, src, scale, p, policy, k_dim=k_dim)


# ------------------------------------------------------------------------------------------ Matmul quant path
class Matmul:
    """Host-side mirror of `Matmul<A int8, B int8, C, Bias>` on the quant path: SetTensorA/B, SetBias,
    SetQuantScalar / SetQuantVector, IterateAll.  ref: include/adv_api/matmul/matmul.h:73-398,
    impl/adv_api/detail/matmul/matmul_impl_base.h:355-378."""

    def __init__(self, m, n, k, trans_a=False, trans_b=False):
        self.desc = abi.MatmulDesc(m=m, n=n, k=k, trans_a=int(trans_a), trans_b=int(trans_b), out_dtype=abi.I32,
                                   quant_mode=abi.MM_QUANT_NONE, scale_format=abi.MM_SCALE_U64)
        self.a = self.b = self.bias = self.quant = self.tok = None
        self.packed = False
        self._ws_by_stream = {}   # scratch per stream handle: calls of one object on two streams may overlap
        self._need = {}           # scratch size per (shape, options)

    def set_tensor_a(self, a):
        self.a = a

    def set_tensor_b(self, b, nz=False):
        """b: int8 [k, n] row-major, or with nz=True the fractal layout [n/32, k/16, 16, 32] (CubeFormat::NZ)."""
        self.b = b
        self.packed = False
        self.desc.b_format = abi.MM_B_NZ if nz else abi.MM_B_ND

    def set_tensor_b_packed(self, w_packed):
        """b in the layout of pack_weight_w8 (packed once, when the weights are loaded): iterate_all then runs the
        one-launch kernel for few activation rows, which needs no scratch."""
        self.b = w_packed
        self.packed = True
        self.desc.b_format = abi.MM_B_ND

    def set_bias(self, bias):
        """int32 bias: initial value of the accumulator; float32 / bfloat16 bias: added after dequantisation."""
        self.bias = bias
        self.desc.bias_kind = {torch.int32: abi.MM_BIAS_I32_PRE, torch.float32: abi.MM_BIAS_F32_POST,
                               torch.bfloat16: abi.MM_BIAS_BF16_POST}[bias.dtype]

    def set_quant_scalar(self, quant_scalar):
        """uint64 parameter word (ref: SetQuantScalar), or a Python float for a full-precision fp32 scale."""
        self.desc.quant_mode = abi.MM_QUANT_SCALAR
        if isinstance(quant_scalar, float):
            self.desc.scale_format = abi.MM_SCALE_F32
            self.desc.quant_scalar = int(torch.tensor(quant_scalar, dtype=torch.float32).view(torch.int32).item()) \
                & 0xFFFFFFFF
        else:
            self.desc.scale_format, self.desc.quant_scalar = abi.MM_SCALE_U64, int(quant_scalar)

    def set_quant_vector(self, quant_vector):
        """uint64 parameter words (as an int64 / uint64 tensor; ref: SetQuantVector) or a float32 scale tensor."""
        self.desc.quant_mode = abi.MM_QUANT_VECTOR
        self.desc.scale_format = abi.MM_SCALE_F32 if quant_vector.dtype == torch.float32 else abi.MM_SCALE_U64
        self.quant = quant_vector

    def set_token_scale(self, tok_scale):
        self.tok, self.desc.has_tok_scale = tok_scale, 1

    def set_activation(self, activation, beta=1.0):
        """MM_ACT_FASTER_GELU, or MM_ACT_SWIGLU: columns 2j / 2j + 1 of the product are src0 / src1 of
        SwiGLU(src0, src1, beta) and c is [m, n / 2] (ref: include/adv_api/activation/swiglu.h)."""
        self.desc.activation = activation
        self.desc.act_beta = beta

    def _scratch(self, need_bytes, device):
        """The object's scratch buffer for the current stream (grown when a larger one is needed)."""
        key = _stream().value
        ws = self._ws_by_stream.get(key)
        if ws is None or ws.numel() * 4 < need_bytes:
            ws = torch.empty((need_bytes + 3) // 4, dtype=torch.int32, device=device)
            self._ws_by_stream[key] = ws
        return ws

    @property
    def _ws(self):
        return self._ws_by_stream.get(_stream().value)

    def iterate_all(self, c):
        self.desc.out_dtype = _dt(c)
        lib = load_library()
        if self.packed:
            check(lib.ascq_matmul_w8a8_packed(C.byref(self.desc), _ptr(c), _ptr(self.a), _ptr(self.b), _ptr(self.bias),
                                              _ptr(self.quant), _ptr(self.tok), _stream()))
            return c
        # the size query is a host call of its own, which a decode step of a dozen microseconds notices: asked once per
        # shape and option set
        d = self.desc
        key = (d.m, d.n, d.k, d.trans_a, d.trans_b, d.out_dtype, d.quant_mode, d.scale_format, d.bias_kind,
               d.has_tok_scale, d.activation, d.b_format)
        need = self._need.get(key)
        if need is None:
            size = C.c_size_t(0)
            check(lib.ascq_matmul_w8a8_workspace_size(C.byref(d), C.byref(size)))
            need = self._need[key] = size.value
        if need:
            self._scratch(need, c.device)
        check(lib.ascq_matmul_w8a8(C.byref(d), _ptr(c), _ptr(self.a), _ptr(self.b), _ptr(self.bias),
                                   _ptr(self.quant), _ptr(self.tok), _ptr(self._ws) if need else None, need, _stream()))
        return c

    def plan(self, c):
        """The launch plan `iterate_all(c)` would follow (kernel family, tile shape, workgroups, K splits), as a
        MatmulPlan; nothing is launched.  The counterpart of the reference's host-side TCubeTiling
        (include/adv_api/matmul/matmul_tilingdata.h:21-72)."""
        self.desc.out_dtype = _dt(c)
        lib = load_library()
        need = C.c_size_t(0)
        check(lib.ascq_matmul_w8a8_workspace_size(C.byref(self.desc), C.byref(need)))
        if need.value:
            self._scratch(need.value, c.device)
        plan = abi.MatmulPlan()
        check(lib.ascq_matmul_w8a8_plan(C.byref(self.desc), _ptr(c), _ptr(self.a), _ptr(self.b), _ptr(self.bias),
                                        _ptr(self.quant), _ptr(self.tok), _ptr(self._ws) if need.value else None,
                                        need.value, C.byref(plan)))
        return plan


class MatmulInt4(Matmul):
    """`Matmul<int4b_t, int4b_t, C>`: a and b are uint8 / int8 tensors holding two int4 per byte (even element in the
    low nibble): a [m, k/2], b [k, n/2] ([n, k/2] with trans_b).  Everything else as Matmul.
    ref: examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_int4/matmul_int4.asc:52-58."""

    def iterate_all(self, c):
        self.desc.out_dtype = _dt(c)
        lib = load_library()
        need = C.c_size_t(0)
        check(lib.ascq_matmul_w4a4_workspace_size(C.byref(self.desc), C.byref(need)))
        self._scratch(max(need.value, 4), c.device)
        check(lib.ascq_matmul_w4a4(C.byref(self.desc), _ptr(c), _ptr(self.a), _ptr(self.b), _ptr(self.bias),
                                   _ptr(self.quant), _ptr(self.tok), _ptr(self._ws), need.value, _stream()))
        return c

    def plan(self, c):
        raise NotImplementedError("the plan query describes the int8 matmul; widen the operands with unpack_int4")


def unpack_int4(src, out=None):
    """Packed int4 (two per byte, even element in the low nibble) -> int8, same leading shape, last dimension doubled."""
    if not src.is_contiguous() or src.element_size() != 1:
        raise ValueError("unpack_int4: a contiguous one-byte tensor is expected")
    if out is None:
        out = torch.empty(tuple(src.shape[:-1]) + (src.shape[-1] * 2,), dtype=torch.int8, device=src.device)
    check(load_library().ascq_unpack_int4(_ptr(out), _ptr(src), src.numel() * 2, _stream()))
    return out


_lin_ws = {}
_lin_need = {}


def _linear_workspace(lib, d, device):
    """The scratch buffer of the one-call linear: sized once per shape (the size query is a host call of its own, which
    a decode step of a dozen microseconds notices), one buffer per stream (calls on two streams may overlap)."""
    shape = (d.m, d.n, d.k, d.trans_b, d.out_dtype, d.activation, d.bias_kind)
    need = _lin_need.get(shape)
    if need is None:
        size = C.c_size_t(0)
        check(lib.ascq_linear_w8a8_dynamic_workspace_size(C.byref(d), C.byref(size)))
        need = _lin_need[shape] = size.value
    key = (device, need, _stream().value)
    ws = _lin_ws.get(key)
    if ws is None:
        ws = _lin_ws[key] = torch.empty(max(need, 16), dtype=torch.uint8, device=device)
    return ws


def linear_w8a8_dynamic(c, x, weight, channel_scale, bias=None, activation=abi.MM_ACT_NONE, trans_b=False, act_beta=1.0):
    """c = dequant(dynamic_quant_per_token(x) @ weight): the activation quantiser and the int8 matmul in one call, with
    the results of calling the two one after the other.  x half / bfloat16 / float32 [m, k]; weight int8 [k, n];
    channel_scale float32 [n]; bias float32 / bfloat16 [n] (added after dequantisation)."""
    m, k = x.shape
    n = weight.shape[0] if trans_b else weight.shape[1]    # with SwiGLU c has n / 2 columns
    d = abi.MatmulDesc(m=m, n=n, k=k, trans_b=int(trans_b), out_dtype=_dt(c), quant_mode=abi.MM_QUANT_VECTOR,
                       scale_format=abi.MM_SCALE_F32, activation=activation, act_beta=act_beta)
    if bias is not None:
        d.bias_kind = abi.MM_BIAS_F32_POST if bias.dtype == torch.float32 else abi.MM_BIAS_BF16_POST
    lib = load_library()
    ws = _linear_workspace(lib, d, x.device)
    check(lib.ascq_linear_w8a8_dynamic(C.byref(d), _dt(x), _ptr(c), _ptr(x), _ptr(weight), _ptr(bias),
                                       _ptr(channel_scale), _ptr(ws), ws.numel(), _stream()))
    return c


class DynamicLinear:
    """The one-call W8A8 linear with everything that does not change between calls prepared once (descriptor, scratch,
    argument pointers): a decode step of ten microseconds notices a descriptor built per call.  weight: int8 [k, n],
    [n, k] with trans_b, or, with packed_n, the buffer of pack_weight_w8 for n columns."""

    def __init__(self, m, k, weight, channel_scale, bias=None, trans_b=False, packed_n=None, out_dtype=torch.bfloat16,
                 x_dtype=torch.bfloat16, activation=abi.MM_ACT_NONE, act_beta=1.0):
        n = packed_n if packed_n is not None else (weight.shape[0] if trans_b else weight.shape[1])
        self.desc = abi.MatmulDesc(m=m, n=n, k=k, trans_b=int(trans_b and packed_n is None), out_dtype=_DT[out_dtype],
                                   quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32, activation=activation,
                                   act_beta=act_beta)
        if bias is not None:
            self.desc.bias_kind = abi.MM_BIAS_F32_POST if bias.dtype == torch.float32 else abi.MM_BIAS_BF16_POST
        self.lib = load_library()
        self.fn = self.lib.ascq_linear_w8a8_dynamic_packed if packed_n is not None else self.lib.ascq_linear_w8a8_dynamic
        self.keep = (weight, channel_scale, bias)
        self.ws = _linear_workspace(self.lib, self.desc, weight.device)
        self.x_dt, self.out_dtype = _DT[x_dtype], out_dtype
        self.args = (_ptr(weight), _ptr(bias), _ptr(channel_scale), _ptr(self.ws), self.ws.numel())
        self.ref = C.byref(self.desc)

    def __call__(self, c, x):
        """c [m, n] of out_dtype (n / 2 columns with SwiGLU), x [m, k] of x_dtype, on the current stream (the scratch
        belongs to the stream the object was made on: calls on other streams at the same time would share it)."""
        if not (c.is_contiguous() and x.is_contiguous() and c.is_cuda and x.is_cuda):
            raise ValueError("ascq operators take contiguous device tensors")
        check(self.fn(self.ref, self.x_dt, c.data_ptr(), x.data_ptr(), *self.args, _stream()))
        return c


def linear_w8a8_dynamic_noalloc(c, x, weight, channel_scale, bias=None, activation=abi.MM_ACT_NONE, trans_b=False,
                                act_beta=1.0):
    """linear_w8a8_dynamic on the library's built-in scratch buffer: no workspace, no allocation.  Calls that overlap
    on one GPU share that buffer and race."""
    m, k = x.shape
    n = weight.shape[0] if trans_b else weight.shape[1]    # with SwiGLU c has n / 2 columns
    d = abi.MatmulDesc(m=m, n=n, k=k, trans_b=int(trans_b), out_dtype=_dt(c), quant_mode=abi.MM_QUANT_VECTOR,
                       scale_format=abi.MM_SCALE_F32, activation=activation, act_beta=act_beta)
    if bias is not None:
        d.bias_kind = abi.MM_BIAS_F32_POST if bias.dtype == torch.float32 else abi.MM_BIAS_BF16_POST
    check(load_library().ascq_linear_w8a8_dynamic_noalloc(C.byref(d), _dt(x), _ptr(c), _ptr(x), _ptr(weight), _ptr(bias),
                                                          _ptr(channel_scale), _stream()))
    return c


def linear_w8a8_dynamic_packed(c, x, w_packed, n, channel_scale, bias=None, activation=abi.MM_ACT_NONE):
    """linear_w8a8_dynamic on weights packed by pack_weight_w8 (n = their column count): up to 8 rows of half /
    bfloat16 x are one launch; the results are those of linear_w8a8_dynamic on the unpacked weights."""
    m, k = x.shape
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=_dt(c), quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                       activation=activation, act_beta=1.0)
    if bias is not None:
        d.bias_kind = abi.MM_BIAS_F32_POST if bias.dtype == torch.float32 else abi.MM_BIAS_BF16_POST
    lib = load_library()
    ws = _linear_workspace(lib, d, x.device)
    check(lib.ascq_linear_w8a8_dynamic_packed(C.byref(d), _dt(x), _ptr(c), _ptr(x), _ptr(w_packed), _ptr(bias),
                                              _ptr(channel_scale), _ptr(ws), ws.numel(), _stream()))
    return c


def quant_group_matmul(y, x, weight, group_list, scale, per_token_scale=None, bias=None,
                       group_list_kind=abi.GROUP_LIST_COUNTS, activation=abi.MM_ACT_NONE, weight_nz=False, act_beta=1.0):
    """The quantized grouped matmul of the reference's MoE example: x int8 [m, k], weight int8 [g, k, n] (or, with
    weight_nz, the example's fractal layout [g, n/32, k/16, 16, 32]), scale float32 [g, n], per_token_scale float32
    [m], group_list int64 [g] (counts or prefix sums).
    ref: examples/01_simd_cpp_api/05_best_practices/03_fusion_compute/quant_group_matmul_high_performance/
    quant_group_matmul_custom.asc:255-454."""
    if weight_nz:
        g, k, n = weight.shape[0], weight.shape[2] * weight.shape[3], weight.shape[1] * weight.shape[4]
    else:
        g, k, n = weight.shape
    mm = abi.MatmulDesc(m=x.shape[0], n=n, k=k, out_dtype=_dt(y), quant_mode=abi.MM_QUANT_VECTOR,
                        scale_format=abi.MM_SCALE_F32, has_tok_scale=int(per_token_scale is not None),
                        activation=activation, act_beta=act_beta, b_format=abi.MM_B_NZ if weight_nz else abi.MM_B_ND)
    if bias is not None:
        mm.bias_kind = abi.MM_BIAS_F32_POST if bias.dtype == torch.float32 else abi.MM_BIAS_BF16_POST
    d = abi.GroupMatmulDesc(mm=mm, groups=g, group_list_kind=group_list_kind)
    check(load_library().ascq_group_matmul_w8a8(C.byref(d), _ptr(y), _ptr(x), _ptr(weight), _ptr(bias), _ptr(scale),
                                                _ptr(per_token_scale), _ptr(group_list), _stream()))
    return y


# ------------------------------------------------------------------------------------------------------ W4A16
_w4_ws = {}


def matmul_w4a16(y, x, w_packed, scale, offset=None, group_size=128, workspace=None):
    """y f16 [m, n] = x f16 [m, k] @ AscendAntiQuant<int4b_t, half>(w [k, n] packed two per byte, per-group params)."""
    m, k = x.shape
    n = y.shape[1]
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=group_size, has_offset=int(offset is not None))
    lib = load_library()
    need = C.c_size_t(0)
    check(lib.ascq_matmul_w4a16_workspace_size(C.byref(d), C.byref(need)))
    if workspace is None:
        key = (x.device, need.value, _stream().value)   # one scratch buffer per stream: calls on two streams may overlap
        if key not in _w4_ws:
            _w4_ws[key] = torch.zeros(max(need.value // 4, 4), dtype=torch.float32, device=x.device)
        workspace = _w4_ws[key]
    check(lib.ascq_matmul_w4a16(C.byref(d), _ptr(y), _ptr(x), _ptr(w_packed), _ptr(scale), _ptr(offset),
                                _ptr(workspace), workspace.numel() * workspace.element_size(), _stream()))
    return y


def pack_weight_w8(b, k, n, trans_b=False):
    """int8 weights [k, n] ([n, k] with trans_b) -> the GPU-native packed layout of Matmul.set_tensor_b_packed."""
    lib = load_library()
    need = C.c_size_t(0)
    check(lib.ascq_pack_weight_w8_size(k, n, C.byref(need)))
    out = torch.empty(need.value, dtype=torch.uint8, device=b.device)
    check(lib.ascq_pack_weight_w8(_ptr(b), _ptr(out), k, n, int(trans_b), _stream()))
    return out


def pack_weight_w4(w_nd, k, n):
    """int4 weights [k, n / 2] bytes (two per byte along n) -> the GPU-native packed layout of matmul_w4a16_packed."""
    lib = load_library()
    need = C.c_size_t(0)
    check(lib.ascq_pack_weight_w4_size(k, n, C.byref(need)))
    out = torch.empty(need.value, dtype=torch.uint8, device=w_nd.device)
    check(lib.ascq_pack_weight_w4(_ptr(w_nd), _ptr(out), k, n, _stream()))
    return out


def matmul_w4a16_packed(y, x, w_gpu, scale, offset=None, group_size=128, mode=abi.W4A16_PER_WEIGHT):
    """matmul_w4a16 on weights packed by pack_weight_w4: one launch, no workspace.  mode abi.W4A16_PER_WEIGHT (default)
    keeps AscendAntiQuant's two roundings to half per weight; abi.W4A16_GROUP_SUM applies scale and offset once per
    quantisation group to fp32 sums (same value, no per-weight roundings, faster)."""
    m, k = x.shape
    n = y.shape[1]
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=group_size, has_offset=int(offset is not None), mode=mode)
    check(load_library().ascq_matmul_w4a16_packed(C.byref(d), _ptr(y), _ptr(x), _ptr(w_gpu), _ptr(scale),
                                                  _ptr(offset), _stream()))
    return y


# ------------------------------------------------------------------------------------------------------ W8A16
def matmul_w8a16(y, x, w, offset=None, scale=None, workspace=None, trans_b=False, mode=abi.W8A16_PER_WEIGHT):
    """y f16 / f32 [m, n] = x f16 [m, k] @ AscendAntiQuant<int8_t, half>(w int8 [k, n]); trans_b: w is [n, k]
    (SetTensorB(b, isTransposeB=true)) and the call is one launch without a workspace.

    scale / offset: f16 tensors of n elements (SetAntiQuantVector) or Python floats (SetAntiQuantScalar); offset None =
    MatmulConfig::hasAntiQuantOffset false.  mode: abi.W8A16_CHANNEL_SUM applies scale and offset once per output to
    fp32 sums (up to 4 rows on [n, k] weights; elsewhere the per-weight form runs).
    """
    m, k = x.shape
    n = y.shape[1]
    per_tensor = not torch.is_tensor(scale)
    d = abi.W8A16Desc(m=m, n=n, k=k, per_tensor=int(per_tensor), has_offset=int(offset is not None),
                      scale=float(scale) if per_tensor else 0.0,
                      offset=float(offset) if per_tensor and offset is not None else 0.0, out_dtype=_DT[y.dtype],
                      trans_b=int(trans_b), mode=mode)
    lib = load_library()
    need = C.c_size_t(0)
    check(lib.ascq_matmul_w8a16_workspace_size(C.byref(d), C.byref(need)))
    if workspace is None:
        key = (x.device, need.value, _stream().value)   # one scratch buffer per stream: calls on two streams may overlap
        if key not in _w4_ws:
            _w4_ws[key] = torch.zeros(max(need.value // 4, 4), dtype=torch.float32, device=x.device)
        workspace = _w4_ws[key]
    check(lib.ascq_matmul_w8a16(C.byref(d), _ptr(y), _ptr(x), _ptr(w), None if per_tensor else _ptr(offset),
                                None if per_tensor else _ptr(scale), _ptr(workspace),
                                workspace.numel() * workspace.element_size(), _stream()))
    return y


# ------------------------------------------------------------------------------------------------- MX matmul
_mx_ws = {}


def matmul_mx(c, a, b, a_scale, b_scale, a_format, b_format, k, bias=None, workspace=None):
    """MmadMx on whole matrices: c f32 / bf16 / f16 [m, n] = A @ B^T with a uint8 [m, k or k / 2] and b uint8
    [n, k or k / 2] holding fp8 (abi.QDST_FP8_E4M3FN / _E5M2) or fp4 (abi.QDST_FP4_E2M1 / _E1M2, two per byte along k)
    values and a_scale / b_scale uint8 [rows, scale_k] the fp8_e8m0 scale of every 32 k; bias f32 [n] or None."""
    m, n = c.shape
    d = abi.MxDesc(m=m, n=n, k=k, scale_k=a_scale.shape[1], a_format=a_format, b_format=b_format, out_dtype=_DT[c.dtype],
                   has_bias=int(bias is not None))
    lib = load_library()
    need = C.c_size_t(0)
    check(lib.ascq_matmul_mx_workspace_size(C.byref(d), C.byref(need)))
    if workspace is None and need.value:
        key = (c.device, need.value, _stream().value)   # one scratch buffer per stream: calls on two streams may overlap
        if key not in _mx_ws:
            _mx_ws[key] = torch.empty(need.value, dtype=torch.uint8, device=c.device)
        workspace = _mx_ws[key]
    check(lib.ascq_matmul_mx(C.byref(d), _ptr(c), _ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(bias),
                             _ptr(workspace), workspace.numel() if workspace is not None else 0, _stream()))
    return c


# ------------------------------------------------------------------------------------------- host size queries
def _shape(shape):
    return (C.c_uint32 * len(shape))(*shape), len(shape)


def get_ascend_quant_max_min_tmp_size(shape, type_size):
    """ref: impl/adv_api/tiling/quantization/ascend_quant_tiling_impl.cpp:60-68"""
    mx, mn = C.c_uint32(0), C.c_uint32(0)
    arr, nd = _shape(shape)
    check(load_library().ascq_get_ascend_quant_max_min_tmp_size(arr, nd, type_size, C.byref(mx), C.byref(mn)))
    return mx.value, mn.value


def get_ascend_dequant_max_min_tmp_size(shape, type_size):
    """ref: impl/adv_api/tiling/quantization/ascend_dequant_tiling_impl.cpp:95-118"""
    mx, mn = C.c_uint32(0), C.c_uint32(0)
    arr, nd = _shape(shape)
    check(load_library().ascq_get_ascend_dequant_max_min_tmp_size(arr, nd, type_size, C.byref(mx), C.byref(mn)))
    return mx.value, mn.value


def get_ascend_antiquant_max_min_tmp_size(src_shape, scale_shape, is_transpose, input_dtype, output_dtype):
    """ref: impl/adv_api/tiling/quantization/ascend_antiquant_tiling_impl.cpp:70-190"""
    mx, mn = C.c_uint32(0), C.c_uint32(0)
    a, na = _shape(src_shape)
    b, nb = _shape(scale_shape)
    check(load_library().ascq_get_ascend_antiquant_max_min_tmp_size(a, na, b, nb, int(is_transpose), input_dtype,
                                                                    output_dtype, C.byref(mx), C.byref(mn)))
    return mx.value, mn.value


def pack_quant_param(scale, offset9=0, is_signed=True):
    return int(load_library().ascq_pack_quant_param(float(scale), int(offset9), int(is_signed)))


def pack_weight_nz(w, out=None):
    """int8 [k, n] or [g, k, n] row-major -> the fractal layout [(g,) n/32, k/16, 16, 32] of CubeFormat::NZ, as the
    reference example packs its weights offline (quant_group_matmul_high_performance/scripts/gen_data.py:62-64)."""
    if w.dim() not in (2, 3) or w.dtype != torch.int8 or not w.is_contiguous():
        raise ValueError("pack_weight_nz: a contiguous int8 tensor [k, n] or [g, k, n] is expected")
    g = w.shape[0] if w.dim() == 3 else 1
    k, n = w.shape[-2:]
    if out is None:
        out = torch.empty(tuple(w.shape[:-2]) + (n // 32, k // 16, 16, 32), dtype=torch.int8, device=w.device)
    check(load_library().ascq_pack_weight_nz(g, k, n, _ptr(out), _ptr(w), _stream()))
    return out
