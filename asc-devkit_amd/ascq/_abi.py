"""ctypes view of include/ascq.h: enums, descriptor structs and the library loader.

The shared library is the product; this module only binds it.  Loading fails
loudly when the library has not been built: there is no CPU fallback.
"""
import ctypes as C
import os

# ascq_status
OK, EINVAL, EUNSUPPORTED, EALIGN, EHIP, ENULL = range(6)
# ascq_dtype
F16, BF16, F32, I8, I4, I32, U64, E8M0 = range(8)
# ascq_policy
PER_TENSOR, PER_CHANNEL, PER_TOKEN, PER_GROUP, PER_CHANNEL_PER_GROUP, PER_TOKEN_PER_GROUP = range(6)
# ascq_round_mode (values of the reference's RoundMode enum)
CAST_NONE, CAST_RINT, CAST_FLOOR, CAST_CEIL, CAST_ROUND, CAST_TRUNC, CAST_ODD, CAST_HYBRID = range(8)
# ascq_quant_compute
COMPUTE_F16, COMPUTE_SCALE_T, COMPUTE_F32 = range(3)
# ascq_offset_kind
OFFSET_NONE, OFFSET_SCALAR, OFFSET_TENSOR = range(3)
QDST_I8, QDST_FP8_E4M3FN, QDST_FP8_E5M2, QDST_FP4_E2M1, QDST_FP4_E1M2, QDST_HIF8 = range(6)
# ascq_dequant_mode
DEQUANT_WITH_SINGLE_ROW, DEQUANT_WITH_MULTI_ROW = range(2)
# ascq_mm_*
MM_QUANT_NONE, MM_QUANT_SCALAR, MM_QUANT_VECTOR = range(3)
MM_SCALE_U64, MM_SCALE_F32 = range(2)
MM_BIAS_NONE, MM_BIAS_I32_PRE, MM_BIAS_F32_POST, MM_BIAS_BF16_POST = range(4)
MM_ACT_NONE, MM_ACT_FASTER_GELU, MM_ACT_SWIGLU = range(3)
MM_B_ND, MM_B_NZ = range(2)
GROUP_LIST_COUNTS, GROUP_LIST_PREFIX_SUM = range(2)
W4A16_PER_WEIGHT, W4A16_GROUP_SUM = range(2)

STATUS_NAMES = {OK: "ASCQ_OK", EINVAL: "ASCQ_EINVAL", EUNSUPPORTED: "ASCQ_EUNSUPPORTED", EALIGN: "ASCQ_EALIGN",
                EHIP: "ASCQ_EHIP", ENULL: "ASCQ_ENULL"}


class QuantDesc(C.Structure):
    _fields_ = [("policy", C.c_int32), ("src_dtype", C.c_int32), ("scale_dtype", C.c_int32), ("compute", C.c_int32),
                ("round_mode", C.c_int32), ("offset_kind", C.c_int32), ("k_dim", C.c_int32), ("scale", C.c_float),
                ("offset", C.c_float), ("m", C.c_uint32), ("n", C.c_uint32), ("cal_count", C.c_uint32),
                ("group_size", C.c_uint32), ("dst_format", C.c_int32)]


class DequantDesc(C.Structure):
    _fields_ = [("policy", C.c_int32), ("src_dtype", C.c_int32), ("scale_dtype", C.c_int32), ("dst_dtype", C.c_int32),
                ("mode", C.c_int32), ("k_dim", C.c_int32), ("scale", C.c_float), ("m", C.c_uint32), ("n", C.c_uint32),
                ("cal_count", C.c_uint32), ("group_size", C.c_uint32)]


class AntiQuantDesc(C.Structure):
    _fields_ = [("src_dtype", C.c_int32), ("dst_dtype", C.c_int32), ("is_transpose", C.c_int32),
                ("has_offset", C.c_int32), ("per_tensor", C.c_int32), ("scale", C.c_float), ("offset", C.c_float),
                ("k", C.c_uint32), ("n", C.c_uint32), ("offset_height", C.c_uint32), ("offset_width", C.c_uint32),
                ("scale_height", C.c_uint32), ("scale_width", C.c_uint32)]


class AntiQuantPolicyDesc(C.Structure):
    _fields_ = [("policy", C.c_int32), ("src_format", C.c_int32), ("scale_dtype", C.c_int32), ("dst_dtype", C.c_int32),
                ("compute", C.c_int32), ("has_offset", C.c_int32), ("is_transpose", C.c_int32), ("k_dim", C.c_int32),
                ("m", C.c_uint32), ("n", C.c_uint32), ("cal_count", C.c_uint32), ("group_size", C.c_uint32),
                ("scale", C.c_float), ("offset", C.c_float)]


class MatmulDesc(C.Structure):
    _fields_ = [("m", C.c_uint32), ("n", C.c_uint32), ("k", C.c_uint32), ("trans_a", C.c_int32),
                ("trans_b", C.c_int32), ("out_dtype", C.c_int32), ("quant_mode", C.c_int32),
                ("scale_format", C.c_int32), ("bias_kind", C.c_int32), ("has_tok_scale", C.c_int32),
                ("activation", C.c_int32), ("b_format", C.c_int32), ("quant_scalar", C.c_uint64),
                ("act_beta", C.c_float), ("reserved", C.c_int32)]


class GroupMatmulDesc(C.Structure):
    _fields_ = [("mm", MatmulDesc), ("groups", C.c_uint32), ("group_list_kind", C.c_int32)]


class W4A16Desc(C.Structure):
    _fields_ = [("m", C.c_uint32), ("n", C.c_uint32), ("k", C.c_uint32), ("group_size", C.c_uint32),
                ("has_offset", C.c_int32), ("mode", C.c_int32)]


class W8A16Desc(C.Structure):
    _fields_ = [("m", C.c_uint32), ("n", C.c_uint32), ("k", C.c_uint32), ("per_tensor", C.c_int32),
                ("has_offset", C.c_int32), ("scale", C.c_float), ("offset", C.c_float), ("out_dtype", C.c_int32),
                ("trans_b", C.c_int32), ("mode", C.c_int32)]


W8A16_PER_WEIGHT, W8A16_CHANNEL_SUM = range(2)


class MxDesc(C.Structure):
    _fields_ = [("m", C.c_uint32), ("n", C.c_uint32), ("k", C.c_uint32), ("scale_k", C.c_uint32),
                ("a_format", C.c_int32), ("b_format", C.c_int32), ("out_dtype", C.c_int32), ("has_bias", C.c_int32)]


class MatmulPlan(C.Structure):
    _fields_ = [("kernel", C.c_int32), ("tile_m", C.c_uint32), ("tile_n", C.c_uint32), ("tile_k", C.c_uint32),
                ("workgroups", C.c_uint32), ("k_splits", C.c_uint32), ("launches", C.c_uint32),
                ("lds_bytes", C.c_uint32), ("narrow_tile_n", C.c_uint32), ("narrow_workgroups", C.c_uint32),
                ("workspace_bytes", C.c_size_t)]


MM_KERNEL_GENERIC, MM_KERNEL_STREAM, MM_KERNEL_DMA_128, MM_KERNEL_DMA_256, MM_KERNEL_STAGED = 0, 1, 2, 3, 4

_P = C.c_void_p
# name -> (restype, argtypes): every symbol include/ascq.h declares
SIGNATURES = {
    "ascq_quant": (C.c_int, [C.POINTER(QuantDesc), _P, _P, _P, _P, _P]),
    "ascq_dynamic_quant_per_token": (C.c_int, [C.c_int32, C.c_uint32, C.c_uint32, _P, _P, _P, _P]),
    "ascq_dequant": (C.c_int, [C.POINTER(DequantDesc), _P, _P, _P, _P]),
    "ascq_dequant_dst_stride": (C.c_uint32, [C.c_int32, C.c_uint32]),
    "ascq_antiquant": (C.c_int, [C.POINTER(AntiQuantDesc), _P, _P, _P, _P, _P]),
    "ascq_antiquant_policy": (C.c_int, [C.POINTER(AntiQuantPolicyDesc), _P, _P, _P, _P, _P]),
    "ascq_matmul_w8a8": (C.c_int, [C.POINTER(MatmulDesc), _P, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "ascq_matmul_w8a8_workspace_size": (C.c_int, [C.POINTER(MatmulDesc), C.POINTER(C.c_size_t)]),
    "ascq_linear_w8a8_dynamic": (C.c_int, [C.POINTER(MatmulDesc), C.c_int32, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "ascq_linear_w8a8_dynamic_noalloc": (C.c_int, [C.POINTER(MatmulDesc), C.c_int32, _P, _P, _P, _P, _P, _P]),
    "ascq_matmul_w8a8_plan": (C.c_int, [C.POINTER(MatmulDesc), _P, _P, _P, _P, _P, _P, _P, C.c_size_t,
                                        C.POINTER(MatmulPlan)]),
    "ascq_matmul_w4a4": (C.c_int, [C.POINTER(MatmulDesc), _P, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "ascq_matmul_w4a4_workspace_size": (C.c_int, [C.POINTER(MatmulDesc), C.POINTER(C.c_size_t)]),
    "ascq_unpack_int4": (C.c_int, [_P, _P, C.c_size_t, _P]),
    "ascq_linear_w8a8_dynamic_workspace_size": (C.c_int, [C.POINTER(MatmulDesc), C.POINTER(C.c_size_t)]),
    "ascq_group_matmul_w8a8": (C.c_int, [C.POINTER(GroupMatmulDesc), _P, _P, _P, _P, _P, _P, _P, _P]),
    "ascq_pack_weight_w8_size": (C.c_int, [C.c_uint32, C.c_uint32, C.POINTER(C.c_size_t)]),
    "ascq_pack_weight_w8": (C.c_int, [_P, _P, C.c_uint32, C.c_uint32, C.c_int32, _P]),
    "ascq_matmul_w8a8_packed": (C.c_int, [C.POINTER(MatmulDesc), _P, _P, _P, _P, _P, _P, _P]),
    "ascq_linear_w8a8_dynamic_packed": (C.c_int, [C.POINTER(MatmulDesc), C.c_int32, _P, _P, _P, _P, _P, _P, C.c_size_t,
                                                  _P]),
    "ascq_matmul_w4a16": (C.c_int, [C.POINTER(W4A16Desc), _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "ascq_matmul_w4a16_workspace_size": (C.c_int, [C.POINTER(W4A16Desc), C.POINTER(C.c_size_t)]),
    "ascq_pack_weight_w4_size": (C.c_int, [C.c_uint32, C.c_uint32, C.POINTER(C.c_size_t)]),
    "ascq_pack_weight_w4": (C.c_int, [_P, _P, C.c_uint32, C.c_uint32, _P]),
    "ascq_matmul_w4a16_packed": (C.c_int, [C.POINTER(W4A16Desc), _P, _P, _P, _P, _P, _P]),
    "ascq_matmul_w8a16": (C.c_int, [C.POINTER(W8A16Desc), _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "ascq_matmul_w8a16_workspace_size": (C.c_int, [C.POINTER(W8A16Desc), C.POINTER(C.c_size_t)]),
    "ascq_matmul_mx": (C.c_int, [C.POINTER(MxDesc), _P, _P, _P, _P, _P, _P, _P, C.c_size_t, _P]),
    "ascq_matmul_mx_workspace_size": (C.c_int, [C.POINTER(MxDesc), C.POINTER(C.c_size_t)]),
    "ascq_get_ascend_quant_max_min_tmp_size": (C.c_int, [C.POINTER(C.c_uint32), C.c_uint32, C.c_uint32,
                                                         C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "ascq_get_ascend_dequant_max_min_tmp_size": (C.c_int, [C.POINTER(C.c_uint32), C.c_uint32, C.c_uint32,
                                                           C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "ascq_get_ascend_antiquant_max_min_tmp_size": (C.c_int, [C.POINTER(C.c_uint32), C.c_uint32,
                                                             C.POINTER(C.c_uint32), C.c_uint32, C.c_int32, C.c_int32,
                                                             C.c_int32, C.POINTER(C.c_uint32),
                                                             C.POINTER(C.c_uint32)]),
    "ascq_get_ascend_quant_tmp_buffer_factor_size": (C.c_int, [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]),
    "ascq_get_ascend_dequant_tmp_buffer_factor_size": (C.c_int, [C.POINTER(C.c_uint32), C.c_uint32, C.POINTER(C.c_uint32),
                                                                 C.POINTER(C.c_uint32)]),
    "ascq_get_ascend_antiquant_tmp_buffer_factor_size": (C.c_int, [C.POINTER(C.c_uint32), C.c_uint32,
                                                                   C.POINTER(C.c_uint32), C.c_uint32, C.c_int32, C.c_int32,
                                                                   C.c_int32, C.POINTER(C.c_uint32),
                                                                   C.POINTER(C.c_uint32)]),
    "ascq_pack_quant_param": (C.c_uint64, [C.c_float, C.c_int32, C.c_int32]),
    "ascq_pack_weight_nz": (C.c_int, [C.c_uint32, C.c_uint32, C.c_uint32, _P, _P, _P]),
    "ascq_zero_fill": (C.c_int, [_P, C.c_size_t, _P]),
    "ascq_last_error": (C.c_char_p, []),
    "ascq_version": (C.c_char_p, []),
}

LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib", "libascq.so")
_lib = None


def load_library():
    """Load libascq.so (built in-tree by `make -C asc-devkit_amd/csrc`) and bind every declared symbol."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; "
                           f"g.build()'); there is no fallback path")
    # One HIP runtime per process: torch bundles its own libamdhip64 and this package keeps its tensors in torch's
    # allocations, so torch's copy has to be the one already mapped when libascq.so resolves its dependency;
    # loading libascq.so first would bind it to a second runtime instance that cannot launch on torch's context.
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if a declared symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class AscqError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"{STATUS_NAMES.get(status, status)}: {message}")
        self.status = status


def check(status):
    if status != OK:
        msg = load_library().ascq_last_error()
        raise AscqError(status, msg.decode() if msg else "")
