"""numpy front-end of the CPU oracle (oracle/ascq_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
bench.py's cpu_baseline leg, as the checker.  The product never imports it.
"""
import ctypes as C
import os
import subprocess
import sys

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PKG = os.path.join(os.path.dirname(_HERE), "asc-devkit_amd")
if _PKG not in sys.path:
    sys.path.insert(0, _PKG)
from ascq import _abi as abi  # noqa: E402  (descriptor structs are the ABI's, shared with the library binding)

LIB_PATH = os.path.join(_HERE, "liborc.so")
_lib = None
_P = C.c_void_p


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = C.CDLL(LIB_PATH)
        L.orc_f64_to_f16.restype = C.c_uint16
        L.orc_f64_to_f16.argtypes = [C.c_double]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_round_sat8.restype = C.c_int8
        L.orc_round_sat8.argtypes = [C.c_double, C.c_int]
        L.orc_faster_gelu.restype = C.c_float
        L.orc_faster_gelu.argtypes = [C.c_float]
        L.orc_swiglu.restype = C.c_float
        L.orc_swiglu.argtypes = [C.c_float, C.c_float, C.c_float]
        L.orc_quant_word_scale.restype = C.c_float
        L.orc_quant_word_scale.argtypes = [C.c_uint64, C.c_int]
        L.orc_prescaled_accumulator.restype = C.c_float
        L.orc_prescaled_accumulator.argtypes = [C.c_int32, C.c_uint64, C.c_int, C.c_int]
        L.orc_dequant_dst_stride.restype = C.c_uint32
        L.orc_dequant_dst_stride.argtypes = [C.c_int, C.c_uint32]
        L.orc_f32_to_fp4.restype = C.c_uint8
        L.orc_f32_to_fp4.argtypes = [C.c_float, C.c_int, C.c_int]
        L.orc_fp4_to_f32.restype = C.c_float
        L.orc_fp4_to_f32.argtypes = [C.c_uint8, C.c_int]
        L.orc_f32_to_hif8.restype = C.c_uint8
        L.orc_f32_to_hif8.argtypes = [C.c_float]
        L.orc_hif8_to_f32.restype = C.c_float
        L.orc_hif8_to_f32.argtypes = [C.c_uint8]
        L.orc_set_threads.argtypes = [C.c_int]
        L.orc_quant.argtypes = [C.POINTER(abi.QuantDesc), _P, _P, _P, _P]
        L.orc_dynamic_quant_per_token.argtypes = [C.c_int, C.c_uint32, C.c_uint32, _P, _P, _P]
        L.orc_dequant.argtypes = [C.POINTER(abi.DequantDesc), _P, _P, _P]
        L.orc_antiquant.argtypes = [C.POINTER(abi.AntiQuantDesc), _P, _P, _P, _P]
        L.orc_matmul_w8a8.argtypes = [C.POINTER(abi.MatmulDesc), _P, _P, _P, _P, _P, _P]
        L.orc_matmul_w8a8_rows.argtypes = [C.POINTER(abi.MatmulDesc), _P, _P, _P, _P, _P, _P, C.c_uint32, C.c_uint32]
        L.orc_group_matmul_w8a8.argtypes = [C.POINTER(abi.GroupMatmulDesc), _P, _P, _P, _P, _P, _P, _P]
        L.orc_matmul_w4a16.argtypes = [C.POINTER(abi.W4A16Desc), _P, _P, _P, _P, _P]
        L.orc_matmul_w4a16_cols.argtypes = [C.POINTER(abi.W4A16Desc), _P, _P, _P, _P, _P, C.c_uint32, C.c_uint32]
        L.orc_matmul_w8a16.argtypes = [C.POINTER(abi.W8A16Desc), _P, _P, _P, _P, _P]
        L.orc_matmul_mx.argtypes = [C.POINTER(abi.MxDesc), _P, _P, _P, _P, _P, _P, C.c_uint32, C.c_uint32, C.c_uint32,
                                    C.c_uint32]
        L.orc_antiquant_policy.argtypes = [C.POINTER(abi.AntiQuantPolicyDesc), _P, _P, _P, _P]
        for name in ("orc_f32_to_f16_array", "orc_f16_to_f32_array", "orc_f32_to_bf16_array"):
            getattr(L, name).argtypes = [_P, _P, C.c_size_t]
        for name in ("orc_f16_mul_array", "orc_f16_add_array"):
            getattr(L, name).argtypes = [_P, _P, _P, C.c_size_t]
        L.orc_round_sat8_array.argtypes = [_P, _P, C.c_size_t, C.c_int]
        _lib = L
    return _lib


def set_threads(n):
    lib().orc_set_threads(int(n))


def _ptr(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_P)


_NP = {abi.F16: np.float16, abi.BF16: np.uint16, abi.F32: np.float32, abi.I8: np.int8, abi.I32: np.int32,
       abi.U64: np.uint64}


# ------------------------------------------------------------------ scalar / array numerics
def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_array(_ptr(out), _ptr(x), x.size)
    return out


def f16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_f16_to_f32_array(_ptr(out), _ptr(h), h.size)
    return out


def f32_to_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16_array(_ptr(out), _ptr(x), x.size)
    return out


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f16_mul_bits(a, b):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().orc_f16_mul_array(_ptr(out), _ptr(a), _ptr(b), a.size)
    return out


def f16_add_bits(a, b):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().orc_f16_add_array(_ptr(out), _ptr(a), _ptr(b), a.size)
    return out


def round_sat8(x, round_mode=abi.CAST_RINT):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.int8)
    lib().orc_round_sat8_array(_ptr(out), _ptr(x), x.size, int(round_mode))
    return out


# ------------------------------------------------------------------ operators (host numpy arrays)
def quant(desc, src, scale=None, offset=None):
    if desc.dst_format in (abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2):
        dst = np.zeros(src.size // 2, dtype=np.uint8)      # two codes per byte, even element in the low nibble
        lib().orc_quant(C.byref(desc), _ptr(dst), _ptr(src), _ptr(scale), _ptr(offset))
        return dst.reshape(*src.shape[:-1], src.shape[-1] // 2)
    dst = np.zeros(src.size, dtype=np.int8)
    lib().orc_quant(C.byref(desc), _ptr(dst), _ptr(src), _ptr(scale), _ptr(offset))
    return dst.reshape(src.shape)


def dynamic_quant_per_token(src_dtype, x):
    m, n = x.shape
    q = np.empty((m, n), dtype=np.int8)
    ts = np.empty(m, dtype=np.float32)
    lib().orc_dynamic_quant_per_token(src_dtype, m, n, _ptr(q), _ptr(ts), _ptr(x))
    return q, ts


def dequant(desc, src, scale=None, fill=0):
    """Returns dst [m', stride] (padded columns keep `fill`) after the single-row reshape rule; for PER_TOKEN /
    PER_GROUP m' = cal_count / n, the rows the operator processes."""
    m, n, cal = desc.m, desc.n, desc.cal_count
    if desc.policy >= abi.PER_TOKEN:
        m = cal // n
    per_blk = 8 if desc.dst_dtype == abi.F32 else 16
    if (desc.mode == abi.DEQUANT_WITH_SINGLE_ROW and desc.policy <= abi.PER_CHANNEL and m == 1 and cal
            and cal % per_blk == 0 and n % cal == 0):
        m, n = n // cal, cal
    stride = lib().orc_dequant_dst_stride(desc.dst_dtype, n)
    if desc.dst_dtype == abi.F32:
        dst = np.full((m, stride), fill, dtype=np.float32)
    else:
        dst = np.full((m, stride), fill, dtype=np.uint16)  # `fill` is a bit pattern for the 16-bit types
        if desc.dst_dtype == abi.F16:
            dst = dst.view(np.float16)
    lib().orc_dequant(C.byref(desc), _ptr(dst), _ptr(src), _ptr(scale))
    return dst


def antiquant(desc, src, offset=None, scale=None):
    rows, cols = (desc.n, desc.k) if desc.is_transpose else (desc.k, desc.n)
    dst = np.zeros((rows, cols), dtype=_NP[desc.dst_dtype])
    lib().orc_antiquant(C.byref(desc), _ptr(dst), _ptr(src), _ptr(offset), _ptr(scale))
    return dst


def _out_cols(mm):
    """Columns of the output: n, or n / 2 when the SwiGLU epilogue combines column pairs (activation value 2)."""
    return mm.n // 2 if mm.activation == 2 and mm.quant_mode != 0 else mm.n


def matmul_w8a8(desc, a, b, bias=None, quant_vector=None, tok_scale=None, rows=None):
    c = np.zeros((desc.m, _out_cols(desc)), dtype=_NP[desc.out_dtype])
    if rows is None:
        lib().orc_matmul_w8a8(C.byref(desc), _ptr(c), _ptr(a), _ptr(b), _ptr(bias), _ptr(quant_vector),
                              _ptr(tok_scale))
    else:
        lib().orc_matmul_w8a8_rows(C.byref(desc), _ptr(c), _ptr(a), _ptr(b), _ptr(bias), _ptr(quant_vector),
                                   _ptr(tok_scale), rows[0], rows[1])
    return c


def group_matmul_w8a8(desc, x, w, bias, scale, tok_scale, group_list, fill=0):
    y = np.full((desc.mm.m, _out_cols(desc.mm)), fill, dtype=_NP[desc.mm.out_dtype])
    gl = np.ascontiguousarray(group_list, dtype=np.int64)
    lib().orc_group_matmul_w8a8(C.byref(desc), _ptr(y), _ptr(x), _ptr(w), _ptr(bias), _ptr(scale), _ptr(tok_scale),
                                _ptr(gl))
    return y


def matmul_w4a16(desc, x, w, scale, offset=None, cols=None):
    y = np.zeros((desc.m, desc.n), dtype=np.float16)
    if cols is None:
        lib().orc_matmul_w4a16(C.byref(desc), _ptr(y), _ptr(x), _ptr(w), _ptr(scale), _ptr(offset))
    else:
        lib().orc_matmul_w4a16_cols(C.byref(desc), _ptr(y), _ptr(x), _ptr(w), _ptr(scale), _ptr(offset), cols[0],
                                    cols[1])
    return y


def matmul_w8a16(desc, x, w, offset=None, scale=None):
    y = np.zeros((desc.m, desc.n), dtype=_NP[desc.out_dtype])
    lib().orc_matmul_w8a16(C.byref(desc), _ptr(y), _ptr(x), _ptr(w), _ptr(offset), _ptr(scale))
    return y


def matmul_mx(desc, a, b, a_scale, b_scale, bias=None, rows=None, cols=None):
    """a [m, k] / b [n, k] raw bytes (4-bit formats packed two per byte along k), scales uint8 [rows, scale_k].  Only
    the rows / columns of the given ranges are computed; the rest of the result is zero."""
    c = np.zeros((desc.m, desc.n), dtype=_NP[desc.out_dtype])
    r0, r1 = rows if rows is not None else (0, desc.m)
    c0, c1 = cols if cols is not None else (0, desc.n)
    rc = lib().orc_matmul_mx(C.byref(desc), _ptr(c), _ptr(a), _ptr(b), _ptr(a_scale), _ptr(b_scale), _ptr(bias), r0, r1,
                             c0, c1)
    assert rc == 0
    return c


def antiquant_policy(desc, src, scale, offset=None):
    """src: uint8 / int8 array [m, n] (raw bytes of the one-byte source format)."""
    dst = np.zeros((desc.m, desc.n), dtype=_NP[desc.dst_dtype])
    lib().orc_antiquant_policy(C.byref(desc), _ptr(dst), _ptr(src), _ptr(scale), _ptr(offset))
    return dst



def pack_weight_nz(w):
    """[.., k, n] -> [.., n/32, k/16, 16, 32]: the packing of the reference example's data script
    (quant_group_matmul_high_performance/scripts/gen_data.py:62-64) restated with explicit indices, so that a test
    can hold it against the script's reshape / transpose expression."""
    *lead, k, n = w.shape
    w3 = w.reshape(-1, k, n)
    out = np.empty((w3.shape[0], n // 32, k // 16, 16, 32), dtype=w.dtype)
    for c in range(n // 32):
        for kb in range(k // 16):
            out[:, c, kb] = w3[:, 16 * kb:16 * kb + 16, 32 * c:32 * c + 32]
    return out.reshape(*lead, n // 32, k // 16, 16, 32)
