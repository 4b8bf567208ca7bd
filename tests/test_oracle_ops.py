"""Pins of the oracle's operators: the reference's documented examples, its example golden formulas evaluated with
numpy's own float16 arithmetic, brute-force integer matmul, and closed-form identities."""
import json
import os

import numpy as np
import pytest
import torch

import orc
from ascq import _abi as abi

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "doc_examples.json")))
U16 = np.uint16


def h(x):
    return np.asarray(x, dtype=np.float16)


# ------------------------------------------------------------------ AscendQuant
def quant_desc(**kw):
    d = abi.QuantDesc(policy=abi.PER_TENSOR, src_dtype=abi.F16, scale_dtype=abi.F16, compute=abi.COMPUTE_F16,
                      round_mode=abi.CAST_RINT, offset_kind=abi.OFFSET_SCALAR, k_dim=1, scale=1.0, offset=0.0)
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def test_quant_doc_example():
    g = GOLD["ascend_quant_md_495_509"]
    x = h(g["x"])
    y = orc.quant(quant_desc(scale=g["scale"], offset=g["offset"], cal_count=x.size), x)
    assert list(y[:3]) == g["y_head"] and y[3] == g["y_509"]


def test_quant_per_tensor_matches_example_golden_formula_all_halves():
    # examples/.../03_quantization/quant/scripts/gen_data.py:29 (dav-2201): np.round(src*2.0+0.9) on a half array
    bits = np.arange(65536, dtype=U16)
    x = bits.view(np.float16)
    x = x[np.isfinite(x) & (np.abs(x.astype(np.float32)) <= 60)]
    want = np.round(x * np.float16(2.0) + np.float16(0.9)).astype(np.int8)
    got = orc.quant(quant_desc(scale=2.0, offset=0.9, cal_count=x.size), x)
    assert np.array_equal(got, want)
    # float source is cast to half first (ascend_quant_pre_impl.h:339-343)
    got32 = orc.quant(quant_desc(src_dtype=abi.F32, scale=2.0, offset=0.9, cal_count=x.size), x.astype(np.float32))
    assert np.array_equal(got32, want)


def test_quant_per_channel_half_math_and_saturation():
    rng = np.random.default_rng(5)
    rows, n = 37, 64
    x = h(rng.standard_normal((rows, n)) * 3)
    s = h(rng.uniform(1, 60, n))
    o = h(rng.uniform(-3, 3, n))
    with np.errstate(over="ignore"):
        want = np.clip(np.rint(((x * s) + o).astype(np.float64)), -128, 127).astype(np.int8)  # numpy half ops round once each
    d = quant_desc(policy=abi.PER_CHANNEL, offset_kind=abi.OFFSET_TENSOR, n=n, cal_count=rows * n)
    assert np.array_equal(orc.quant(d, x, s, o), want)
    assert (want == 127).any() and (want == -128).any()
    # invariants: scale 1, offset 0 is the identity on small integers; output is monotone in x
    ints = h(np.arange(-128, 128))
    assert np.array_equal(orc.quant(quant_desc(cal_count=256), ints), np.arange(-128, 128).astype(np.int8))
    xs = np.sort(h(rng.standard_normal(4096) * 50))
    ys = orc.quant(quant_desc(scale=1.7, offset=0.3, cal_count=xs.size), xs)
    assert np.all(np.diff(ys.astype(np.int32)) >= 0)


@pytest.mark.parametrize("rmode", [abi.CAST_RINT, abi.CAST_FLOOR, abi.CAST_CEIL, abi.CAST_ROUND, abi.CAST_TRUNC])
def test_quant_per_token_fp32_and_quantize_agree(rmode):
    rng = np.random.default_rng(6)
    m, n = 10, 288
    x = rng.standard_normal((m, n)).astype(np.float32)
    xb = orc.f32_to_bf16_bits(x)
    s = rng.uniform(5, 90, m).astype(np.float32)
    o = rng.uniform(-2, 2, m).astype(np.float32)
    base = dict(policy=abi.PER_TOKEN, src_dtype=abi.BF16, scale_dtype=abi.F32, round_mode=rmode,
                offset_kind=abi.OFFSET_TENSOR, m=m, n=n, cal_count=m * n)
    a3 = orc.quant(quant_desc(compute=abi.COMPUTE_SCALE_T, **base), xb, s, o)
    a4 = orc.quant(quant_desc(compute=abi.COMPUTE_F32, **base), xb, s, o)
    assert np.array_equal(a3, a4)
    xf = orc.bf16_bits_to_f32(xb)
    v = (xf * s[:, None] + o[:, None]).astype(np.float64)          # numpy fp32 ops: one rounding each
    fn = {abi.CAST_RINT: np.rint, abi.CAST_FLOOR: np.floor, abi.CAST_CEIL: np.ceil, abi.CAST_TRUNC: np.trunc,
          abi.CAST_ROUND: lambda t: np.sign(t) * np.floor(np.abs(t) + 0.5)}[rmode]
    assert np.array_equal(a3, np.clip(fn(v), -128, 127).astype(np.int8).reshape(a3.shape))


@pytest.mark.parametrize("k_dim", [0, 1])
@pytest.mark.parametrize("gs", [32, 64, 128, 256])
def test_quant_per_group_indexing(k_dim, gs):
    rng = np.random.default_rng(7)
    m, n = (10, 256) if k_dim == 1 else (256, 32)
    x = rng.standard_normal((m, n)).astype(np.float32)
    if k_dim == 1:
        s = rng.uniform(5, 60, (m, -(-n // gs))).astype(np.float32)
        sx = np.repeat(s, gs, axis=1)[:, :n]
    else:
        s = rng.uniform(5, 60, (-(-m // gs), n)).astype(np.float32)
        sx = np.repeat(s, gs, axis=0)[:m]
    d = quant_desc(policy=abi.PER_GROUP, src_dtype=abi.F32, scale_dtype=abi.F32, compute=abi.COMPUTE_F32,
                   offset_kind=abi.OFFSET_NONE, k_dim=k_dim, m=m, n=n, cal_count=m * n, group_size=gs)
    want = np.clip(np.rint((x * sx).astype(np.float64)), -128, 127).astype(np.int8)
    assert np.array_equal(orc.quant(d, x, s), want)


def test_quant_half_and_bf16_scale_type_math():
    rng = np.random.default_rng(8)
    m, n = 7, 288
    x = h(rng.standard_normal((m, n)))
    s = h(rng.uniform(5, 90, m))
    d = quant_desc(policy=abi.PER_TOKEN, compute=abi.COMPUTE_SCALE_T, offset_kind=abi.OFFSET_NONE, m=m, n=n,
                   cal_count=m * n)
    want = np.clip(np.rint((x * s[:, None]).astype(np.float64)), -128, 127).astype(np.int8)
    assert np.array_equal(orc.quant(d, x, s), want)
    # bf16: product rounded to bf16 before the integer rounding (checked with torch's bf16 multiply)
    import torch
    xb = torch.randn(m, n, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    sb = (torch.rand(m, generator=torch.Generator().manual_seed(1)) * 80 + 5).to(torch.bfloat16)
    prod = (xb * sb[:, None]).float().numpy().astype(np.float64)
    d = quant_desc(policy=abi.PER_TOKEN, src_dtype=abi.BF16, scale_dtype=abi.BF16, compute=abi.COMPUTE_SCALE_T,
                   offset_kind=abi.OFFSET_NONE, m=m, n=n, cal_count=m * n)
    got = orc.quant(d, xb.view(torch.int16).numpy().view(U16), sb.view(torch.int16).numpy().view(U16))
    assert np.array_equal(got, np.clip(np.rint(prod), -128, 127).astype(np.int8))


def test_dynamic_quant_per_token():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((5, 4096)).astype(np.float32)
    x[3] = 0
    xb = orc.f32_to_bf16_bits(x)
    xf = orc.bf16_bits_to_f32(xb)
    q, ts = orc.dynamic_quant_per_token(abi.BF16, xb)
    amax = np.abs(xf).max(axis=1)
    assert ts[3] == 1.0 and not q[3].any()
    ok = amax > 0
    assert np.array_equal(ts[ok], (amax[ok] / np.float32(127.0)).astype(np.float32))
    inv = (np.float32(127.0) / amax[ok]).astype(np.float32)
    want = np.clip(np.rint((xf[ok] * inv[:, None]).astype(np.float64)), -128, 127).astype(np.int8)
    assert np.array_equal(q[ok], want)
    assert np.abs(q[ok]).max(axis=1).min() == 127  # the row maximum always maps to +-127


# ------------------------------------------------------------------ AscendDequant
def test_dequant_doc_example():
    g = GOLD["ascend_dequant_md_385_401"]
    src = np.array(g["src"], dtype=np.int32)
    scale = np.array(g["scale"], dtype=np.float32)
    d = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.F32,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, m=g["m"], n=g["n"], cal_count=g["cal_count"])
    got = orc.dequant(d, src, scale)
    want = np.array(g["dst"], dtype=np.float32)
    assert np.allclose(got, want, rtol=1e-6, atol=0) and np.array_equal(got[:, 6:], src[:, 6:].astype(np.float32))
    # scalar form of the same example (columns >= calCount converted, not scaled)
    d.policy, d.scale = abi.PER_TENSOR, 2.2
    got = orc.dequant(d, src)
    assert np.array_equal(got[:, :6], (src[:, :6].astype(np.float32) * np.float32(2.2)))
    assert np.array_equal(got[:, 6:], src[:, 6:].astype(np.float32))


@pytest.mark.parametrize("dst,scale_t", [(abi.F16, abi.U64), (abi.F32, abi.F32), (abi.F32, abi.BF16),
                                         (abi.BF16, abi.BF16), (abi.BF16, abi.F32)])
def test_dequant_type_table_and_row_padding(dst, scale_t):
    # examples/.../03_quantization/dequant/scripts/gen_data.py:21-27: golden[j][i] = inp[j][i] * scale[i]
    import torch
    rng = np.random.default_rng(10)
    m, n, cal = 6, 40, 24            # 40 bf16/half columns pad to 48; fp32 rows need no padding
    src = rng.integers(-2**20, 2**20, (m, n), dtype=np.int32)
    sf = rng.uniform(1e-5, 1e-3, n).astype(np.float32)
    if scale_t == abi.BF16:
        sc = orc.f32_to_bf16_bits(sf)
        sf = orc.bf16_bits_to_f32(sc)
    elif scale_t == abi.U64:
        sc = sf.view(np.uint32).astype(np.uint64) | (np.uint64(0x1234) << np.uint64(32))  # the high word is ignored
    else:
        sc = sf
    d = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=scale_t, dst_dtype=dst,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, m=m, n=n, cal_count=cal)
    fill = 0x7E7E if dst != abi.F32 else 0
    got = orc.dequant(d, src, sc, fill=fill)
    v = src.astype(np.float32)
    v[:, :cal] = v[:, :cal] * sf[:cal]
    if dst == abi.F32:
        assert got.shape == (m, 40) and np.array_equal(got, v)
    else:
        assert got.shape == (m, 48)
        t = torch.from_numpy(v)
        want = (t.to(torch.bfloat16) if dst == abi.BF16 else t.to(torch.float16)).view(torch.int16).numpy().view(U16)
        assert np.array_equal(got[:, :40].view(U16), want)
        assert np.all(got[:, 40:].view(U16) == 0x7E7E)      # padding columns are never written


def test_dequant_single_row_reshape_rule():
    # ascend_dequant_common_impl.h:207-223: {1, 16, 8} + fp32 dst becomes {2, 8, 8}; + bf16 dst stays {1, 16, 8}
    src = np.arange(16, dtype=np.int32).reshape(1, 16)
    sc = np.arange(1, 9, dtype=np.float32)
    d = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.F32,
                        mode=abi.DEQUANT_WITH_SINGLE_ROW, m=1, n=16, cal_count=8)
    got = orc.dequant(d, src, sc)
    assert got.shape == (2, 8) and np.array_equal(got, src.reshape(2, 8).astype(np.float32) * sc)
    d.dst_dtype = abi.BF16
    got = orc.bf16_bits_to_f32(orc.dequant(d, src, sc))
    assert got.shape == (1, 16)
    assert np.array_equal(got[0, :8], np.arange(8) * sc) and np.array_equal(got[0, 8:], np.arange(8, 16))
    d.mode, d.dst_dtype = abi.DEQUANT_WITH_MULTI_ROW, abi.F32
    assert orc.dequant(d, src, sc).shape == (1, 16)


def test_dequant_per_token_and_group():
    rng = np.random.default_rng(11)
    m, n, gs = 10, 256, 64
    src = rng.integers(-1000, 1000, (m, n), dtype=np.int32)
    st = rng.uniform(0.01, 1, m).astype(np.float32)
    d = abi.DequantDesc(policy=abi.PER_TOKEN, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.F32,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, m=m, n=n, cal_count=m * n)
    assert np.array_equal(orc.dequant(d, src, st), src.astype(np.float32) * st[:, None])
    # calCount counts elements: calCount / n rows are processed (ascend_dequant_3510_impl.h:230)
    d.cal_count = 3 * n
    assert np.array_equal(orc.dequant(d, src, st), (src.astype(np.float32) * st[:, None])[:3])
    d.cal_count = m * n
    sg = rng.uniform(0.01, 1, (m, n // gs)).astype(np.float32)
    d.policy, d.group_size, d.k_dim = abi.PER_GROUP, gs, 1
    assert np.array_equal(orc.dequant(d, src, sg), src.astype(np.float32) * np.repeat(sg, gs, axis=1))
    m2 = 128
    src2 = rng.integers(-1000, 1000, (m2, 32), dtype=np.int32)
    sg0 = rng.uniform(0.01, 1, (m2 // gs, 32)).astype(np.float32)
    d2 = abi.DequantDesc(policy=abi.PER_GROUP, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.F32,
                         mode=abi.DEQUANT_WITH_MULTI_ROW, k_dim=0, m=m2, n=32, cal_count=m2 * 32, group_size=gs)
    assert np.array_equal(orc.dequant(d2, src2, sg0), src2.astype(np.float32) * np.repeat(sg0, gs, axis=0))


# ------------------------------------------------------------------ AscendAntiQuant
def aq_desc(**kw):
    d = abi.AntiQuantDesc(src_dtype=abi.I8, dst_dtype=abi.F16, is_transpose=0, has_offset=1, per_tensor=0)
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def test_antiquant_doc_example():
    g = GOLD["ascend_antiquant_md_469_490"]
    src = np.full((g["k"], g["n"]), g["src"], dtype=np.int8)
    off = h(np.full((1, g["n"]), g["offset"]))
    sc = h(np.full((1, g["n"]), g["scale"]))
    got = orc.antiquant(aq_desc(k=g["k"], n=g["n"], scale_height=1, scale_width=g["n"], offset_height=1,
                                offset_width=g["n"]), src, off, sc)
    assert np.all(got == np.float16(g["dst"]))


def test_antiquant_example_golden_formula():
    # examples/.../03_quantization/antiquant/scripts/gen_data.py:27-39 (seed 10, dav-2201: half arithmetic)
    np.random.seed(10)
    src = np.random.uniform(-10, 10, [8, 128]).astype(np.int8)
    offset = np.random.uniform(-10, 10, [1, 128]).astype(np.float16)
    scale = np.random.uniform(-10, 10, [1, 128]).astype(np.float16)
    want = (scale * (src.astype(np.float16) + offset)).astype(np.float16)
    got = orc.antiquant(aq_desc(k=8, n=128, scale_height=1, scale_width=128), src, offset, scale)
    assert np.array_equal(got.view(U16), want.view(U16))
    # bf16 output: fp32 add and multiply, one rounding to bf16 (ascend_antiquant_c220_impl.h:58-75)
    import torch
    ob, sb = orc.f32_to_bf16_bits(offset.astype(np.float32)), orc.f32_to_bf16_bits(scale.astype(np.float32))
    v = (src.astype(np.float32) + orc.bf16_bits_to_f32(ob)) * orc.bf16_bits_to_f32(sb)
    wantb = torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(U16)
    gotb = orc.antiquant(aq_desc(dst_dtype=abi.BF16, k=8, n=128, scale_height=1, scale_width=128), src, ob, sb)
    assert np.array_equal(gotb, wantb)


@pytest.mark.parametrize("transpose", [0, 1])
def test_antiquant_all_int8_and_int4_values_per_group(transpose):
    rng = np.random.default_rng(12)
    K, N, G = 256, 32, 4
    gs = K // G
    w8 = np.tile(np.arange(-128, 128, dtype=np.int8)[:, None], (1, N))          # every int8 value in every column
    w4 = rng.integers(-8, 8, (K, N)).astype(np.int8)
    w4[:16, :] = np.arange(-8, 8, dtype=np.int8)[:, None]
    sc = h(rng.uniform(-2, 2, (G, N)))
    of = h(rng.uniform(-9, 9, (G, N)))
    for src, dt in ((w8, abi.I8), (w4, abi.I4)):
        want = (np.repeat(sc, gs, 0) * (src.astype(np.float16) + np.repeat(of, gs, 0))).astype(np.float16)
        s_in, sc_in, of_in = src, sc, of
        if transpose:
            s_in, sc_in, of_in = (np.ascontiguousarray(t.T) for t in (src, sc, of))
            want = np.ascontiguousarray(want.T)
        if dt == abi.I4:
            flat = s_in.reshape(-1).astype(np.uint8) & 0xF
            s_in = (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)           # even element in the low nibble
        if transpose:
            d = aq_desc(src_dtype=dt, is_transpose=1, k=K, n=N, scale_height=N, scale_width=G, offset_height=N,
                        offset_width=G)
        else:
            d = aq_desc(src_dtype=dt, k=K, n=N, scale_height=G, scale_width=N, offset_height=G, offset_width=N)
        got = orc.antiquant(d, s_in, of_in, sc_in)
        assert np.array_equal(got.view(U16), want.view(U16))
        d.has_offset = 0                                                         # scale-only overload
        want0 = (np.repeat(sc, gs, 0) * src.astype(np.float16)).astype(np.float16)
        got0 = orc.antiquant(d, s_in, None, sc_in)
        assert np.array_equal(got0.view(U16), (want0.T if transpose else want0).copy().view(U16))


def test_antiquant_per_tensor_scalar():
    src = np.arange(-128, 128, dtype=np.int8).reshape(8, 32)
    d = aq_desc(per_tensor=1, scale=0.37, offset=-3.25, k=8, n=32)
    want = (np.float16(0.37) * (src.astype(np.float16) + np.float16(-3.25))).astype(np.float16)
    assert np.array_equal(orc.antiquant(d, src).view(U16), want.view(U16))


# ------------------------------------------------------------------ Matmul quant path
def mm_desc(m, n, k, **kw):
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.I32, quant_mode=abi.MM_QUANT_NONE, scale_format=abi.MM_SCALE_F32)
    for key, v in kw.items():
        setattr(d, key, v)
    return d


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_matmul_int32_brute_force_and_identities(ta, tb):
    rng = np.random.default_rng(13)
    m, n, k = 19, 23, 77
    a = rng.integers(-128, 128, (m, k)).astype(np.int8)
    b = rng.integers(-128, 128, (k, n)).astype(np.int8)
    bias = rng.integers(-1000, 1000, n).astype(np.int32)
    want = a.astype(np.int64) @ b.astype(np.int64) + bias
    a_in = np.ascontiguousarray(a.T) if ta else a
    b_in = np.ascontiguousarray(b.T) if tb else b
    got = orc.matmul_w8a8(mm_desc(m, n, k, trans_a=ta, trans_b=tb, bias_kind=abi.MM_BIAS_I32_PRE), a_in, b_in, bias)
    assert np.array_equal(got.astype(np.int64), want)
    ones = np.ones((m, k), dtype=np.int8)
    got = orc.matmul_w8a8(mm_desc(m, n, k, trans_b=tb), ones, b_in)
    assert np.array_equal(got[0], b.astype(np.int64).sum(axis=0))           # A = 1 gives the column sums of B


def spec_extract_scale(word):
    # fixpipe_l0c2gm/scripts/gen_data_s322f16.py:37-66: bits [31:13] decoded as sign, 8 exponent, 10 mantissa bits
    bits = (int(word) >> 13) & 0x7FFFF
    sign, exponent, mantissa = (bits >> 18) & 1, (bits >> 10) & 0xFF, bits & 0x3FF
    return (-1) ** sign * (1 + mantissa / 1024) * (2.0 ** (exponent - 127))


def test_quant_word_scale_keeps_19_bits():
    rng = np.random.default_rng(14)
    s = np.concatenate([rng.uniform(1e-4, 2.0, 2000), -rng.uniform(1e-4, 2.0, 200)]).astype(np.float32)
    L = orc.lib()
    for v in s:
        w = int(np.float32(v).view(np.uint32)) | (0x155 << 37) | (1 << 46)
        assert L.orc_quant_word_scale(w, abi.MM_SCALE_U64) == np.float32(spec_extract_scale(w))
        assert L.orc_quant_word_scale(w, abi.MM_SCALE_F32) == v


def test_matmul_deqf16_vector_follows_fixpipe_spec():
    rng = np.random.default_rng(15)
    m, n, k = 16, 48, 64
    a = rng.integers(-10, 10, (m, k)).astype(np.int8)
    b = rng.integers(-10, 10, (k, n)).astype(np.int8)
    bias = rng.integers(-2, 2, n).astype(np.int32)
    qf = rng.uniform(0.1, 2.0, n).astype(np.float32)
    qf[0], qf[1] = 3000.0, -3000.0                      # forces fp16 saturation on both sides
    qv = qf.view(np.uint32).astype(np.uint64)
    acc = a.astype(np.int64) @ b.astype(np.int64) + bias
    acc[:, 0] = np.abs(acc[:, 0]) + 30
    # deqf16 (gen_data_s322f16.py:76-102): fp32 multiply by the 19-bit scale, clip to the fp16 range, round to fp16
    trunc = (qf.view(np.uint32) & np.uint32(0xFFFFE000)).view(np.float32)
    d = mm_desc(m, n, k, out_dtype=abi.F16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_U64,
                bias_kind=abi.MM_BIAS_I32_PRE)
    got = orc.matmul_w8a8(d, a, b, bias, qv)
    acc2 = a.astype(np.int64) @ b.astype(np.int64) + bias
    want = np.clip(acc2.astype(np.float32) * trunc, -65504, 65504).astype(np.float16)
    assert np.array_equal(got.view(U16), want.view(U16))
    assert (np.abs(want.astype(np.float32)) == 65504).any()
    # the matmul_quant example's own golden (gen_data.py:26-42 casts acc to half first) agrees within its gate
    gold = (acc2.astype(np.float16).astype(np.float32) * trunc)
    okc = np.abs(gold) < 60000
    assert np.isclose(got.astype(np.float32)[okc], gold[okc], rtol=1e-3, atol=1e-3).mean() > 0.999
    # scalar mode
    d.quant_mode, d.quant_scalar = abi.MM_QUANT_SCALAR, int(np.float32(0.1).view(np.uint32))
    got = orc.matmul_w8a8(d, a, b, bias)
    s01 = (np.float32(0.1).view(np.uint32) & np.uint32(0xFFFFE000)).view(np.float32)
    assert np.array_equal(got.view(U16), (acc2.astype(np.float32) * s01).astype(np.float16).view(U16))


def _fixpipe_fields(word):
    """extract_quant_params of the reference's golden scripts (gen_data_s322f16.py:37-66), field by field."""
    bits = (word >> 13) & 0xFFFFF
    sign_bit, exponent, mantissa = (bits >> 18) & 1, (bits >> 10) & 0xFF, bits & 0x3FF
    alpha = (-1) ** sign_bit * (1 + mantissa / 1024) * (2.0 ** (exponent - 127))
    return np.float32(alpha), (word >> 37) & 0x1FF, (word >> 46) & 1, (word >> 32) & 0xF, (word >> 36) & 1


def test_matmul_pre_shift_follows_fixpipe_scripts():
    """Mode-control bit 36: the scripts shift the accumulator right by bits [35:32] and saturate it (to the half range,
    cast to half, in gen_data_s322f16.py:84-90; to int16 in gen_data_s322s8.py:84-86) before the multiply.  The
    expected values below follow those lines with numpy's own >>, clip and casts."""
    rng = np.random.default_rng(77)
    m, n, k = 12, 40, 256
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    bias = rng.integers(-2000000, 2000000, n).astype(np.int32)       # accumulators beyond the half range and int16
    acc = (a.astype(np.int64) @ b.astype(np.int64) + bias).astype(np.int32)
    assert (np.abs(acc) > 70000).any() and (acc < 0).any()
    scales = rng.uniform(0.01, 1.5, n).astype(np.float32)
    shifts = rng.integers(0, 16, n)
    on = rng.integers(0, 2, n)
    on[:4], shifts[:4] = 1, (0, 1, 4, 15)
    words = np.array([int(np.float32(s).view(np.uint32)) | (int(sh) << 32) | (int(o) << 36)
                      for s, sh, o in zip(scales, shifts, on)], dtype=np.uint64)
    # ---- half output (DEQF16)
    d = mm_desc(m, n, k, out_dtype=abi.F16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_U64,
                bias_kind=abi.MM_BIAS_I32_PRE)
    got = orc.matmul_w8a8(d, a, b, bias, words)
    want = np.empty((m, n), np.float16)
    for j in range(n):
        alpha, _, _, n_shift, mode = _fixpipe_fields(int(words[j]))
        data = acc[:, j]
        if mode == 1:
            data = np.clip(data >> n_shift, np.finfo(np.float16).min, np.finfo(np.float16).max).astype(np.float16)
        want[:, j] = np.clip(data.astype(np.float32) * alpha, -65504, 65504).astype(np.float16)
    assert np.array_equal(got.view(U16), want.view(U16))
    L = orc.lib()
    # what the arithmetic fixes: a shift of 0 on accumulators a half holds exactly changes nothing; negative
    # accumulators round towards minus infinity (-1 >> 4 == -1)
    assert L.orc_prescaled_accumulator(1234, (1 << 36), abi.MM_SCALE_U64, abi.F16) == 1234.0
    assert L.orc_prescaled_accumulator(-1, (1 << 36) | (4 << 32), abi.MM_SCALE_U64, abi.F16) == -1.0
    assert L.orc_prescaled_accumulator(-4096, (1 << 36) | (4 << 32), abi.MM_SCALE_U64, abi.F16) == -256.0
    assert L.orc_prescaled_accumulator(2 ** 31 - 1, (1 << 36), abi.MM_SCALE_U64, abi.F16) == 65504.0
    assert L.orc_prescaled_accumulator(-2 ** 31, (1 << 36), abi.MM_SCALE_U64, abi.I8) == -32768.0
    assert L.orc_prescaled_accumulator(4097, (1 << 36), abi.MM_SCALE_U64, abi.F16) == 4096.0      # rounded to half
    assert L.orc_prescaled_accumulator(4097, (4 << 32), abi.MM_SCALE_U64, abi.F16) == 4097.0      # bit 36 clear
    assert L.orc_prescaled_accumulator(4097, (1 << 36), abi.MM_SCALE_F32, abi.F16) == 4097.0      # plain float scales
    # ---- 8-bit output (REQ8): shift, saturate to int16, multiply, round, 9 bits, + offset, 8 bits
    offs = rng.integers(0, 512, n)
    sgn = rng.integers(0, 2, n)
    words8 = np.array([int(w) | (int(o) << 37) | (int(sg) << 46) for w, o, sg in zip(words, offs, sgn)], dtype=np.uint64)
    d8 = mm_desc(m, n, k, out_dtype=abi.I8, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_U64,
                 bias_kind=abi.MM_BIAS_I32_PRE)
    got8 = orc.matmul_w8a8(d8, a, b, bias, words8)
    for j in range(n):
        alpha, offset, sign, n_shift, mode = _fixpipe_fields(int(words8[j]))
        data = acc[:, j]
        if mode == 1:
            data = np.clip(data >> n_shift, -32768, 32767).astype(np.int16)
        q = np.clip(np.rint(data.astype(np.float32) * alpha), -256, 255).astype(np.int16) + offset
        w8 = np.clip(q, -128, 127) if sign else np.clip(q, 0, 255)
        assert np.array_equal(got8[:, j].view(np.uint8), w8.astype(np.int64).astype(np.uint8)), j


def test_matmul_req8_follows_spec():
    # gen_data_s322s8.py:76-97: round, clip to [-256, 255], add the 9-bit offset, clip to int8 (sign = 1)
    rng = np.random.default_rng(16)
    m, n, k = 8, 32, 32
    a = rng.integers(-20, 20, (m, k)).astype(np.int8)
    b = rng.integers(-20, 20, (k, n)).astype(np.int8)
    scale, off = np.float32(0.0625), 5
    word = int(scale.view(np.uint32)) | (off << 37) | (1 << 46)
    d = mm_desc(m, n, k, out_dtype=abi.I8, quant_mode=abi.MM_QUANT_SCALAR, scale_format=abi.MM_SCALE_U64,
                quant_scalar=word)
    acc = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    want = np.clip(np.clip(np.rint(acc * scale), -256, 255) + off, -128, 127).astype(np.int8)
    assert np.array_equal(orc.matmul_w8a8(d, a, b), want)


def test_matmul_bf16_epilogue_order_token_scale_and_bias():
    import torch
    rng = np.random.default_rng(17)
    m, n, k = 9, 40, 128
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-3, 1e-1, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    acc = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    v = (acc * cs) * ts[:, None] + bias                     # numpy fp32: one rounding per operation, this order
    want = torch.from_numpy(v).to(torch.bfloat16).view(torch.int16).numpy().view(U16)
    d = mm_desc(m, n, k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, bias_kind=abi.MM_BIAS_F32_POST,
                has_tok_scale=1)
    assert np.array_equal(orc.matmul_w8a8(d, a, b, bias, cs, ts), want)


def fast_gelu(x):
    # quant_group_matmul_high_performance/scripts/gen_data.py:19-23
    ax = np.abs(x)
    return x * np.exp(0.851 * (x - ax)) / (1 + np.exp(-1.702 * ax))


@pytest.mark.parametrize("kind", [abi.GROUP_LIST_COUNTS, abi.GROUP_LIST_PREFIX_SUM])
def test_group_matmul_against_example_golden(kind):
    rng = np.random.default_rng(18)
    G, m, k, n = 5, 96, 64, 48
    counts = np.array([30, 0, 1, 45, 12], dtype=np.int64)      # an empty group, a one-row group, 8 unassigned rows
    x = rng.integers(-10, 10, (m, k)).astype(np.int8)
    w = rng.integers(-10, 10, (G, k, n)).astype(np.int8)
    scale = rng.normal(0, 0.01, (G, n)).astype(np.float32)
    tok = rng.normal(0, 0.01, m).astype(np.float32)
    d = abi.GroupMatmulDesc(mm=mm_desc(m, n, k, out_dtype=abi.F16, quant_mode=abi.MM_QUANT_VECTOR, has_tok_scale=1,
                                       activation=abi.MM_ACT_FASTER_GELU), groups=G, group_list_kind=kind)
    gl = counts if kind == abi.GROUP_LIST_COUNTS else np.cumsum(counts)
    got = orc.group_matmul_w8a8(d, x, w, None, scale, tok, gl, fill=np.float16(777).view(U16).item()
                                if False else 0)
    idx = np.concatenate([[0], np.cumsum(counts)])
    gold = np.zeros((m, n), dtype=np.float64)
    for g in range(G):
        s, e = idx[g], idx[g + 1]
        gold[s:e] = (x[s:e].astype(np.float64) @ w[g].astype(np.float64)) * scale[g].astype(np.float64) \
            * tok[s:e, None].astype(np.float64)
    gold = fast_gelu(gold)
    rows = idx[-1]
    # the example's gate: rtol = atol = 1e-3, at most 0.01 % mismatches (scripts/verify_result.py:19-21)
    assert np.isclose(got[:rows].astype(np.float64), gold[:rows], rtol=1e-3, atol=1e-3).mean() >= 0.9999
    assert not got[rows:].any()                                # rows past the last group are left alone


def test_w4a16_against_numpy_half_dequant():
    rng = np.random.default_rng(19)
    M, K, N, gs = 3, 256, 64, 128
    x = h(rng.standard_normal((M, K)))
    wq = rng.integers(-8, 8, (K, N)).astype(np.int8)
    flat = wq.reshape(-1).astype(np.uint8) & 0xF
    packed = (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8)
    sc = h(rng.uniform(1e-3, 1e-2, (K // gs, N)))
    of = h(rng.integers(-8, 8, (K // gs, N)))
    wdq = (np.repeat(sc, gs, 0) * (wq.astype(np.float16) + np.repeat(of, gs, 0))).astype(np.float16)
    want = (x.astype(np.float64) @ wdq.astype(np.float64)).astype(np.float16)
    d = abi.W4A16Desc(m=M, n=N, k=K, group_size=gs, has_offset=1)
    got = orc.matmul_w4a16(d, x, packed, sc, of)
    assert np.array_equal(got.view(U16), want.view(U16))
    sub = orc.matmul_w4a16(d, x, packed, sc, of, cols=(8, 24))
    assert np.array_equal(sub[:, 8:24].view(U16), want[:, 8:24].view(U16))


@pytest.mark.parametrize("per_tensor", [False, True])
@pytest.mark.parametrize("has_offset", [True, False])
def test_w8a16_is_antiquant_then_half_matmul(per_tensor, has_offset):
    """The W8A16 oracle = the AscendAntiQuant<int8_t, half> oracle (pinned by the documentation examples) applied to
    B, followed by numpy's float64 matmul and one rounding; non-integer offsets make both half roundings matter."""
    rng = np.random.default_rng(23 + per_tensor + 2 * has_offset)
    M, K, N = 5, 192, 80
    x = h(rng.standard_normal((M, K)))
    w = rng.integers(-128, 128, (K, N)).astype(np.int8)
    if per_tensor:
        sc_s, of_s = 0.0123, 3.3
        sc, of = h(np.full(N, sc_s)), h(np.full(N, of_s))
    else:
        sc, of = h(rng.uniform(1e-3, 1e-2, N)), h(rng.uniform(-9, 9, N))
    wdq = (sc[None, :] * ((w.astype(np.float16) + of[None, :]).astype(np.float16) if has_offset
                          else w.astype(np.float16))).astype(np.float16)
    ad = aq_desc(has_offset=int(has_offset), k=K, n=N, scale_height=1, scale_width=N, offset_height=1, offset_width=N)
    assert np.array_equal(orc.antiquant(ad, w, of[None, :] if has_offset else None, sc[None, :]).view(U16),
                          wdq.view(U16))
    for out_dtype, npdt in ((abi.F16, np.float16), (abi.F32, np.float32)):
        d = abi.W8A16Desc(m=M, n=N, k=K, per_tensor=int(per_tensor), has_offset=int(has_offset),
                          scale=sc_s if per_tensor else 0.0, offset=of_s if per_tensor else 0.0, out_dtype=out_dtype)
        got = orc.matmul_w8a16(d, x, w, None if per_tensor else (of if has_offset else None),
                               None if per_tensor else sc)
        want = (x.astype(np.float64) @ wdq.astype(np.float64)).astype(npdt)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("fmt,tdt,top", [(abi.QDST_FP8_E4M3FN, torch.float8_e4m3fn, 448.0),
                                         (abi.QDST_FP8_E5M2, torch.float8_e5m2, 57344.0)])
@pytest.mark.parametrize("sc_dt", [abi.F16, abi.F32])
def test_quant_fp8_is_fp32_arithmetic_then_one_conversion(fmt, tdt, top, sc_dt):
    """8-bit float outputs: source and parameters widened to fp32, one fp32 multiply, one fp32 add, one conversion
    (ascend_quant_per_group_3510_impl.h:54-74), checked against numpy fp32 arithmetic + torch's float8 conversion on
    data kept below the overflow threshold; whatever the scale dtype or `compute` says."""
    rng = np.random.default_rng(fmt * 10 + sc_dt)
    m, n = 6, 64
    x = h(rng.standard_normal((m, n)))
    npdt = np.float16 if sc_dt == abi.F16 else np.float32
    s = rng.uniform(1e-3, top / 8, m).astype(npdt)
    o = rng.uniform(-1, 1, m).astype(npdt)
    v = (x.astype(np.float32) * s.astype(np.float32)[:, None]) + o.astype(np.float32)[:, None]
    assert np.abs(v).max() < top
    want = torch.from_numpy(v).to(tdt).view(torch.uint8).numpy()
    for compute in (abi.COMPUTE_SCALE_T, abi.COMPUTE_F32):
        d = abi.QuantDesc(policy=abi.PER_TOKEN, src_dtype=abi.F16, scale_dtype=sc_dt, compute=compute,
                          round_mode=abi.CAST_FLOOR, offset_kind=abi.OFFSET_TENSOR, k_dim=1, m=m, n=n, cal_count=m * n,
                          dst_format=fmt)
        assert np.array_equal(orc.quant(d, x, s, o).view(np.uint8), want)


@pytest.mark.parametrize("fmt", [abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2])
@pytest.mark.parametrize("src_t,sc_t", [(torch.float16, torch.float16), (torch.float16, torch.float32),
                                        (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("k_dim", [0, 1])
def test_quant_fp4_is_a_product_in_the_scale_type_then_bf16_then_fp4(fmt, src_t, sc_t, k_dim):
    """fp4 outputs (ascend_quant_per_group_3510_impl.h:346-379, ascend_quant_3510_impl.h:994-1032): the product is
    formed in the scale's type by torch (an independent implementation of half / bfloat16 / float multiplication),
    rounded to bfloat16 by torch, converted element by element with the scalar conversion pinned in
    test_oracle_numerics.py, and packed with the even element in the low nibble; the offset must have no effect."""
    rng = np.random.default_rng(fmt + k_dim)
    m, n, gs = 64, 96, 32
    xt = torch.from_numpy(rng.standard_normal((m, n)).astype(np.float32)).to(src_t)
    sshape = (m, n // gs) if k_dim == 1 else (m // gs, n)
    st = torch.from_numpy(rng.uniform(0.1, 8.0, sshape).astype(np.float32)).to(sc_t)
    full = st.repeat_interleave(gs, dim=1) if k_dim == 1 else st.repeat_interleave(gs, dim=0)
    prod = (xt.to(sc_t) * full).to(torch.bfloat16).to(torch.float32).numpy()
    e1m2 = int(fmt == abi.QDST_FP4_E1M2)
    L = orc.lib()
    codes = np.array([L.orc_f32_to_fp4(float(v), e1m2, abi.CAST_ROUND) for v in prod.reshape(-1)], dtype=np.uint8)
    want = (codes[0::2] | (codes[1::2] << 4)).astype(np.uint8)

    def raw(t):
        return t.view(torch.int16).numpy().view(np.uint16) if t.dtype != torch.float32 else t.numpy()

    x_np = raw(xt) if src_t == torch.bfloat16 else xt.numpy()
    s_np = raw(st) if sc_t == torch.bfloat16 else st.numpy()
    o_np = (np.full(sshape, 5.0, dtype=np.float32) if sc_t == torch.float32
            else raw(torch.full(sshape, 5.0).to(sc_t)) if sc_t == torch.bfloat16 else np.full(sshape, 5.0, np.float16))
    d = abi.QuantDesc(policy=abi.PER_GROUP, src_dtype=abi.F16 if src_t == torch.float16 else abi.BF16,
                      scale_dtype={torch.float16: abi.F16, torch.bfloat16: abi.BF16, torch.float32: abi.F32}[sc_t],
                      compute=abi.COMPUTE_SCALE_T, round_mode=abi.CAST_ROUND, offset_kind=abi.OFFSET_TENSOR,
                      k_dim=k_dim, m=m, n=n, cal_count=m * n, group_size=gs, dst_format=fmt)
    got = orc.quant(d, x_np, s_np, o_np)
    assert got.shape == (m, n // 2) and np.array_equal(got.reshape(-1), want)


# ------------------------------------------------------------------ AscendAntiQuant PER_TOKEN / PER_GROUP
def _b8_source(rng, fmt, shape):
    """Random one-byte sources (no NaN / infinity codes) and their exact fp32 values."""
    codes = rng.integers(0, 256, shape).astype(np.uint8)
    if fmt == abi.QDST_I8:
        return codes, codes.view(np.int8).astype(np.float32)
    if fmt == abi.QDST_FP8_E4M3FN:
        codes[(codes & 0x7F) == 0x7F] = 0x3C
        return codes, torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    codes[(codes & 0x7F) >= 0x7C] = 0x3C
    return codes, torch.from_numpy(codes).view(torch.float8_e5m2).float().numpy()


@pytest.mark.filterwarnings("ignore:overflow encountered")      # half arithmetic on the largest e5m2 values overflows
@pytest.mark.parametrize("fmt", [abi.QDST_I8, abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2])
@pytest.mark.parametrize("mode", ["token", "group_n", "group_m", "group_n_via_transpose"])
def test_antiquant_policy_against_numpy_and_torch_arithmetic(fmt, mode):
    """(src + offset) * scale in the scale's type: numpy float16 arithmetic, torch bfloat16 arithmetic (both round
    once per operation) and numpy float32 arithmetic are the independent implementations; the group axis is
    kDim XOR isTranspose (ascend_antiquant_3510_impl.h:2204-2212)."""
    rng = np.random.default_rng(31 + fmt)
    m, n, gs = 64, 96, 32
    codes, x = _b8_source(rng, fmt, (m, n))
    policy = abi.PER_TOKEN if mode == "token" else abi.PER_GROUP
    k_dim, tr = {"token": (1, 0), "group_n": (1, 0), "group_m": (0, 0), "group_n_via_transpose": (0, 1)}[mode]
    if mode == "token":
        pshape, expand = (m,), lambda p: p[:, None]
    elif mode == "group_m":
        pshape, expand = (m // gs, n), lambda p: np.repeat(p, gs, axis=0)
    else:
        pshape, expand = (m, n // gs), lambda p: np.repeat(p, gs, axis=1)
    s32 = rng.uniform(0.01, 2.0, pshape).astype(np.float32)
    o32 = rng.uniform(-3.0, 3.0, pshape).astype(np.float32)

    def desc(sc_dt, dst_dt, compute):
        return abi.AntiQuantPolicyDesc(policy=policy, src_format=fmt, scale_dtype=sc_dt, dst_dtype=dst_dt,
                                       compute=compute, has_offset=1, is_transpose=tr, k_dim=k_dim, m=m, n=n,
                                       cal_count=m * n, group_size=gs if policy == abi.PER_GROUP else 0)

    # half arithmetic
    s16, o16 = s32.astype(np.float16), o32.astype(np.float16)
    want = ((x.astype(np.float16) + expand(o16)).astype(np.float16) * expand(s16)).astype(np.float16)
    got = orc.antiquant_policy(desc(abi.F16, abi.F16, abi.COMPUTE_SCALE_T), codes, s16, o16)
    assert np.array_equal(got.view(U16), want.view(U16))
    # bfloat16 arithmetic
    sb, ob = torch.from_numpy(s32).bfloat16(), torch.from_numpy(o32).bfloat16()
    tb = (torch.from_numpy(x).bfloat16() + torch.from_numpy(expand(ob.float().numpy())).bfloat16())
    wantb = (tb * torch.from_numpy(expand(sb.float().numpy())).bfloat16()).view(torch.int16).numpy().view(U16)
    gotb = orc.antiquant_policy(desc(abi.BF16, abi.BF16, abi.COMPUTE_SCALE_T), codes,
                                sb.view(torch.int16).numpy().view(U16), ob.view(torch.int16).numpy().view(U16))
    assert np.array_equal(gotb.view(U16), wantb)
    # fp32 arithmetic, fp32 and half outputs; and AntiQuantize (fp32 arithmetic on half parameters)
    want32 = (x + expand(o32)) * expand(s32)
    assert np.array_equal(orc.antiquant_policy(desc(abi.F32, abi.F32, abi.COMPUTE_SCALE_T), codes, s32, o32), want32)
    got16 = orc.antiquant_policy(desc(abi.F32, abi.F16, abi.COMPUTE_SCALE_T), codes, s32, o32)
    sat = lambda v: np.clip(v, -65504.0, 65504.0).astype(np.float16)   # the fp32 -> half cast saturates (RndR SatS)
    assert np.array_equal(got16.view(U16), sat(want32).view(U16))
    wantq = sat((x + expand(o16).astype(np.float32)) * expand(s16).astype(np.float32))
    gotq = orc.antiquant_policy(desc(abi.F16, abi.F16, abi.COMPUTE_F32), codes, s16, o16)
    assert np.array_equal(gotq.view(U16), wantq.view(U16))


def test_pack_weight_nz_is_the_data_scripts_reshape_transpose():
    """The explicit-index packing against the expression of the reference example's script (gen_data.py:62-64), and
    the element address the C header states."""
    rng = np.random.default_rng(62)
    g, k, n = 3, 48, 96
    w = rng.integers(-128, 128, (g, k, n)).astype(np.int8)
    want = w.reshape([g, k // 16, 16, n // 32, 32]).transpose([0, 3, 1, 2, 4])
    got = orc.pack_weight_nz(w)
    assert got.shape == (g, n // 32, k // 16, 16, 32) and np.array_equal(got, want)
    flat = got.reshape(-1)
    for gi, kk, c in [(0, 0, 0), (1, 17, 33), (2, 47, 95), (1, 16, 31), (0, 15, 32)]:
        assert flat[((gi * (n // 32) + c // 32) * k + kk) * 32 + c % 32] == w[gi, kk, c]


@pytest.mark.filterwarnings("ignore:overflow encountered")
@pytest.mark.parametrize("fmt", [abi.QDST_I8, abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2])
def test_antiquantize_per_channel_and_per_tensor_against_numpy_fp32(fmt):
    """AntiQuantize PER_CHANNEL / PER_TENSOR (antiquantize_3510_impl.h:253-362): parameters of the output's type are
    widened to fp32, (src + offset) * scale in fp32 (numpy), one saturating half-even cast (numpy / torch)."""
    rng = np.random.default_rng(53 + fmt)
    m, n = 48, 64
    codes, x = _b8_source(rng, fmt, (m, n))
    s16 = rng.uniform(0.01, 2.0, n).astype(np.float16)
    o16 = rng.uniform(-3.0, 3.0, n).astype(np.float16)
    sat = lambda v: np.clip(v, -65504.0, 65504.0).astype(np.float16)

    def desc(policy, dst_dt, has_offset=1, **kw):
        return abi.AntiQuantPolicyDesc(policy=policy, src_format=fmt, scale_dtype=dst_dt, dst_dtype=dst_dt,
                                       compute=abi.COMPUTE_F32, has_offset=has_offset, is_transpose=0, k_dim=1, m=m,
                                       n=n, cal_count=m * n, group_size=0, **kw)

    want = sat((x + o16.astype(np.float32)[None, :]) * s16.astype(np.float32)[None, :])
    got = orc.antiquant_policy(desc(abi.PER_CHANNEL, abi.F16), codes, s16, o16)
    assert np.array_equal(got.view(U16), want.view(U16))
    want = sat(x * s16.astype(np.float32)[None, :])
    got = orc.antiquant_policy(desc(abi.PER_CHANNEL, abi.F16, has_offset=0), codes, s16, None)
    assert np.array_equal(got.view(U16), want.view(U16))
    # bfloat16 parameters and output
    sb, ob = torch.from_numpy(s16.astype(np.float32)).bfloat16(), torch.from_numpy(o16.astype(np.float32)).bfloat16()
    wantb = ((torch.from_numpy(x) + ob.float()[None, :]) * sb.float()[None, :]).bfloat16()
    gotb = orc.antiquant_policy(desc(abi.PER_CHANNEL, abi.BF16), codes, sb.view(torch.int16).numpy().view(U16),
                                ob.view(torch.int16).numpy().view(U16))
    assert np.array_equal(gotb.view(U16), wantb.view(torch.int16).numpy().view(U16))
    # per tensor: the scalars are rounded once to the output's type
    sv, ov = 0.37123, -3.2517
    want = sat((x + np.float32(np.float16(ov))) * np.float32(np.float16(sv)))
    got = orc.antiquant_policy(desc(abi.PER_TENSOR, abi.F16, scale=sv, offset=ov), codes, None, None)
    assert np.array_equal(got.view(U16), want.view(U16))
    svb = torch.tensor(sv).bfloat16().float().item()
    ovb = torch.tensor(ov).bfloat16().float().item()
    wantb = ((torch.from_numpy(x) + np.float32(ovb)) * np.float32(svb)).bfloat16()
    gotb = orc.antiquant_policy(desc(abi.PER_TENSOR, abi.BF16, scale=sv, offset=ov), codes, None, None)
    assert np.array_equal(gotb.view(U16), wantb.view(torch.int16).numpy().view(U16))


@pytest.mark.parametrize("fmt", [abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2])
@pytest.mark.parametrize("k_dim", [0, 1])
def test_antiquant_fp4_sources_are_value_times_power_of_two(fmt, k_dim):
    """fp4 sources with fp8_e8m0 scales (ascend_antiquant_3510_impl.h:1727-1779): every product of a 4-bit float and
    2^(code - 127) is exact, so the expected bfloat16 output is the closed form ldexp(value, code - 127) (numpy float64,
    then torch's bfloat16 conversion, which has nothing to round), and the half output its clipped half-even cast.
    The special scale codes follow the reference's constants (:69-74): 0 is 2^-127, 255 is NaN."""
    rng = np.random.default_rng(fmt * 2 + k_dim)
    m, n, gs = 64, 96, 32
    codes = rng.integers(0, 16, (m, n)).astype(np.uint8)
    codes.reshape(-1)[:16] = np.arange(16)
    packed = (codes[:, 0::2] | (codes[:, 1::2] << 4)).astype(np.uint8)
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6] if fmt == abi.QDST_FP4_E2M1 else [0, .25, .5, .75, 1, 1.25, 1.5, 1.75])
    vals = np.where(codes & 8, -1.0, 1.0) * grid[codes & 7]
    sshape = (m, n // gs) if k_dim == 1 else (m // gs, n)
    sc = rng.integers(100, 150, sshape).astype(np.uint8)             # 2^-27 .. 2^22: inside half's range and beyond it
    sc.reshape(-1)[:4] = [0, 1, 254, 127]                            # the ends of the exponent range, and 1.0
    full = np.repeat(sc, gs, axis=1) if k_dim == 1 else np.repeat(sc, gs, axis=0)
    exact = np.ldexp(vals, full.astype(np.int64) - 127)              # float64: exact, 6 * 2^127 overflows bfloat16 only
    with np.errstate(over="ignore"):
        want_bf16 = torch.from_numpy(exact.astype(np.float32)).bfloat16().view(torch.int16).numpy().view(U16)
    d = abi.AntiQuantPolicyDesc(policy=abi.PER_GROUP, src_format=fmt, scale_dtype=abi.E8M0, dst_dtype=abi.BF16,
                                compute=abi.COMPUTE_SCALE_T, has_offset=0, is_transpose=0, k_dim=k_dim, m=m, n=n,
                                cal_count=m * n, group_size=gs)
    got = orc.antiquant_policy(d, packed, sc, None)
    assert np.array_equal(got.view(U16), want_bf16)
    d.dst_dtype = abi.F16
    got16 = orc.antiquant_policy(d, packed, sc, None)
    with np.errstate(over="ignore"):
        want16 = np.clip(exact, -65504.0, 65504.0).astype(np.float16)
    assert np.array_equal(got16.view(U16), want16.view(U16))
    # a NaN scale: NaN in bfloat16, +0 through the saturating cast to half
    sc2 = np.full(sshape, 255, dtype=np.uint8)
    d.dst_dtype = abi.BF16
    nb = orc.antiquant_policy(d, packed, sc2, None).view(U16)
    assert np.all((nb & 0x7F80) == 0x7F80) and np.all(nb & 0x7F)
    d.dst_dtype = abi.F16
    assert not orc.antiquant_policy(d, packed, sc2, None).view(U16).any()


def test_swiglu_epilogue_is_the_reference_vector_chain():
    """SwiGLU in the matmul epilogue: columns 2j / 2j + 1 are src0 / src1 and out[j] = src0 * (src1 / (1 + exp(-beta src1)))
    in fp32, one rounding per step (swiglu_common_impl.h:154-190), pinned by numpy float32 arithmetic written as the
    reference's five vector instructions, by the example's golden formula (swiglu/scripts/gen_data.py:32: src0 * src1 /
    (1 + exp(-src1)) in float32) and by torch's bfloat16 rounding of the result."""
    import torch
    rng = np.random.default_rng(11)
    m, k, n = 9, 64, 48
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-127, 128, (k, n)).astype(np.int8)
    cs = rng.uniform(1e-4, 4e-4, n).astype(np.float32)
    ts = rng.uniform(0.5, 2.0, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    acc = a.astype(np.int64) @ b.astype(np.int64)
    v = ((acc.astype(np.float32) * cs[None, :]) * ts[:, None] + bias[None, :]).astype(np.float32)
    for beta in (1.0, 1.702):
        d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.F32, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                           has_tok_scale=1, bias_kind=abi.MM_BIAS_F32_POST, activation=abi.MM_ACT_SWIGLU, act_beta=beta)
        got = orc.matmul_w8a8(d, a, b, bias, cs, ts)
        assert got.shape == (m, n // 2)
        s0, s1 = v[:, 0::2], v[:, 1::2]
        t = (s1 * np.float32(-beta)).astype(np.float32)                       # Muls
        with np.errstate(over="ignore"):                                    # exp of a large argument is inf: swish -> 0
            e = np.exp(t.astype(np.float32)).astype(np.float32)              # Exp
        dd = (e + np.float32(1.0)).astype(np.float32)                        # Adds
        sw = (s1 / dd).astype(np.float32)                                    # Div
        want = (s0 * sw).astype(np.float32)                                  # Mul
        # expf of libm against numpy's float32 exp: at most 1 ulp apart, which the later steps carry through
        assert np.all(np.abs(got - want) <= 4 * np.spacing(np.abs(want)) + 1e-30)
        if beta == 1.0:
            with np.errstate(over="ignore"):
                gold = (s0 * s1 / (1 + np.exp(-1 * s1))).astype(np.float32)  # the example's golden
            assert np.allclose(got, gold, rtol=1e-5, atol=1e-7)
        # bf16 output = torch's rounding of the fp32 result
        d.out_dtype = abi.BF16
        got16 = orc.matmul_w8a8(d, a, b, bias, cs, ts)
        ref16 = torch.from_numpy(got).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got16, ref16)
    # the scalar function itself on special arguments: swish(0) = 0, large |x| saturates to x or to -0
    assert orc.lib().orc_swiglu(3.0, 0.0, 1.0) == 0.0
    assert orc.lib().orc_swiglu(2.0, 100.0, 1.0) == 200.0
    assert abs(orc.lib().orc_swiglu(2.0, -100.0, 1.0)) < 1e-40


def test_hifloat8_codec_is_the_reference_script():
    """hifloat8 has no document table in the reference; its codec ships as a Python script beside the fp8 matmul example
    (matmul_fp8/scripts/hif8.py).  tests/golden/hif8_vectors.npz holds that script's answers (made by
    tests/golden/make_hif8_vectors.py): the decoding of all 256 codes, the float32 encoder with "round" on 13,625 inputs
    (every code value, every midpoint between neighbours and the float32 values beside them, the range ends, random
    values) and the float16 encoder on all 65,536 halves.  The oracle's encoder is a nearest-value search, not the
    script's bit arithmetic.  Outside the pin, because the script is wrong there: the 1,024 halves on which it raises
    (a mantissa that rounds up into a smaller negative exponent: hif8.py:262-265 shifts by a negative count; the float32
    path, which has no such shift, gives what the oracle gives), and negative float16 overflow (hif8.py:228-233 tests for
    overflow before it has looked at the sign and answers with the positive code)."""
    import os
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hif8_vectors.npz"))
    L = orc.lib()
    dec = np.array([L.orc_hif8_to_f32(c) for c in range(256)], dtype=np.float32)
    assert np.array_equal(np.isnan(dec), np.isnan(g["decode"])) and np.isnan(dec).sum() == 1 and np.isnan(dec[0x80])
    ok = ~np.isnan(dec)
    assert np.array_equal(dec[ok].view(np.uint32), g["decode"][ok].view(np.uint32))
    enc = np.array([L.orc_f32_to_hif8(float(x)) for x in g["f32_in"]], dtype=np.uint8)
    assert np.array_equal(enc, g["f32_round"])
    # the non-saturating form of the script differs only where this one saturates: infinities and NaN
    differs = enc != g["f32_round_inf"]
    assert set(g["f32_round_inf"][differs].tolist()) <= {0x6F, 0xEF, 0x80}
    halves = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    ench = np.array([L.orc_f32_to_hif8(float(x)) for x in halves], dtype=np.uint8)
    pinned = ~g["f16_round_raised"] & ~(halves <= -40960.0)
    assert pinned.sum() == 65536 - 1024 - int((halves <= -40960.0).sum())
    assert np.array_equal(ench[pinned], g["f16_round"][pinned])
    assert set(ench[halves <= -40960.0].tolist()) == {0xEE}             # the float32 path's answer for the same values
    # what the mathematics fixes: encode(decode(c)) == c for every finite code; monotone in the value
    finite = [c for c in range(256) if c not in (0x80, 0x6F, 0xEF)]
    assert all(L.orc_f32_to_hif8(float(dec[c])) == c for c in finite)
    xs = np.sort(np.abs(g["f32_in"][np.isfinite(g["f32_in"])]))
    vals = np.array([L.orc_hif8_to_f32(L.orc_f32_to_hif8(float(x))) for x in xs])
    assert np.all(np.diff(vals) >= 0)


# ------------------------------------------------------------------------------------------------- MX matmul
MX_FP4 = {abi.QDST_FP4_E2M1: [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0],
          abi.QDST_FP4_E1M2: [0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75]}
MX_FP8 = {abi.QDST_FP8_E4M3FN: torch.float8_e4m3fn, abi.QDST_FP8_E5M2: torch.float8_e5m2}


def mx_random_operand(rng, rows, k, fmt):
    """Raw bytes of a [rows, k] operand with finite values: fp8 one per byte, fp4 two per byte (even k low)."""
    if fmt in MX_FP8:
        code = rng.integers(0, 256, (rows, k)).astype(np.uint8)
        bad = (code & 0x7F) == 0x7F if fmt == abi.QDST_FP8_E4M3FN else (code & 0x7C) == 0x7C
        code[bad] &= 0x80    # NaN / infinity codes become +-0
        return code
    return rng.integers(0, 256, (rows, k // 2)).astype(np.uint8)


def mx_values(raw, k, fmt):
    """The operand's values as float64 [rows, k], decoded by torch's 8-bit float types or the 4-bit formats' value
    tables (an implementation that shares nothing with the oracle's)."""
    if fmt in MX_FP8:
        return torch.from_numpy(raw.copy()).view(MX_FP8[fmt]).to(torch.float64).numpy()
    nib = np.stack([raw & 15, raw >> 4], axis=-1).reshape(raw.shape[0], k)
    mag = np.array(MX_FP4[fmt])[nib & 7]
    return np.where(nib & 8, -mag, mag)


def mx_golden(a, b, sa, sb, k, fa, fb, bias=None):
    """The data scripts' computation: decompress (value * 2^(scale - 127), block of 32 along k), float64 matmul, float32
    (mmad_mx/scripts/gen_data.py:52-83, 117-126)."""
    blk = np.arange(k) // 32
    af = mx_values(a, k, fa) * np.power(2.0, sa.astype(np.float64) - 127.0)[:, blk]
    bf = mx_values(b, k, fb) * np.power(2.0, sb.astype(np.float64) - 127.0)[:, blk]
    out = np.matmul(af, bf.T).astype(np.float32)
    return out if bias is None else out + bias


@pytest.mark.parametrize("fa,fb", [(abi.QDST_FP4_E1M2, abi.QDST_FP4_E2M1), (abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2),
                                   (abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2), (abi.QDST_FP8_E5M2, abi.QDST_FP8_E4M3FN),
                                   (abi.QDST_FP8_E4M3FN, abi.QDST_FP4_E2M1)])
@pytest.mark.parametrize("bias", [False, True])
def test_matmul_mx_is_the_data_scripts_decompress_then_float64_matmul(fa, fb, bias):
    """The reference example's own shape ([40, 70] x [50, 70], scale_k = ceil(70 / 32) rounded up to even = 4) and its
    four format pairs plus a mixed one, against numpy float64 on operands decoded by torch / value tables."""
    rng = np.random.default_rng(70 + fa * 8 + fb)
    m, n, k, sk = 40, 50, 70, 4
    a, b = mx_random_operand(rng, m, k, fa), mx_random_operand(rng, n, k, fb)
    sa, sb = rng.integers(120, 135, (m, sk)).astype(np.uint8), rng.integers(120, 135, (n, sk)).astype(np.uint8)
    bv = rng.integers(-10, 10, n).astype(np.float32) if bias else None
    d = abi.MxDesc(m=m, n=n, k=k, scale_k=sk, a_format=fa, b_format=fb, out_dtype=abi.F32, has_bias=int(bias))
    got = orc.matmul_mx(d, a, b, sa, sb, bv)
    assert np.array_equal(got, mx_golden(a, b, sa, sb, k, fa, fb, bv))
    d.out_dtype = abi.BF16
    want16 = torch.from_numpy(mx_golden(a, b, sa, sb, k, fa, fb, bv)).to(torch.bfloat16).view(torch.int16).numpy()
    assert np.array_equal(orc.matmul_mx(d, a, b, sa, sb, bv).view(np.int16), want16)


def test_matmul_mx_closed_forms():
    """All-ones operands count k; one more in a scale byte doubles exactly that row's block; the sub-range arguments
    leave the rest of the result alone."""
    m, n, k, sk = 3, 5, 96, 4
    one8, one4 = 0x38, 0x22   # 1.0 in e4m3fn, (1.0, 1.0) in e2m1
    a = np.full((m, k), one8, np.uint8)
    b = np.full((n, k // 2), one4, np.uint8)
    sa, sb = np.full((m, sk), 127, np.uint8), np.full((n, sk), 127, np.uint8)
    d = abi.MxDesc(m=m, n=n, k=k, scale_k=sk, a_format=abi.QDST_FP8_E4M3FN, b_format=abi.QDST_FP4_E2M1,
                   out_dtype=abi.F32, has_bias=0)
    assert np.all(orc.matmul_mx(d, a, b, sa, sb) == k)
    sa[1, 2] = 128
    want = np.full((m, n), float(k), np.float32)
    want[1, :] += 32
    assert np.array_equal(orc.matmul_mx(d, a, b, sa, sb), want)
    sb[4, 0] = 125
    want[:, 4] -= 32 * 0.75
    assert np.array_equal(orc.matmul_mx(d, a, b, sa, sb), want)
    part = orc.matmul_mx(d, a, b, sa, sb, rows=(1, 2), cols=(3, 5))
    assert np.array_equal(part[1, 3:5], want[1, 3:5]) and np.count_nonzero(part) == 2
