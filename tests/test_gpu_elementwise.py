"""GPU parity of AscendQuant / AscendDequant / AscendAntiQuant / dynamic per-token quant against the CPU oracle,
through the C ABI.  int8 outputs must be bit-exact; 16-bit float outputs are compared bit for bit as well (every
operation of these operators rounds once, so there is no tolerance to grant)."""
import numpy as np
import pytest
import torch

import orc
from ascq import _abi as abi
from ascq import ops
from gpu_util import DEV, announce, bits, pack_int4, src_array, src_array_uniform, to_dev

pytestmark = pytest.mark.gpu
TDT = {abi.F16: torch.float16, abi.BF16: torch.bfloat16, abi.F32: torch.float32}


# ------------------------------------------------------------------ AscendQuant, fp16 contract
@pytest.mark.parametrize("src_dt", [abi.F16, abi.F32, abi.BF16])
@pytest.mark.parametrize("count", [256, 1022, 8192 * 3, 2048 * 37 + 8])
def test_quant_per_tensor(src_dt, count):
    announce("quant per-tensor", src_dt, count)
    rng = np.random.default_rng(100 + count)
    x, xd = src_array(rng, count, src_dt, 40.0)
    dst = torch.zeros(count, dtype=torch.int8, device=DEV)
    ops.ascend_quant(dst, xd, 2.0, 0.9)
    d = abi.QuantDesc(policy=abi.PER_TENSOR, src_dtype=src_dt, scale_dtype=src_dt, compute=abi.COMPUTE_F16,
                      round_mode=abi.CAST_RINT, offset_kind=abi.OFFSET_SCALAR, scale=2.0, offset=0.9, cal_count=count)
    want = orc.quant(d, x)
    assert np.array_equal(dst.cpu().numpy(), want)


@pytest.mark.parametrize("src_dt", [abi.F16, abi.F32])
@pytest.mark.parametrize("rows,n", [(37, 64), (8, 4096), (5, 36), (129, 2080)])
@pytest.mark.parametrize("tensor_offset", [False, True])
def test_quant_per_channel(src_dt, rows, n, tensor_offset):
    announce("quant per-channel", src_dt, rows, n, tensor_offset)
    rng = np.random.default_rng(7 * rows + n)
    x, xd = src_array(rng, (rows, n), src_dt, 2.0)
    amax = np.abs(x.astype(np.float32)).max(axis=0) + 1e-3
    s, sd = (127.0 / amax).astype(np.float32), None
    s = s.astype(np.float16) if src_dt == abi.F16 else s
    sd = to_dev(s)
    dst = torch.zeros((rows, n), dtype=torch.int8, device=DEV)
    d = abi.QuantDesc(policy=abi.PER_CHANNEL, src_dtype=src_dt, scale_dtype=src_dt, compute=abi.COMPUTE_F16,
                      round_mode=abi.CAST_RINT, n=n, cal_count=rows * n)
    if tensor_offset:
        o, od = src_array_uniform(rng, n, src_dt, -3, 3)
        ops.ascend_quant(dst, xd, sd, od)
        d.offset_kind = abi.OFFSET_TENSOR
        want = orc.quant(d, x, s, o)
    else:
        ops.ascend_quant(dst, xd, sd, 0.0)
        d.offset_kind, d.offset = abi.OFFSET_SCALAR, 0.0
        want = orc.quant(d, x, s)
    got = dst.cpu().numpy()
    assert np.array_equal(got, want)
    assert np.abs(got.astype(np.int32)).max() >= 126     # the column maxima reach the int8 range


# ------------------------------------------------------------------ PER_TOKEN / PER_GROUP / Quantize
SHAPES = [(10, 288, 1152), (7, 288, 864), (6, 288, 1440), (8, 512, 3584), (4, 256, 768)]   # {m, n, calCount}
PAIRS = [(abi.F16, abi.F16), (abi.BF16, abi.BF16), (abi.F32, abi.F32), (abi.F16, abi.F32), (abi.BF16, abi.F32)]


@pytest.mark.parametrize("compute", [abi.COMPUTE_SCALE_T, abi.COMPUTE_F32])
@pytest.mark.parametrize("pair", PAIRS)
@pytest.mark.parametrize("offset", ["tensor", "scalar", "none"])
def test_quant_per_token_matrix(compute, pair, offset):
    src_dt, sc_dt = pair
    for (m, n, cal) in SHAPES:
        for rmode in (abi.CAST_RINT, abi.CAST_FLOOR, abi.CAST_CEIL, abi.CAST_ROUND, abi.CAST_TRUNC):
            announce("quant per-token", compute, pair, offset, m, n, cal, rmode)
            rng = np.random.default_rng(m * 1000 + n + rmode)
            x, xd = src_array(rng, (m, n), src_dt, 1.0)
            s, sd = src_array_uniform(rng, m, sc_dt, 5, 60)
            o, od = src_array_uniform(rng, m, sc_dt, -2, 2)
            dst = torch.full((m, n), 99, dtype=torch.int8, device=DEV)
            cfg = ops.AscendQuantConfig(has_offset=offset != "none", k_dim=1, round_mode=rmode)
            para = ops.AscendQuantParam(m=m, n=n, cal_count=cal)
            fn = ops.ascend_quant_policy if compute == abi.COMPUTE_SCALE_T else ops.quantize
            d = abi.QuantDesc(policy=abi.PER_TOKEN, src_dtype=src_dt, scale_dtype=sc_dt, compute=compute,
                              round_mode=rmode, k_dim=1, m=m, n=n, cal_count=cal)
            if offset == "tensor":
                fn(dst, xd, sd, od, para, abi.PER_TOKEN, cfg)
                d.offset_kind = abi.OFFSET_TENSOR
            elif offset == "scalar":
                fn(dst, xd, sd, 0.75, para, abi.PER_TOKEN, cfg)
                d.offset_kind, d.offset = abi.OFFSET_SCALAR, 0.75
            else:
                fn(dst, xd, sd, None, para, abi.PER_TOKEN, cfg)
            want = orc.quant(d, x.reshape(-1)[:cal].copy(), s, o)
            got = dst.cpu().numpy().reshape(-1)
            assert np.array_equal(got[:cal], want)
            assert np.all(got[cal:] == 99)               # only the first calCount elements are written


@pytest.mark.parametrize("k_dim", [0, 1])
@pytest.mark.parametrize("gs", [32, 64, 128, 256])
@pytest.mark.parametrize("pair", PAIRS)
def test_quant_per_group(k_dim, gs, pair):
    announce("quant per-group", k_dim, gs, pair)
    src_dt, sc_dt = pair
    m, n = (10, 256) if k_dim == 1 else (256, 64)
    rng = np.random.default_rng(gs + k_dim)
    x, xd = src_array(rng, (m, n), src_dt, 1.0)
    sshape = (m, -(-n // gs)) if k_dim == 1 else (-(-m // gs), n)
    s, sd = src_array_uniform(rng, sshape, sc_dt, 5, 60)
    o, od = src_array_uniform(rng, sshape, sc_dt, -2, 2)
    for compute, fn in ((abi.COMPUTE_SCALE_T, ops.ascend_quant_policy), (abi.COMPUTE_F32, ops.quantize)):
        dst = torch.zeros((m, n), dtype=torch.int8, device=DEV)
        fn(dst, xd, sd, od, ops.AscendQuantParam(m, n, m * n, gs), abi.PER_GROUP,
           ops.AscendQuantConfig(has_offset=True, k_dim=k_dim))
        d = abi.QuantDesc(policy=abi.PER_GROUP, src_dtype=src_dt, scale_dtype=sc_dt, compute=compute,
                          round_mode=abi.CAST_RINT, offset_kind=abi.OFFSET_TENSOR, k_dim=k_dim, m=m, n=n,
                          cal_count=m * n, group_size=gs)
        assert np.array_equal(dst.cpu().numpy(), orc.quant(d, x, s, o))


@pytest.mark.parametrize("src_dt", [abi.BF16, abi.F16, abi.F32])
@pytest.mark.parametrize("m,n", [(1, 4096), (16, 4096), (5, 1000), (3, 8192), (2, 12288), (4, 20000), (7, 37)])
def test_dynamic_quant_per_token(src_dt, m, n):
    announce("dynamic quant", src_dt, m, n)
    rng = np.random.default_rng(m + n)
    x, xd = src_array(rng, (m, n), src_dt, 1.0)
    if m > 2:
        x[1] = 0
        xd[1] = 0
    q, ts = ops.dynamic_quant_per_token(xd)
    wq, wts = orc.dynamic_quant_per_token(src_dt, x)
    assert np.array_equal(ts.cpu().numpy(), wts)
    assert np.array_equal(q.cpu().numpy(), wq)


# ------------------------------------------------------------------ 8-bit float destinations
FP8 = {abi.QDST_FP8_E4M3FN: torch.float8_e4m3fn, abi.QDST_FP8_E5M2: torch.float8_e5m2}


def typed(x, dtype):
    """fp32 values -> (host array in `dtype`'s representation, device tensor)."""
    x = np.asarray(x, dtype=np.float32)
    if dtype == abi.F32:
        return x, to_dev(x)
    if dtype == abi.F16:
        return x.astype(np.float16), to_dev(x.astype(np.float16))
    b = orc.f32_to_bf16_bits(x)
    return b, to_dev(b, "bf16")


@pytest.mark.parametrize("fmt", [abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2])
@pytest.mark.parametrize("pair", PAIRS)
@pytest.mark.parametrize("policy", ["token", "group0", "group1", "channel", "tensor"])
def test_quant_fp8(fmt, pair, policy):
    """fp8_e4m3fn / fp8_e5m2 outputs (fp32 arithmetic, half-even, saturating): bit-exact against the oracle.  The
    scales push part of the data past the largest finite value and part of it into the subnormal range."""
    src_dt, sc_dt = pair
    for (m, n, cal) in [(10, 288, 1152), (8, 512, 3584), (6, 36 * 8, 6 * 36 * 8)]:
        announce("quant fp8", fmt, pair, policy, m, n, cal)
        rng = np.random.default_rng(m + n + fmt)
        x, xd = src_array(rng, (m, n), src_dt, 1.0)
        top = 300.0 if fmt == abi.QDST_FP8_E4M3FN else 40000.0
        gs = 32
        pol = {"token": abi.PER_TOKEN, "group0": abi.PER_GROUP, "group1": abi.PER_GROUP, "channel": abi.PER_CHANNEL,
               "tensor": abi.PER_TENSOR}[policy]
        k_dim = 0 if policy == "group0" else 1
        sshape = {"token": (m,), "group0": (-(-m // gs), n), "group1": (m, -(-n // gs)), "channel": (n,),
                  "tensor": (1,)}[policy]
        # log-uniform scales: products from 1e-3 (subnormal for e4m3fn) to beyond the largest finite value
        s = np.exp(rng.uniform(np.log(1e-3), np.log(top), sshape)).astype(np.float32)
        s.flat[0], s.flat[-1] = min(top * 8, 6e4), 1e-3  # both ends are present whatever the draw (finite in half)
        o = rng.uniform(-0.5, 0.5, sshape).astype(np.float32)
        (s, sdev), (o, odev) = typed(s, sc_dt), typed(o, sc_dt)
        dst = torch.zeros((m, n), dtype=FP8[fmt], device=DEV)
        cfg = ops.AscendQuantConfig(has_offset=True, k_dim=k_dim, round_mode=abi.CAST_RINT)
        para = ops.AscendQuantParam(m=m, n=n, cal_count=cal, group_size=gs if pol == abi.PER_GROUP else 0)
        d = abi.QuantDesc(policy=pol, src_dtype=src_dt, scale_dtype=sc_dt, compute=abi.COMPUTE_F32,
                          round_mode=abi.CAST_RINT, k_dim=k_dim, m=m, n=n, cal_count=cal,
                          group_size=para.group_size, dst_format=fmt, offset_kind=abi.OFFSET_TENSOR)
        if pol == abi.PER_TENSOR:
            sv, ov = float(np.float32(3.7)), 0.25
            ops.quantize(dst, xd, sv, ov, para, pol, cfg)
            d.scale, d.offset, d.offset_kind, d.scale_dtype = sv, ov, abi.OFFSET_SCALAR, src_dt
            want = orc.quant(d, x.reshape(-1)[:cal].copy())
        else:
            fn = ops.ascend_quant_policy if pol in (abi.PER_TOKEN, abi.PER_GROUP) else ops.quantize
            if fn is ops.ascend_quant_policy:
                d.compute = abi.COMPUTE_SCALE_T        # the library widens to fp32 by itself for these outputs
            fn(dst, xd, sdev, odev, para, pol, cfg)
            want = orc.quant(d, x.reshape(-1)[:cal].copy(), s, o)
        got = dst.view(torch.uint8).cpu().numpy().reshape(-1)
        assert np.array_equal(got[:cal], want.view(np.uint8))
        assert np.all(got[cal:] == 0)
        if pol != abi.PER_TENSOR and cal == m * n:
            top_code = 0x7E if fmt == abi.QDST_FP8_E4M3FN else 0x7B
            assert np.any((got[:cal] & 0x7F) == top_code)          # saturation was exercised


@pytest.mark.parametrize("pair", PAIRS)
@pytest.mark.parametrize("policy", ["token", "group0", "group1", "channel", "tensor"])
def test_quant_hifloat8(pair, policy):
    """hifloat8 outputs: arithmetic in the scale's type (PER_TOKEN / PER_GROUP) or in fp32 (Quantize), then the cast
    that rounds ties away from zero and saturates: bit-exact against the oracle.  The scales spread the products from
    below the smallest code (2^-22) to beyond the largest (2^15)."""
    src_dt, sc_dt = pair
    for (m, n, cal) in [(10, 288, 1152), (8, 512, 3584), (6, 36 * 8, 6 * 36 * 8)]:
        announce("quant hifloat8", pair, policy, m, n, cal)
        rng = np.random.default_rng(m + n + 5)
        x, xd = src_array(rng, (m, n), src_dt, 1.0)
        gs = 32
        pol = {"token": abi.PER_TOKEN, "group0": abi.PER_GROUP, "group1": abi.PER_GROUP, "channel": abi.PER_CHANNEL,
               "tensor": abi.PER_TENSOR}[policy]
        k_dim = 0 if policy == "group0" else 1
        sshape = {"token": (m,), "group0": (-(-m // gs), n), "group1": (m, -(-n // gs)), "channel": (n,),
                  "tensor": (1,)}[policy]
        s = np.exp(rng.uniform(np.log(1e-7), np.log(3e4), sshape)).astype(np.float32)
        s.flat[0], s.flat[-1] = 6e4, 1e-7
        o = rng.uniform(-1e-6, 1e-6, sshape).astype(np.float32)
        (s, sdev), (o, odev) = typed(s, sc_dt), typed(o, sc_dt)
        dst = torch.zeros((m, n), dtype=torch.uint8, device=DEV)
        cfg = ops.AscendQuantConfig(has_offset=True, k_dim=k_dim, round_mode=abi.CAST_ROUND)
        para = ops.AscendQuantParam(m=m, n=n, cal_count=cal, group_size=gs if pol == abi.PER_GROUP else 0)
        d = abi.QuantDesc(policy=pol, src_dtype=src_dt, scale_dtype=sc_dt, compute=abi.COMPUTE_F32,
                          round_mode=abi.CAST_ROUND, k_dim=k_dim, m=m, n=n, cal_count=cal,
                          group_size=para.group_size, dst_format=abi.QDST_HIF8, offset_kind=abi.OFFSET_TENSOR)
        if pol == abi.PER_TENSOR:
            sv, ov = float(np.float32(3.7)), 0.25
            ops.quantize(dst, xd, sv, ov, para, pol, cfg, dst_format=abi.QDST_HIF8)
            d.scale, d.offset, d.offset_kind, d.scale_dtype = sv, ov, abi.OFFSET_SCALAR, src_dt
            want = orc.quant(d, x.reshape(-1)[:cal].copy())
        elif pol in (abi.PER_TOKEN, abi.PER_GROUP):
            d.compute = abi.COMPUTE_SCALE_T
            ops.ascend_quant_policy(dst, xd, sdev, odev, para, pol, cfg, dst_format=abi.QDST_HIF8)
            want = orc.quant(d, x.reshape(-1)[:cal].copy(), s, o)
        else:
            ops.quantize(dst, xd, sdev, odev, para, pol, cfg, dst_format=abi.QDST_HIF8)
            want = orc.quant(d, x.reshape(-1)[:cal].copy(), s, o)
        got = dst.cpu().numpy().reshape(-1)
        assert np.array_equal(got[:cal], want.view(np.uint8))
        assert np.all(got[cal:] == 0)
        if pol != abi.PER_TENSOR and cal == m * n:
            # both ends were exercised: the largest code, and zero or the mantissa-less powers of two 2^-22 .. 2^-16
            assert np.any((got[:cal] & 0x7F) == 0x6E) and np.any((got[:cal] & 0x7F) < 8)


def test_hifloat8_cast_against_the_reference_script_vectors():
    """The device's cast itself, not through the oracle: Quantize per tensor with scale 1 on the float32 inputs of the
    committed vectors (the reference script's answers), and AscendQuant's half chain (scale 1, offset 0) on every
    float16 value the script answers correctly; then AntiQuantize of all codes against the script's decoding."""
    import os
    announce("hifloat8 vectors")
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hif8_vectors.npz"))
    x = g["f32_in"][:-(g["f32_in"].size % 32) or None].copy()
    n = 32
    m = x.size // n
    dst = torch.zeros((m, n), dtype=torch.uint8, device=DEV)
    cfg = ops.AscendQuantConfig(has_offset=False, k_dim=1, round_mode=abi.CAST_ROUND)
    ops.quantize(dst, to_dev(x.reshape(m, n)), 1.0, 0.0, ops.AscendQuantParam(m=m, n=n, cal_count=m * n, group_size=0),
                 abi.PER_TENSOR, cfg, dst_format=abi.QDST_HIF8)
    assert np.array_equal(dst.cpu().numpy().reshape(-1), g["f32_round"][:x.size])
    halves = np.arange(65536, dtype=np.uint16).view(np.float16)
    h32 = halves.astype(np.float32)
    pinned = ~g["f16_round_raised"] & ~(h32 <= -40960.0) & ~np.isnan(h32)
    dsth = torch.zeros(65536, dtype=torch.uint8, device=DEV)
    ops.ascend_quant(dsth, to_dev(halves), 1.0, 0.0, dst_format=abi.QDST_HIF8)
    assert np.array_equal(dsth.cpu().numpy()[pinned], g["f16_round"][pinned])
    codes = np.arange(256, dtype=np.uint8).repeat(32).reshape(256, 32)
    out = torch.zeros((256, 32), dtype=torch.float32, device=DEV)
    ones = torch.ones(256, dtype=torch.float32, device=DEV)
    ops.ascend_antiquant_policy(out, to_dev(codes), ones, None, ops.AscendAntiQuantParam(m=256, n=32, cal_count=256 * 32),
                                abi.PER_TOKEN, ops.AscendAntiQuantConfig(has_offset=False), src_format=abi.QDST_HIF8)
    got = out.cpu().numpy()[:, 0]
    want = g["decode"]
    fin = ~np.isnan(want)
    assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32)) and np.isnan(got[0x80])


@pytest.mark.parametrize("fmt", [abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2])
@pytest.mark.parametrize("pair", [(abi.F16, abi.F16), (abi.F16, abi.F32), (abi.BF16, abi.BF16), (abi.BF16, abi.F32)])
@pytest.mark.parametrize("mode", [abi.CAST_RINT, abi.CAST_ROUND, abi.CAST_FLOOR, abi.CAST_CEIL, abi.CAST_TRUNC])
@pytest.mark.parametrize("k_dim", [0, 1])
def test_quant_fp4(fmt, pair, mode, k_dim):
    """fp4x2_e2m1_t / fp4x2_e1m2_t outputs of AscendQuant PER_GROUP, every type pair of the reference's table and
    every rounding mode: the packed bytes are bit-equal to the oracle's.  The scales put part of the data past the
    largest magnitude and the data holds exact midpoints of the grid; the offset tensor is passed and must be ignored,
    as in the reference."""
    src_dt, sc_dt = pair
    top = 6.0 if fmt == abi.QDST_FP4_E2M1 else 1.75
    for (m, n, cal) in [(10, 288, 1152), (64, 512, 64 * 512), (6, 64, 6 * 64)]:
        announce("quant fp4", fmt, pair, mode, k_dim, m, n, cal)
        rng = np.random.default_rng(m + n + fmt + mode)
        x, xd = src_array(rng, (m, n), src_dt, 1.0)
        gs = 32
        sshape = (m, -(-n // gs)) if k_dim == 1 else (-(-m // gs), n)
        s = np.exp(rng.uniform(np.log(0.05), np.log(4 * top), sshape)).astype(np.float32)
        if k_dim == 1:
            s[0, 0] = 1.0                                        # this group keeps the midpoints planted below
        else:
            s[0, :10] = 1.0
        (s, sdev) = typed(s, sc_dt)
        mids = np.float32([0.25, 0.75, 1.25, 2.5, 5.0, -0.125, -0.375, -3.5, 7.0, -9.0])
        if src_dt == abi.F16:
            x[0, :10] = mids.astype(np.float16)
            xd = to_dev(x)
        else:
            x[0, :10] = orc.f32_to_bf16_bits(mids)
            xd = to_dev(x, "bf16")
        o = rng.uniform(-3, 3, sshape).astype(np.float32)
        (o, odev) = typed(o, sc_dt)
        dst = torch.zeros(m * n // 2, dtype=torch.uint8, device=DEV)
        cfg = ops.AscendQuantConfig(has_offset=True, k_dim=k_dim, round_mode=mode)
        para = ops.AscendQuantParam(m=m, n=n, cal_count=cal, group_size=gs)
        ops.ascend_quant_policy(dst, xd, sdev, odev, para, abi.PER_GROUP, cfg, dst_format=fmt)
        d = abi.QuantDesc(policy=abi.PER_GROUP, src_dtype=src_dt, scale_dtype=sc_dt, compute=abi.COMPUTE_SCALE_T,
                          round_mode=mode, k_dim=k_dim, m=m, n=n, cal_count=cal, group_size=gs, dst_format=fmt,
                          offset_kind=abi.OFFSET_TENSOR)
        want = orc.quant(d, x.reshape(-1)[:cal].copy(), s, o).reshape(-1)
        got = dst.cpu().numpy()
        assert np.array_equal(got[:cal // 2], want)
        assert np.all(got[cal // 2:] == 0)
        codes = np.concatenate([got[:cal // 2] & 15, got[:cal // 2] >> 4])
        assert set(np.unique(codes & 7)) == set(range(8)) and np.any(codes & 8)    # every magnitude, both signs


def test_quant_fp4_rejects():
    announce("quant fp4 rejects")
    x = torch.zeros((4, 64), dtype=torch.float16, device=DEV)
    s = torch.ones((4, 2), dtype=torch.float16, device=DEV)
    dst = torch.zeros(128, dtype=torch.uint8, device=DEV)
    para = ops.AscendQuantParam(m=4, n=64, cal_count=256, group_size=32)
    cfg = ops.AscendQuantConfig(has_offset=False, k_dim=1)
    with pytest.raises(ops.AscqError, match="PER_GROUP only"):
        ops.ascend_quant_policy(dst, x, s[:, 0].contiguous(), None, para, abi.PER_TOKEN, cfg,
                                dst_format=abi.QDST_FP4_E2M1)
    xf = torch.zeros((4, 64), dtype=torch.float32, device=DEV)
    sf = torch.ones((4, 2), dtype=torch.float32, device=DEV)
    with pytest.raises(ops.AscqError, match="half / bfloat16 sources"):
        ops.ascend_quant_policy(dst, xf, sf, None, para, abi.PER_GROUP, cfg, dst_format=abi.QDST_FP4_E1M2)


# ------------------------------------------------------------------ AscendDequant
@pytest.mark.parametrize("dst_dt,sc_dt", [(abi.F16, abi.U64), (abi.F32, abi.F32), (abi.F32, abi.BF16),
                                          (abi.BF16, abi.BF16), (abi.BF16, abi.F32)])
@pytest.mark.parametrize("m,n,cal", [(4, 8, 6), (6, 40, 24), (128, 32, 32), (33, 4096, 4096), (3, 136, 130)])
def test_dequant_per_channel(dst_dt, sc_dt, m, n, cal):
    announce("dequant per-channel", dst_dt, sc_dt, m, n, cal)
    rng = np.random.default_rng(m * n + cal)
    src = rng.integers(-2**20, 2**20, (m, n), dtype=np.int32)
    sf = rng.uniform(1e-5, 1e-3, n).astype(np.float32) * rng.choice([-1, 1], n).astype(np.float32)
    if sc_dt == abi.BF16:
        sc = orc.f32_to_bf16_bits(sf)
        scd = to_dev(sc, "bf16")
    elif sc_dt == abi.U64:
        sc = sf.view(np.uint32).astype(np.uint64) | (np.uint64(0xABC) << np.uint64(40))
        scd = to_dev(sc)
    else:
        sc, scd = sf, to_dev(sf)
    stride = ops.dequant_dst_stride(TDT[dst_dt], n)
    fill = 0x7E7E if dst_dt != abi.F32 else 0
    dst = torch.zeros((m, stride), dtype=TDT[dst_dt], device=DEV)
    if dst_dt != abi.F32:
        dst.view(torch.int16).fill_(0x7E7E)
    ops.ascend_dequant(dst, to_dev(src), scd, ops.DequantParams(m, n, cal), mode=abi.DEQUANT_WITH_MULTI_ROW)
    d = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=sc_dt, dst_dtype=dst_dt,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, m=m, n=n, cal_count=cal)
    want = orc.dequant(d, src, sc, fill=fill)
    got = bits(dst)
    assert np.array_equal(got, want.view(np.uint16) if dst_dt != abi.F32 else want)


def test_dequant_scalar_single_row_and_policies():
    announce("dequant scalar / single-row / per-token / per-group")
    rng = np.random.default_rng(5)
    src = rng.integers(-5000, 5000, (1, 64), dtype=np.int32)
    for dst_dt in (abi.F32, abi.BF16):
        dst = torch.zeros((8, ops.dequant_dst_stride(TDT[dst_dt], 8)), dtype=TDT[dst_dt], device=DEV)
        sc = np.arange(1, 9, dtype=np.float32) * 0.37
        ops.ascend_dequant(dst, to_dev(src), to_dev(sc), ops.DequantParams(1, 64, 8))      # SINGLE_ROW default
        d = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=dst_dt,
                            mode=abi.DEQUANT_WITH_SINGLE_ROW, m=1, n=64, cal_count=8)
        want = orc.dequant(d, src, sc)
        if dst_dt == abi.F32:
            assert want.shape == (8, 8) and np.array_equal(bits(dst), want)
        else:                                                     # 8 bf16 is not 32 bytes: stays {1, 64, 8}
            assert want.shape == (1, 64)
            assert np.array_equal(bits(dst).reshape(-1)[:64], want.reshape(-1))
    src = rng.integers(-2**20, 2**20, (12, 256), dtype=np.int32)
    dst = torch.zeros((12, 256), dtype=torch.float32, device=DEV)
    ops.ascend_dequant(dst, to_dev(src), 2.2, ops.DequantParams(12, 256, 200), mode=abi.DEQUANT_WITH_MULTI_ROW)
    d = abi.DequantDesc(policy=abi.PER_TENSOR, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.F32,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, scale=2.2, m=12, n=256, cal_count=200)
    assert np.array_equal(bits(dst), orc.dequant(d, src))
    for policy, k_dim, gs, sshape in ((abi.PER_TOKEN, 1, 0, (12,)), (abi.PER_GROUP, 1, 64, (12, 4)),
                                      (abi.PER_GROUP, 0, 32, (1, 256))):
        for sc_dt in (abi.F32, abi.BF16, abi.F16):
            for src_f32 in (False, True):
                s, sd = src_array_uniform(rng, sshape, sc_dt, 0.01, 1.0)
                sin = src.astype(np.float32) * np.float32(0.37) if src_f32 else src
                dstb = torch.zeros((12, 256), dtype=torch.bfloat16, device=DEV)
                for cal in (12 * 256, 5 * 256):       # every row, and the first five only (the rest stays untouched)
                    dstb.zero_()
                    para = ops.AscendQuantParam(12, 256, cal, gs)
                    ops.ascend_dequant_policy(dstb, to_dev(sin), sd, para, policy, k_dim)
                    d = abi.DequantDesc(policy=policy, src_dtype=abi.F32 if src_f32 else abi.I32, scale_dtype=sc_dt,
                                        dst_dtype=abi.BF16, mode=abi.DEQUANT_WITH_MULTI_ROW, k_dim=k_dim, m=12, n=256,
                                        cal_count=cal, group_size=gs)
                    got = bits(dstb)
                    assert np.array_equal(got[:cal // 256], orc.dequant(d, sin, s))
                    assert not got[cal // 256:].any()


# ------------------------------------------------------------------ AscendAntiQuant
@pytest.mark.parametrize("int4", [False, True])
@pytest.mark.parametrize("dst_dt", [abi.F16, abi.BF16])
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("K,N,G", [(64, 128, 1), (256, 32, 4), (2048, 64, 1), (5888 // 256, 256, 1), (96, 128, 3),
                                   (64, 40, 2)])
@pytest.mark.parametrize("has_offset", [True, False])
def test_antiquant(int4, dst_dt, transpose, K, N, G, has_offset):
    if transpose and K % (64 if int4 else 32):
        pytest.skip("transposed input needs a 32-byte aligned k axis")
    announce("antiquant", int4, dst_dt, transpose, K, N, G, has_offset)
    rng = np.random.default_rng(K + N + G)
    w = rng.integers(-8, 8, (K, N)).astype(np.int8) if int4 else rng.integers(-128, 128, (K, N)).astype(np.int8)
    sc, _ = src_array_uniform(rng, (G, N), dst_dt, -2, 2)
    of, _ = src_array_uniform(rng, (G, N), dst_dt, -9, 9)
    if transpose:
        w, sc, of = (np.ascontiguousarray(t.T) for t in (w, sc, of))
        d = abi.AntiQuantDesc(src_dtype=abi.I4 if int4 else abi.I8, dst_dtype=dst_dt, is_transpose=1,
                              has_offset=int(has_offset), k=K, n=N, scale_height=N, scale_width=G, offset_height=N,
                              offset_width=G)
        info = ops.AntiQuantShapeInfo(N, G, N, G)
    else:
        d = abi.AntiQuantDesc(src_dtype=abi.I4 if int4 else abi.I8, dst_dtype=dst_dt, has_offset=int(has_offset), k=K,
                              n=N, scale_height=G, scale_width=N, offset_height=G, offset_width=N)
        info = ops.AntiQuantShapeInfo(G, N, G, N)
    src = pack_int4(w) if int4 else w
    kind = "bf16" if dst_dt == abi.BF16 else None
    dst = torch.zeros(w.shape, dtype=TDT[dst_dt], device=DEV)
    ops.ascend_antiquant(dst, to_dev(src), to_dev(of, kind) if has_offset else None, to_dev(sc, kind), K, info,
                         is_transpose=transpose, int4=int4)
    want = orc.antiquant(d, src, of if has_offset else None, sc)
    assert np.array_equal(bits(dst), want.view(np.uint16))


# ------------------------------------------------------------------ AscendAntiQuant PER_TOKEN / PER_GROUP
B8 = {abi.QDST_I8: torch.int8, abi.QDST_FP8_E4M3FN: torch.float8_e4m3fn, abi.QDST_FP8_E5M2: torch.float8_e5m2,
      abi.QDST_HIF8: torch.uint8}
AQP_TYPES = [(abi.F16, abi.F16, abi.COMPUTE_SCALE_T), (abi.BF16, abi.BF16, abi.COMPUTE_SCALE_T),
             (abi.F32, abi.F32, abi.COMPUTE_SCALE_T), (abi.F32, abi.F16, abi.COMPUTE_SCALE_T),
             (abi.F32, abi.BF16, abi.COMPUTE_SCALE_T), (abi.F16, abi.F16, abi.COMPUTE_F32),
             (abi.BF16, abi.F32, abi.COMPUTE_F32)]                     # (scale, dst, arithmetic)


@pytest.mark.parametrize("fmt", [abi.QDST_I8, abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2, abi.QDST_HIF8])
@pytest.mark.parametrize("types", AQP_TYPES)
@pytest.mark.parametrize("mode", ["token", "group_n", "group_m", "group_m_via_transpose"])
def test_antiquant_policy(fmt, types, mode):
    """Every source code of the one-byte formats (NaN / infinity codes aside), every legal type combination, both
    group axes: bit-exact against the oracle."""
    sc_dt, dst_dt, compute = types
    for (m, n, cal, has_offset) in [(64, 256, 64 * 256, True), (40, 96, 32 * 96, False), (33, 2080, 33 * 2080, True)]:
        announce("antiquant policy", fmt, types, mode, m, n, cal)
        rng = np.random.default_rng(m + n + fmt)
        codes = rng.integers(0, 256, (m, n)).astype(np.uint8)
        codes.reshape(-1)[:256] = np.arange(256, dtype=np.uint8)          # every code at least once
        if fmt == abi.QDST_FP8_E4M3FN:
            codes[(codes & 0x7F) == 0x7F] = 0x3C
        elif fmt == abi.QDST_FP8_E5M2:
            codes[(codes & 0x7F) >= 0x7C] = 0x3C
        elif fmt == abi.QDST_HIF8:
            codes[(codes == 0x80) | ((codes & 0x7F) == 0x6F)] = 0x3C
        gs = 32
        policy = abi.PER_TOKEN if mode == "token" else abi.PER_GROUP
        k_dim, tr = {"token": (1, 0), "group_n": (1, 0), "group_m": (0, 0), "group_m_via_transpose": (1, 1)}[mode]
        pshape = {"token": (m,), "group_n": (m, -(-n // gs))}.get(mode, (-(-m // gs), n))
        (s, sdev), (o, odev) = typed(rng.uniform(0.01, 2.0, pshape), sc_dt), typed(rng.uniform(-3, 3, pshape), sc_dt)
        dst = torch.zeros((m, n), dtype=TDT[dst_dt], device=DEV)
        cfg = ops.AscendAntiQuantConfig(has_offset=has_offset, is_transpose=bool(tr), k_dim=k_dim)
        para = ops.AscendAntiQuantParam(m=m, n=n, cal_count=cal, group_size=gs if policy == abi.PER_GROUP else 0)
        fn = ops.ascend_antiquant_policy if compute == abi.COMPUTE_SCALE_T else ops.antiquantize
        fn(dst, to_dev(codes).view(B8[fmt]), sdev, odev, para, policy, cfg, src_format=fmt)
        d = abi.AntiQuantPolicyDesc(policy=policy, src_format=fmt, scale_dtype=sc_dt, dst_dtype=dst_dt, compute=compute,
                                    has_offset=int(has_offset), is_transpose=tr, k_dim=k_dim, m=m, n=n, cal_count=cal,
                                    group_size=para.group_size)
        want = orc.antiquant_policy(d, codes, s, o)
        got = bits(dst)
        want = want.view(np.uint16) if want.dtype == np.float16 else want
        rows = cal // n
        if dst_dt == abi.F32:
            assert np.array_equal(got[:rows].view(np.uint32), want[:rows].view(np.uint32))
        else:
            assert np.array_equal(got[:rows], want[:rows])
        assert not got[rows:].any()


@pytest.mark.parametrize("fmt", [abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2])
@pytest.mark.parametrize("dst_dt", [abi.F16, abi.BF16])
def test_antiquant_policy_nan_and_infinity_codes_through_the_saturating_cast(fmt, dst_dt):
    """fp8 sources that are NaN or infinity, fp32 arithmetic, 16-bit destination: the saturating cast gives the
    largest finite value for infinities and +0 for NaN (the saturation-mode column of the reference's boundary table,
    rows float/half and float/bfloat16_t); bit-equal to the oracle, and the expected patterns spelt out."""
    announce("antiquant policy nan/inf", fmt, dst_dt)
    m, n = 8, 64
    codes = np.full((m, n), 0x3C, dtype=np.uint8)
    nan_codes = [0x7F, 0xFF] if fmt == abi.QDST_FP8_E4M3FN else [0x7D, 0x7E, 0x7F, 0xFD]
    inf_codes = [] if fmt == abi.QDST_FP8_E4M3FN else [0x7C, 0xFC]
    special = nan_codes + inf_codes
    codes[0, :len(special)] = special
    s = np.full(m, 2.0, dtype=np.float32)
    dst = torch.zeros((m, n), dtype=TDT[dst_dt], device=DEV)
    cfg = ops.AscendAntiQuantConfig(has_offset=False, is_transpose=False, k_dim=1)
    para = ops.AscendAntiQuantParam(m=m, n=n, cal_count=m * n, group_size=0)
    ops.ascend_antiquant_policy(dst, to_dev(codes).view(B8[fmt]), to_dev(s), None, para, abi.PER_TOKEN, cfg)
    d = abi.AntiQuantPolicyDesc(policy=abi.PER_TOKEN, src_format=fmt, scale_dtype=abi.F32, dst_dtype=dst_dt,
                                compute=abi.COMPUTE_SCALE_T, has_offset=0, is_transpose=0, k_dim=1, m=m, n=n,
                                cal_count=m * n, group_size=0)
    want = orc.antiquant_policy(d, codes, s, None)
    want = want.view(np.uint16) if want.dtype == np.float16 else want
    got = bits(dst)
    assert np.array_equal(got, want)
    top = 0x7BFF if dst_dt == abi.F16 else 0x7F7F
    assert list(got[0, :len(nan_codes)]) == [0] * len(nan_codes)
    assert list(got[0, len(nan_codes):len(special)]) == [top, 0x8000 | top][:len(inf_codes)]


@pytest.mark.parametrize("fmt", [abi.QDST_I8, abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2])
@pytest.mark.parametrize("dst_dt", [abi.F16, abi.BF16])
@pytest.mark.parametrize("policy", [abi.PER_CHANNEL, abi.PER_TENSOR])
@pytest.mark.parametrize("has_offset", [True, False])
def test_antiquantize_per_channel_and_per_tensor(fmt, dst_dt, policy, has_offset):
    """AntiQuantize PER_CHANNEL / PER_TENSOR: fp32 arithmetic on parameters of the output's type, saturating cast;
    every source code, bit-exact against the oracle."""
    for (m, n) in [(64, 256), (33, 2080), (5, 32)]:
        announce("antiquantize", fmt, dst_dt, policy, has_offset, m, n)
        rng = np.random.default_rng(m + n + fmt)
        codes = rng.integers(0, 256, (m, n)).astype(np.uint8)
        codes.reshape(-1)[:min(256, m * n)] = np.arange(min(256, m * n), dtype=np.uint8)
        if fmt == abi.QDST_FP8_E4M3FN:
            codes[(codes & 0x7F) == 0x7F] = 0x3C
        elif fmt == abi.QDST_FP8_E5M2:
            codes[(codes & 0x7F) >= 0x7C] = 0x3C
        dst = torch.zeros((m, n), dtype=TDT[dst_dt], device=DEV)
        cfg = ops.AscendAntiQuantConfig(has_offset=has_offset, is_transpose=False, k_dim=1)
        para = ops.AscendAntiQuantParam(m=m, n=n, cal_count=m * n, group_size=0)
        d = abi.AntiQuantPolicyDesc(policy=policy, src_format=fmt, scale_dtype=dst_dt, dst_dtype=dst_dt,
                                    compute=abi.COMPUTE_F32, has_offset=int(has_offset), is_transpose=0, k_dim=1,
                                    m=m, n=n, cal_count=m * n, group_size=0)
        if policy == abi.PER_CHANNEL:
            (s, sdev), (o, odev) = typed(rng.uniform(0.01, 2.0, n), dst_dt), typed(rng.uniform(-3, 3, n), dst_dt)
            ops.antiquantize(dst, to_dev(codes).view(B8[fmt]), sdev, odev, para, policy, cfg)
            want = orc.antiquant_policy(d, codes, s, o)
        else:
            sv, ov = 0.37123, -3.2517                      # not representable in half / bfloat16: rounded once
            ops.antiquantize(dst, to_dev(codes).view(B8[fmt]), sv, ov, para, policy, cfg)
            d.scale, d.offset = sv, ov
            want = orc.antiquant_policy(d, codes, None, None)
        want = want.view(np.uint16) if want.dtype == np.float16 else want
        assert np.array_equal(bits(dst), want)


@pytest.mark.parametrize("fmt", [abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2])
@pytest.mark.parametrize("dst_dt", [abi.F16, abi.BF16])
@pytest.mark.parametrize("mode", ["group_n", "group_m", "group_m_via_transpose"])
def test_antiquant_fp4_sources(fmt, dst_dt, mode):
    """fp4x2 sources with fp8_e8m0 scales, PER_GROUP along either axis, half and bfloat16 outputs: bit-equal to the
    oracle (NaN outputs compared as NaN).  The scales cover both ends of the exponent range, NaN, and products beyond
    half's range."""
    k_dim, tr = {"group_n": (1, 0), "group_m": (0, 0), "group_m_via_transpose": (1, 1)}[mode]
    along_n = (k_dim == 1) != bool(tr)
    for (m, n, cal) in [(64, 256, 64 * 256), (40, 96, 32 * 96), (33, 2080, 33 * 2080)]:
        announce("antiquant fp4", fmt, dst_dt, mode, m, n, cal)
        rng = np.random.default_rng(m + n + fmt)
        gs = 32
        packed = rng.integers(0, 256, (m, n // 2)).astype(np.uint8)
        packed.reshape(-1)[:256] = np.arange(256, dtype=np.uint8)                 # every code in both nibbles
        sshape = (m, -(-n // gs)) if along_n else (-(-m // gs), n)
        sc = rng.integers(96, 160, sshape).astype(np.uint8)
        sc.reshape(-1)[:6] = [0, 1, 254, 255, 127, 143]
        dst = torch.zeros((m, n), dtype=TDT[dst_dt], device=DEV)
        cfg = ops.AscendAntiQuantConfig(has_offset=False, is_transpose=bool(tr), k_dim=k_dim)
        para = ops.AscendAntiQuantParam(m=m, n=n, cal_count=cal, group_size=gs)
        ops.ascend_antiquant_policy(dst, to_dev(packed), to_dev(sc), None, para, abi.PER_GROUP, cfg, src_format=fmt)
        d = abi.AntiQuantPolicyDesc(policy=abi.PER_GROUP, src_format=fmt, scale_dtype=abi.E8M0, dst_dtype=dst_dt,
                                    compute=abi.COMPUTE_SCALE_T, has_offset=0, is_transpose=tr, k_dim=k_dim, m=m, n=n,
                                    cal_count=cal, group_size=gs)
        want = orc.antiquant_policy(d, packed, sc, None).view(np.uint16)
        got = bits(dst)
        rows = cal // n
        if dst_dt == abi.BF16:
            nan_w = (want & 0x7FFF) > 0x7F80
            nan_g = (got & 0x7FFF) > 0x7F80
            assert np.array_equal(nan_w[:rows], nan_g[:rows]) and nan_w.any()
            assert np.array_equal(got[:rows][~nan_w[:rows]], want[:rows][~nan_w[:rows]])
            if fmt == abi.QDST_FP4_E2M1:          # 6 * 2^127 overflows bfloat16; 1.75 * 2^127 (e1m2) does not
                assert np.any((want[:rows] & 0x7FFF) == 0x7F80)
        else:
            assert np.array_equal(got[:rows], want[:rows])
            assert np.any((want[:rows] & 0x7FFF) == 0x7BFF)                      # saturation was exercised
        assert not got[rows:].any()


def test_antiquant_fp4_rejects():
    announce("antiquant fp4 rejects")
    src = torch.zeros((4, 32), dtype=torch.uint8, device=DEV)
    sc = torch.full((4, 2), 127, dtype=torch.uint8, device=DEV)
    dst = torch.zeros((4, 64), dtype=torch.float16, device=DEV)
    para = ops.AscendAntiQuantParam(m=4, n=64, cal_count=256, group_size=32)
    with pytest.raises(ops.AscqError, match="PER_GROUP only"):
        ops.ascend_antiquant_policy(dst, src, sc[:, 0].contiguous(), None, para, abi.PER_TOKEN,
                                    ops.AscendAntiQuantConfig(has_offset=False), src_format=abi.QDST_FP4_E2M1)
    with pytest.raises(ops.AscqError, match="no offset"):
        ops.ascend_antiquant_policy(dst, src, sc, sc, para, abi.PER_GROUP,
                                    ops.AscendAntiQuantConfig(has_offset=True), src_format=abi.QDST_FP4_E1M2)
    dst32 = torch.zeros((4, 64), dtype=torch.float32, device=DEV)
    with pytest.raises(ops.AscqError, match="half or bfloat16"):
        ops.ascend_antiquant_policy(dst32, src, sc, None, para, abi.PER_GROUP,
                                    ops.AscendAntiQuantConfig(has_offset=False), src_format=abi.QDST_FP4_E2M1)


@pytest.mark.parametrize("policy", ["tensor", "channel", "token", "group0", "group1"])
def test_dequantize_is_the_matching_ascend_dequant(policy):
    """The unified Dequantize: each policy gives what the operator it forwards to gives (and the oracle)."""
    announce("dequantize", policy)
    rng = np.random.default_rng(17)
    m, n, gs = 40, 96, 32
    src = rng.integers(-2 ** 20, 2 ** 20, (m, n)).astype(np.int32)
    pol = {"tensor": abi.PER_TENSOR, "channel": abi.PER_CHANNEL, "token": abi.PER_TOKEN, "group0": abi.PER_GROUP,
           "group1": abi.PER_GROUP}[policy]
    k_dim = 0 if policy == "group0" else 1
    sshape = {"channel": (n,), "token": (m,), "group0": (-(-m // gs), n), "group1": (m, -(-n // gs))}.get(policy)
    para = ops.AscendQuantParam(m=m, n=n, cal_count=m * n, group_size=gs if pol == abi.PER_GROUP else 0)
    dst = torch.zeros((m, n), dtype=torch.bfloat16, device=DEV)
    d = abi.DequantDesc(policy=pol, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.BF16,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, k_dim=k_dim, m=m, n=n,
                        cal_count=n if pol in (abi.PER_TENSOR, abi.PER_CHANNEL) else m * n, group_size=para.group_size)
    if pol == abi.PER_TENSOR:
        ops.dequantize(dst, to_dev(src), 3.1e-4, para, pol)
        d.scale = 3.1e-4
        want = orc.dequant(d, src)
    else:
        s = rng.uniform(1e-5, 1e-3, sshape).astype(np.float32)
        ops.dequantize(dst, to_dev(src), to_dev(s), para, pol, k_dim=k_dim)
        want = orc.dequant(d, src, s)
    assert np.array_equal(bits(dst), np.asarray(want).reshape(m, -1)[:, :n])


def test_antiquant_per_tensor():
    announce("antiquant per-tensor")
    w = np.arange(-128, 128, dtype=np.int8).reshape(8, 32)
    for dst_dt in (abi.F16, abi.BF16):
        dst = torch.zeros((8, 32), dtype=TDT[dst_dt], device=DEV)
        ops.ascend_antiquant(dst, to_dev(w), -3.25, 0.37, 8)
        d = abi.AntiQuantDesc(src_dtype=abi.I8, dst_dtype=dst_dt, has_offset=1, per_tensor=1, scale=0.37,
                              offset=-3.25, k=8, n=32)
        assert np.array_equal(bits(dst), orc.antiquant(d, w).view(np.uint16))


# ------------------------------------------------------------------ full-size configurations
def test_config2a_full_size_quant():
    announce("config 2a: fp16 [8192, 4096] per-channel quant")
    rng = np.random.default_rng(0x2A)
    x = (rng.standard_normal((8192, 4096)) * 2).astype(np.float16)
    s = (np.float32(127.0) / np.abs(x.astype(np.float32)).max(axis=0)).astype(np.float16)
    dst = torch.zeros((8192, 4096), dtype=torch.int8, device=DEV)
    ops.ascend_quant(dst, to_dev(x), to_dev(s), 0.0)
    d = abi.QuantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.F16, scale_dtype=abi.F16, compute=abi.COMPUTE_F16,
                      round_mode=abi.CAST_RINT, offset_kind=abi.OFFSET_SCALAR, n=4096, cal_count=x.size)
    orc.set_threads(16)
    assert np.array_equal(dst.cpu().numpy(), orc.quant(d, x, s))


def test_config2b_full_size_dequant():
    announce("config 2b: int32 [8192, 4096] per-channel dequant to bf16")
    rng = np.random.default_rng(0x2B)
    src = rng.integers(-2**20, 2**20 + 1, (8192, 4096), dtype=np.int32)
    sc = rng.uniform(1e-5, 1e-3, 4096).astype(np.float32)
    dst = torch.zeros((8192, 4096), dtype=torch.bfloat16, device=DEV)
    ops.ascend_dequant(dst, to_dev(src), to_dev(sc), ops.DequantParams(8192, 4096, 4096),
                       mode=abi.DEQUANT_WITH_MULTI_ROW)
    d = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.BF16,
                        mode=abi.DEQUANT_WITH_MULTI_ROW, m=8192, n=4096, cal_count=4096)
    orc.set_threads(16)
    assert np.array_equal(bits(dst), orc.dequant(d, src, sc))


def test_config2c_full_size_antiquant():
    announce("config 2c: int8 [4096, 11008] per-channel antiquant to fp16")
    rng = np.random.default_rng(0x2C)
    w = rng.integers(-127, 128, (4096, 11008)).astype(np.int8)
    sc = rng.uniform(1e-3, 1e-1, (1, 11008)).astype(np.float16)
    of = rng.integers(-8, 9, (1, 11008)).astype(np.float16)
    dst = torch.zeros((4096, 11008), dtype=torch.float16, device=DEV)
    ops.ascend_antiquant(dst, to_dev(w), to_dev(of), to_dev(sc), 4096, ops.AntiQuantShapeInfo(1, 11008, 1, 11008))
    d = abi.AntiQuantDesc(src_dtype=abi.I8, dst_dtype=abi.F16, has_offset=1, k=4096, n=11008, scale_height=1,
                          scale_width=11008, offset_height=1, offset_width=11008)
    orc.set_threads(16)
    assert np.array_equal(bits(dst), orc.antiquant(d, w, of, sc).view(np.uint16))
