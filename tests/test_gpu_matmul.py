"""GPU parity of the int8 matmul quant path, the quantized grouped matmul and W4A16 against the CPU oracle, through
the C ABI.  int32 accumulators and every epilogue without a transcendental are compared bit for bit (each epilogue
step rounds once in fp32, in the reference's order); FasterGelu outputs within 1 ulp of the output type; W4A16
(free summation order) within the stated tolerance."""
import ctypes as C

import numpy as np
import pytest
import torch

import orc
from ascq import _abi as abi
from ascq import ops
import gpu_util
from gpu_util import DEV, announce, bits, max_ulp, pack_int4, to_dev

pytestmark = pytest.mark.gpu


def rand_i8(rng, shape, lo=-127, hi=127):
    return rng.integers(lo, hi + 1, shape).astype(np.int8)


def run_mm(m, n, k, a, b, *, out, bias=None, quant=None, tok=None, trans_a=False, trans_b=False, act=abi.MM_ACT_NONE,
           scalar=None):
    mm = ops.Matmul(m, n, k, trans_a, trans_b)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b(to_dev(b))
    if bias is not None:
        mm.set_bias(to_dev(bias[0], bias[1]))
    if quant is not None:
        mm.set_quant_vector(to_dev(quant))
    if scalar is not None:
        mm.set_quant_scalar(scalar)
    if tok is not None:
        mm.set_token_scale(to_dev(tok))
    mm.set_activation(act)
    c = torch.zeros((m, n), dtype=out, device=DEV)
    mm.iterate_all(c)
    torch.cuda.synchronize()
    return c, mm.desc


def oracle_mm(desc, a, b, bias=None, quant=None, tok=None):
    orc.set_threads(16)
    return orc.matmul_w8a8(desc, a, b, None if bias is None else bias[0], quant, tok)


# shapes chosen to hit: the 32-row split-K tile, the 128-row tile with a row tail, the 256-row tile with row and
# column tails, K tails (K not a multiple of 128), and the generic kernel (odd sizes)
SHAPES = [(1, 256, 512), (16, 1024, 4096), (32, 264, 1040), (33, 256, 256), (128, 512, 384), (300, 520, 272),
          (1100, 776, 400), (2048, 512, 128), (19, 23, 77), (40, 100, 48),
          # the weight-stream kernel (m <= 32, k % 64 == 0): one chunk, column tails, runs that cross column blocks
          (1, 16, 64), (7, 144, 192), (32, 400, 64), (32, 1040, 2048), (5, 2064, 8192),
          # 128 x 128 tiles with and without a K split, row / column tails
          (33, 144, 128), (200, 528, 384), (512, 272, 256), (130, 2064, 1024),
          # 256-row tiles: a partial last round (narrow tiles), K steps odd and even
          (513, 528, 256), (2048, 2832, 384),
          # four and five K steps: the steady-state loop runs once, then two steps / one step are peeled
          (600, 528, 512), (600, 528, 640), (300, 272, 512), (300, 272, 640),
          # 344 tiles of 256 x 256: wide and narrow tiles in one launch, for B as [k, n] and as [n, k]
          (2048, 11008, 128),
          # more than 8 row tiles: bands of 8 row tiles and a last band of 2 (with a partial last row tile)
          (2500, 784, 128)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("trans_b", [False, True])
def test_int32_accumulators_bit_exact(m, n, k, trans_b):
    announce("matmul int32", m, n, k, trans_b)
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rand_i8(rng, (m, k), -128, 127)
    b = rand_i8(rng, (k, n), -128, 127)
    bias = rng.integers(-10000, 10000, n).astype(np.int32)
    b_in = np.ascontiguousarray(b.T) if trans_b else b
    c, desc = run_mm(m, n, k, a, b_in, out=torch.int32, bias=(bias, None), trans_b=trans_b)
    want = a.astype(np.int64) @ b.astype(np.int64) + bias
    assert np.array_equal(c.cpu().numpy().astype(np.int64), want)
    assert np.array_equal(oracle_mm(desc, a, b_in, (bias, None)).astype(np.int64), want)


def test_trans_a_generic_path():
    announce("matmul trans_a")
    rng = np.random.default_rng(3)
    m, n, k = 48, 64, 96
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    c, _ = run_mm(m, n, k, np.ascontiguousarray(a.T), b, out=torch.int32, trans_a=True)
    assert np.array_equal(c.cpu().numpy().astype(np.int64), a.astype(np.int64) @ b.astype(np.int64))


def test_config1_small_w8a8_bf16_with_bias():
    """A int8 [256,1024], B int8 [1024,1024], per-channel fp32 deqScale in [1e-4,1e-3], fp32 bias N(0,1) -> bf16."""
    announce("config 1")
    rng = np.random.default_rng(0xC1)
    m, n, k = 256, 1024, 1024
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    sc = rng.uniform(1e-4, 1e-3, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c, desc = run_mm(m, n, k, a, b, out=torch.bfloat16, bias=(bias, None), quant=sc)
    assert np.array_equal(bits(c), oracle_mm(desc, a, b, (bias, None), sc))


@pytest.mark.parametrize("m", [1, 16, 128, 2048])
def test_config3_w8a8_linear(m):
    """bf16 activations quantised per token on the GPU, int8 weights [4096,11008], fused dequant to bf16."""
    announce("config 3", m)
    rng = np.random.default_rng(0xC3 + m)
    k, n = 4096, 11008
    x = orc.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    w = rand_i8(rng, (k, n))
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    q, ts = ops.dynamic_quant_per_token(to_dev(x, "bf16"))
    wq, wts = orc.dynamic_quant_per_token(abi.BF16, x)
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(ts.cpu().numpy(), wts)
    c, desc = run_mm(m, n, k, wq, w, out=torch.bfloat16, quant=cs, tok=wts)
    want = oracle_mm(desc, wq, w, None, cs, wts)
    got = bits(c)
    assert max_ulp(got, want) <= 1
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m", [1, 16, 17, 32])
def test_config3_w8a8_linear_weights_as_n_k(m):
    """Config 3's decode sizes on weights kept as [n, k] (isTransposeB): the whole-column kernel, one launch, no
    workspace; bf16 output with channel and token scales, bit-exact against the oracle on the same weights."""
    announce("config 3 [n, k]", m)
    rng = np.random.default_rng(0xC3 + 100 + m)
    k, n = 4096, 11008
    a = rand_i8(rng, (m, k))
    wt = rand_i8(rng, (n, k))
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c, desc = run_mm(m, n, k, a, wt, out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts, trans_b=True)
    orc.set_threads(16)
    assert np.array_equal(bits(c), oracle_mm(desc, a, wt, (bias, None), cs, ts))
    wsz = C.c_size_t(1)
    assert abi.load_library().ascq_matmul_w8a8_workspace_size(C.byref(desc), C.byref(wsz)) == abi.OK and wsz.value == 0
    # int8 requantised output and SwiGLU through the same kernel
    words = (cs * 50).astype(np.float32).view(np.uint32).astype(np.uint64) | (np.uint64(1) << np.uint64(46))
    c8, d8 = run_mm(m, n, k, a, wt, out=torch.int8, quant=words, trans_b=True)
    assert np.array_equal(bits(c8), oracle_mm(d8, a, wt, None, words))


def run_mm_packed(m, n, k, a, b, *, out, bias=None, quant=None, tok=None, trans_b=False, act=abi.MM_ACT_NONE,
                  scalar=None):
    """run_mm on weights packed by ops.pack_weight_w8 (from [k, n], or from [n, k] with trans_b); the descriptor it
    returns describes the same matmul on the unpacked [k, n] weights, for the oracle."""
    mm = ops.Matmul(m, n, k)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b_packed(ops.pack_weight_w8(to_dev(b), k, n, trans_b))
    if bias is not None:
        mm.set_bias(to_dev(bias[0], bias[1]))
    if quant is not None:
        mm.set_quant_vector(to_dev(quant))
    if scalar is not None:
        mm.set_quant_scalar(scalar)
    if tok is not None:
        mm.set_token_scale(to_dev(tok))
    mm.set_activation(act)
    c = torch.zeros((m, n), dtype=out, device=DEV)
    mm.iterate_all(c)
    torch.cuda.synchronize()
    return c, mm.desc


def w8_packed_reference(w, k, n):
    """The packed int8 layout restated in numpy: slabs of 16 columns, tiles of 64 k, lane l of a tile owns column
    l % 16 and the 16 bytes k 16 (l / 16) .. + 15; zeros past n and k, 16 tiles of zeros behind the last slab."""
    slabs, ktiles = (n + 15) // 16, (k + 63) // 64
    full = np.zeros((ktiles * 64, slabs * 16), dtype=np.int8)
    full[:k, :n] = w
    t = full.reshape(ktiles, 4, 16, slabs, 16)            # tile, k quarter, byte, slab, column
    body = np.ascontiguousarray(t.transpose(3, 0, 1, 4, 2)).reshape(-1)   # slab, tile, k quarter, column, byte
    return np.concatenate([body, np.zeros(16 * 1024, dtype=np.int8)]).view(np.uint8)


@pytest.mark.parametrize("k,n", [(64, 16), (128, 40), (200, 1040), (1024, 272)])
def test_pack_weight_w8_layout(k, n):
    announce("pack w8", k, n)
    rng = np.random.default_rng(k + n)
    w = rand_i8(rng, (k, n))
    want = w8_packed_reference(w, k, n)
    assert np.array_equal(ops.pack_weight_w8(to_dev(w), k, n).cpu().numpy(), want)
    assert np.array_equal(ops.pack_weight_w8(to_dev(np.ascontiguousarray(w.T)), k, n, trans_b=True).cpu().numpy(), want)


@pytest.mark.parametrize("m", [1, 2, 3, 5, 8, 16, 17, 20, 31, 32, 33, 50])
@pytest.mark.parametrize("n,k", [(16, 64), (48, 128), (1040, 512), (272, 4096), (96, 8192), (32, 16384), (2064, 192)])
def test_w8a8_packed_small(m, n, k):
    """The one-launch kernel on packed weights computes what ascq_matmul_w8a8 computes: int32 accumulators and the
    dequantising epilogues bit for bit against the oracle on the unpacked weights.  k of one tile (seven wavefronts
    without work), column tails, more rows than a pass, k long enough for several batches per slab; more rows than a
    pass holds with the weights held in registers (k up to 16384)."""
    announce("w8a8 packed", m, n, k)
    rng = np.random.default_rng(m * 31 + n + k)
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    c, desc = run_mm_packed(m, n, k, a, b, out=torch.int32)
    assert np.array_equal(c.cpu().numpy(), a.astype(np.int64) @ b.astype(np.int64))
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c, desc = run_mm_packed(m, n, k, a, np.ascontiguousarray(b.T), out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts,
                            trans_b=True)
    assert np.array_equal(bits(c), oracle_mm(desc, a, b, (bias, None), cs, ts))
    # requantised int8 output from uint64 words, int32 bias ahead of the dequantisation, FasterGelu to half
    words = (cs * 50).astype(np.float32).view(np.uint32).astype(np.uint64) | (np.uint64(1) << np.uint64(46))
    bias_i = rng.integers(-1000, 1000, n).astype(np.int32)
    c8, d8 = run_mm_packed(m, n, k, a, b, out=torch.int8, bias=(bias_i, None), quant=words)
    assert np.array_equal(bits(c8), oracle_mm(d8, a, b, (bias_i, None), words))
    cg, dg = run_mm_packed(m, n, k, a, b, out=torch.float16, scalar=1e-3, act=abi.MM_ACT_FASTER_GELU)
    assert max_ulp(bits(cg), oracle_mm(dg, a, b).view(np.uint16), "f16") <= 1


@pytest.mark.parametrize("m", [1, 2, 3, 5, 8, 13, 16])
@pytest.mark.parametrize("n,k", [(16, 64), (48, 128), (1040, 512), (272, 4096), (2064, 192), (100, 5632), (96, 8192),
                                 (40, 11008), (4100, 256)])
def test_w8a8_decode_on_n_k_weights_through_lds(m, n, k):
    """Up to 16 rows on weights kept as [n, k]: where the staged activations leave 64 KiB of LDS free the weights go
    through a ring there (four columns' 256 bytes per load, XOR-swizzled pieces), otherwise straight into registers
    (long k with many rows).  k of one tile (seven wavefronts without work), column counts that are no multiple of 16
    (the last slab's columns past n read as zeros), several slabs per workgroup, batches that end inside a wavefront's
    range.  int32 accumulators exactly, the dequantising and the requantising epilogue against the oracle."""
    announce("w8a8 [n, k] decode", m, n, k)
    rng = np.random.default_rng(m * 47 + n + k)
    a, b = rand_i8(rng, (m, k), -128, 127), rand_i8(rng, (k, n), -128, 127)
    bt = np.ascontiguousarray(b.T)
    c, _ = run_mm(m, n, k, a, bt, out=torch.int32, trans_b=True)
    assert np.array_equal(c.cpu().numpy(), a.astype(np.int64) @ b.astype(np.int64))
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c, desc = run_mm(m, n, k, a, bt, out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts, trans_b=True)
    assert np.array_equal(bits(c), oracle_mm(desc, a, bt, (bias, None), cs, ts))  # (the descriptor says [n, k])
    words = (cs * 50).astype(np.float32).view(np.uint32).astype(np.uint64) | (np.uint64(1) << np.uint64(46))
    bias_i = rng.integers(-1000, 1000, n).astype(np.int32)
    c8, d8 = run_mm(m, n, k, a, bt, out=torch.int8, bias=(bias_i, None), quant=words, trans_b=True)
    assert np.array_equal(bits(c8), oracle_mm(d8, a, bt, (bias_i, None), words))


@pytest.mark.parametrize("m", [17, 33, 47, 64, 100, 128, 129, 224, 225, 300])
@pytest.mark.parametrize("n,k", [(16, 64), (48, 128), (1040, 512), (272, 4096), (2064, 192), (13000, 256), (96, 4160)])
def test_w8a8_weights_held_in_registers(m, n, k):
    """More than 16 rows on packed weights (17 to 224 on [n, k] weights): the weights of a workgroup's columns stay in
    registers and the activations stream past them, the sums and the epilogue in blocks of 128 rows (on [n, k]
    weights, more rows take the other kernels).  int32 accumulators against int64
    arithmetic, the dequantising epilogue bit for bit against the oracle, both forms."""
    announce("w8a8 weights in registers", m, n, k)
    rng = np.random.default_rng(m * 37 + n + k)
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    bt = np.ascontiguousarray(b.T)
    want = a.astype(np.int64) @ b.astype(np.int64)
    c, _ = run_mm_packed(m, n, k, a, b, out=torch.int32)
    assert np.array_equal(c.cpu().numpy(), want)
    c, _ = run_mm(m, n, k, a, bt, out=torch.int32, trans_b=True)
    assert np.array_equal(c.cpu().numpy(), want)
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c, desc = run_mm_packed(m, n, k, a, b, out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts)
    gold = oracle_mm(desc, a, b, (bias, None), cs, ts)
    assert np.array_equal(bits(c), gold)
    c, desc = run_mm(m, n, k, a, bt, out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts, trans_b=True)
    assert np.array_equal(bits(c), gold)
    if n > 2064 or k > 4096:
        return
    # requantised int8 output from uint64 words (one of them with the pre-shift), int32 bias ahead of the
    # dequantisation; FasterGelu to half from a scalar scale
    words = (cs * 50).astype(np.float32).view(np.uint32).astype(np.uint64) | (np.uint64(1) << np.uint64(46))
    words[n // 2] |= (np.uint64(1) << np.uint64(36)) | (np.uint64(3) << np.uint64(32))
    bias_i = rng.integers(-1000, 1000, n).astype(np.int32)
    c8, d8 = run_mm_packed(m, n, k, a, b, out=torch.int8, bias=(bias_i, None), quant=words)
    gold8 = oracle_mm(d8, a, b, (bias_i, None), words)
    assert np.array_equal(bits(c8), gold8)
    c8, _ = run_mm(m, n, k, a, bt, out=torch.int8, bias=(bias_i, None), quant=words, trans_b=True)
    assert np.array_equal(bits(c8), gold8)
    cg, dg = run_mm_packed(m, n, k, a, b, out=torch.float16, scalar=1e-3, act=abi.MM_ACT_FASTER_GELU)
    assert max_ulp(bits(cg), oracle_mm(dg, a, b).view(np.uint16), "f16") <= 1


@pytest.mark.parametrize("m", [13, 16, 17, 64, 129, 300])
@pytest.mark.parametrize("n,k", [(48, 11008), (272, 8192), (4112, 4160), (1040, 5632), (40, 16384), (96, 14336),
                                 (528, 12352)])
def test_w8a8_weights_held_in_registers_long_k(m, n, k):
    """k beyond 4096 (up to 16384): a wavefront's k range of its slabs is held in chunks of 8 tiles, two slabs by two
    chunks (k up to 8192; n = 4112 gives workgroups two slabs) or one slab by four, and the activations stream past
    them a chunk at a time.  Also the calls of 13 to 16 rows whose staged activations no longer fit the LDS in one
    pass.  int32 accumulators against exact double arithmetic, the dequantising epilogue bit for bit against the
    oracle, packed and [n, k] weights."""
    announce("w8a8 weights in registers, long k", m, n, k)
    rng = np.random.default_rng(m * 41 + n + k)
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    bt = np.ascontiguousarray(b.T)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.int64)  # sums below 2^53: exact
    c, _ = run_mm_packed(m, n, k, a, b, out=torch.int32)
    assert np.array_equal(c.cpu().numpy(), want)
    c, _ = run_mm(m, n, k, a, bt, out=torch.int32, trans_b=True)
    assert np.array_equal(c.cpu().numpy(), want)
    if n > 2064:
        return
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c, desc = run_mm_packed(m, n, k, a, b, out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts)
    gold = oracle_mm(desc, a, b, (bias, None), cs, ts)
    assert np.array_equal(bits(c), gold)
    c, desc = run_mm(m, n, k, a, bt, out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts, trans_b=True)
    assert np.array_equal(bits(c), gold)


@pytest.mark.parametrize("m", [129, 200, 256, 300, 513, 700, 1100])
@pytest.mark.parametrize("n,k", [(256, 128), (1040, 512), (272, 4096), (2064, 384), (4112 + 16, 256), (96, 1152)])
def test_w8a8_packed_many_rows_on_the_tile_kernels(m, n, k):
    """Many rows on packed weights (n a multiple of 16, k of 128): the direct-to-LDS tile kernels (128 x 128 tiles up to
    512 rows, 256-row tiles beyond, with the narrow tiles of a partly filled last round) read the packed tiles as they
    lie.  int32 accumulators against exact double arithmetic; the dequantising epilogue, the requantising one and
    SwiGLU against the oracle."""
    announce("w8a8 packed, tile kernels", m, n, k)
    rng = np.random.default_rng(m * 43 + n + k)
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.int64)
    c, _ = run_mm_packed(m, n, k, a, b, out=torch.int32)
    assert np.array_equal(c.cpu().numpy(), want)
    if n > 2064:
        return
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c, desc = run_mm_packed(m, n, k, a, np.ascontiguousarray(b.T), out=torch.bfloat16, bias=(bias, None), quant=cs, tok=ts,
                            trans_b=True)
    assert np.array_equal(bits(c), oracle_mm(desc, a, b, (bias, None), cs, ts))
    words = (cs * 50).astype(np.float32).view(np.uint32).astype(np.uint64) | (np.uint64(1) << np.uint64(46))
    words[n // 2] |= (np.uint64(1) << np.uint64(36)) | (np.uint64(3) << np.uint64(32))
    bias_i = rng.integers(-1000, 1000, n).astype(np.int32)
    c8, d8 = run_mm_packed(m, n, k, a, b, out=torch.int8, bias=(bias_i, None), quant=words)
    assert np.array_equal(bits(c8), oracle_mm(d8, a, b, (bias_i, None), words))
    # SwiGLU of the column pairs in the tile kernels' epilogue (16-bit outputs)
    css = rng.uniform(1e-4, 4e-4, n).astype(np.float32)
    tss = rng.uniform(0.5, 2.0, m).astype(np.float32)
    mm = ops.Matmul(m, n, k, False, False)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b_packed(ops.pack_weight_w8(to_dev(b), k, n))
    mm.set_quant_vector(to_dev(css))
    mm.set_token_scale(to_dev(tss))
    mm.set_activation(abi.MM_ACT_SWIGLU, 1.702)
    cg = torch.zeros((m, n // 2), dtype=torch.bfloat16, device=DEV)
    mm.iterate_all(cg)
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                       has_tok_scale=1, activation=abi.MM_ACT_SWIGLU, act_beta=1.702)
    swiglu_close(bits(cg), oracle_mm(d, a, b, None, css, tss).view(np.uint16), "bf16")


@pytest.mark.parametrize("m", [1, 16, 32])
def test_config3_w8a8_linear_packed(m):
    """Config 3's decode sizes on packed weights: per-token quantisation on the GPU, one launch for the matmul, bf16
    output bit-exact against the oracle."""
    announce("config 3 packed", m)
    rng = np.random.default_rng(0xC3 + m)
    k, n = 4096, 11008
    x = orc.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    w = rand_i8(rng, (k, n))
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    q, ts = ops.dynamic_quant_per_token(to_dev(x, "bf16"))
    wq, wts = orc.dynamic_quant_per_token(abi.BF16, x)
    assert np.array_equal(q.cpu().numpy(), wq) and np.array_equal(ts.cpu().numpy(), wts)
    c, desc = run_mm_packed(m, n, k, wq, w, out=torch.bfloat16, quant=cs, tok=wts)
    assert np.array_equal(bits(c), oracle_mm(desc, wq, w, None, cs, wts))


def test_w8a8_packed_rejects():
    lib = abi.load_library()
    t = torch.zeros(1 << 16, dtype=torch.int8, device=DEV)
    c = torch.zeros(1 << 12, dtype=torch.int32, device=DEV)

    def call(**kw):
        d = abi.MatmulDesc(m=1, n=64, k=128, out_dtype=abi.I32, quant_mode=abi.MM_QUANT_NONE, scale_format=abi.MM_SCALE_U64)
        for key, v in kw.items():
            setattr(d, key, v)
        return lib.ascq_matmul_w8a8_packed(C.byref(d), C.c_void_p(c.data_ptr()), C.c_void_p(t.data_ptr()),
                                           C.c_void_p(t.data_ptr()), None, None, None, None)

    assert call() == abi.OK
    assert call(k=100) == abi.EUNSUPPORTED          # k % 64
    assert call(trans_a=1) == abi.EUNSUPPORTED
    assert call(b_format=abi.MM_B_NZ) != abi.OK
    torch.cuda.synchronize()


@pytest.mark.parametrize("m", [48, 128, 300, 512])
def test_config3_w8a8_mid_m_both_weight_layouts(m):
    """Config 3 between the decode sizes and the large tiles: 128 x 128 direct-to-LDS tiles, K split four ways for one
    row tile and not at all for more, on weights as [k, n]; on [n, k] weights the same tiles from 225 rows on and the
    weights-in-registers kernel below; bit-exact against the oracle."""
    announce("config 3 mid m", m)
    rng = np.random.default_rng(0xC3 + 200 + m)
    k, n = 4096, 11008
    a = rand_i8(rng, (m, k))
    w = rand_i8(rng, (k, n))
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    c, desc = run_mm(m, n, k, a, w, out=torch.bfloat16, quant=cs, tok=ts)
    want = oracle_mm(desc, a, w, None, cs, ts)
    assert np.array_equal(bits(c), want)
    ct, _ = run_mm(m, n, k, a, np.ascontiguousarray(w.T), out=torch.bfloat16, quant=cs, tok=ts, trans_b=True)
    assert np.array_equal(bits(ct), want)
    # [k, n]: one row tile splits K four ways through the workspace; [n, k]: up to 224 rows need none
    wsz = C.c_size_t(0)
    assert abi.load_library().ascq_matmul_w8a8_workspace_size(C.byref(desc), C.byref(wsz)) == abi.OK
    assert wsz.value == (4 * m * n * 4 if m <= 128 else 0)
    desc.trans_b = 1
    assert abi.load_library().ascq_matmul_w8a8_workspace_size(C.byref(desc), C.byref(wsz)) == abi.OK
    assert wsz.value == 0


def test_fixpipe_modes_uint64_words():
    announce("matmul fixpipe words: VDEQF16, DEQF16 scalar, VREQ8, bf16")
    rng = np.random.default_rng(21)
    m, n, k = 64, 256, 256
    a, b = rand_i8(rng, (m, k), -10, 10), rand_i8(rng, (k, n), -10, 10)
    bias = rng.integers(-2, 2, n).astype(np.int32)
    qf = rng.uniform(0.1, 2.0, n).astype(np.float32)
    qf[0], qf[1] = 3000.0, -3000.0
    words = qf.view(np.uint32).astype(np.uint64) | (np.uint64(7) << np.uint64(37)) | (np.uint64(1) << np.uint64(46))
    for out in (torch.float16, torch.bfloat16, torch.int8):
        c, desc = run_mm(m, n, k, a, b, out=out, bias=(bias, None), quant=words)
        want = oracle_mm(desc, a, b, (bias, None), words)
        assert np.array_equal(bits(c), want.view(np.uint16) if out == torch.float16 else want)
    assert (np.abs(bits(run_mm(m, n, k, a, b, out=torch.float16, quant=words)[0]).view(np.float16)
                   .astype(np.float32)) == 65504).any()            # the fp16 output saturates instead of overflowing
    c, desc = run_mm(m, n, k, a, b, out=torch.float16, bias=(bias, None),
                     scalar=ops.pack_quant_param(0.1))
    assert np.array_equal(bits(c), oracle_mm(desc, a, b, (bias, None)).view(np.uint16))
    c, desc = run_mm(m, n, k, a, b, out=torch.float32, scalar=0.1)
    assert np.array_equal(bits(c), oracle_mm(desc, a, b))


@pytest.mark.parametrize("m,n,k,trans_b", [(7, 144, 192, False), (64, 256, 256, False), (12, 272, 256, True),
                                           (200, 528, 384, False), (600, 528, 640, False), (19, 23, 77, False)])
def test_fixpipe_pre_shift_words(m, n, k, trans_b):
    """Quant words with the mode-control bit 36: the accumulator is shifted right by bits [35:32] and saturated before
    the multiply.  Every column draws its own bit and shift; all four output types, and a scalar word."""
    announce(f"matmul fixpipe pre-shift words m={m} n={n} k={k} trans_b={trans_b}")
    rng = np.random.default_rng(1000 + m)
    a = rand_i8(rng, (m, k), -127, 128)
    b = rand_i8(rng, (n, k) if trans_b else (k, n), -127, 128)
    bias = rng.integers(-3000000, 3000000, n).astype(np.int32)
    qf = rng.uniform(0.01, 1.5, n).astype(np.float32)
    sh = rng.integers(0, 16, n).astype(np.uint64)
    on = rng.integers(0, 2, n).astype(np.uint64)
    on[:4], sh[:4] = 1, (0, 1, 4, 15)
    words = (qf.view(np.uint32).astype(np.uint64) | (sh << np.uint64(32)) | (on << np.uint64(36)) |
             (rng.integers(0, 512, n).astype(np.uint64) << np.uint64(37)) |
             (rng.integers(0, 2, n).astype(np.uint64) << np.uint64(46)))
    for out in (torch.float16, torch.int8, torch.bfloat16, torch.float32):
        c, desc = run_mm(m, n, k, a, b, out=out, bias=(bias, None), quant=words, trans_b=trans_b)
        want = oracle_mm(desc, a, b, (bias, None), words)
        assert np.array_equal(bits(c), want.view(np.uint16) if out == torch.float16 else want), out
    plain = words & ~(np.uint64(1) << np.uint64(36))
    c0, _ = run_mm(m, n, k, a, b, out=torch.float16, bias=(bias, None), quant=plain, trans_b=trans_b)
    c1, _ = run_mm(m, n, k, a, b, out=torch.float16, bias=(bias, None), quant=words, trans_b=trans_b)
    assert not np.array_equal(bits(c0), bits(c1)), "bit 36 had no effect"
    if n % 2 == 0 and not trans_b:      # SwiGLU over column pairs that shift differently (small scales keep exp in range)
        sw = words & ~np.uint64(0xFFFFFFFF) | (qf * np.float32(1e-4)).view(np.uint32).astype(np.uint64)
        mm = ops.Matmul(m, n, k)
        mm.set_tensor_a(to_dev(a))
        mm.set_tensor_b(to_dev(b))
        mm.set_quant_vector(to_dev(sw))
        mm.set_bias(to_dev(bias))
        mm.set_activation(abi.MM_ACT_SWIGLU, 1.0)
        c = torch.zeros((m, n // 2), dtype=torch.float16, device=DEV)
        mm.iterate_all(c)
        swiglu_close(bits(c), oracle_mm(mm.desc, a, b, (bias, None), sw).view(np.uint16), "f16")
    scalar = int(np.float32(0.37).view(np.uint32)) | (3 << 32) | (1 << 36) | (9 << 37) | (1 << 46)
    for out in (torch.float16, torch.int8):
        c, desc = run_mm(m, n, k, a, b, out=out, bias=(bias, None), scalar=scalar, trans_b=trans_b)
        want = oracle_mm(desc, a, b, (bias, None))
        assert np.array_equal(bits(c), want.view(np.uint16) if out == torch.float16 else want), out


def test_post_bias_bf16_and_gelu():
    announce("matmul bf16 bias + token scale + FasterGelu")
    rng = np.random.default_rng(22)
    m, n, k = 96, 512, 384
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    cs = rng.uniform(1e-4, 1e-3, n).astype(np.float32)
    ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
    bias = orc.f32_to_bf16_bits(rng.standard_normal(n).astype(np.float32))
    c, desc = run_mm(m, n, k, a, b, out=torch.bfloat16, bias=(bias, "bf16"), quant=cs, tok=ts)
    assert np.array_equal(bits(c), oracle_mm(desc, a, b, (bias, None), cs, ts))
    c, desc = run_mm(m, n, k, a, b, out=torch.float16, quant=cs, tok=ts, act=abi.MM_ACT_FASTER_GELU)
    want = oracle_mm(desc, a, b, None, cs, ts)
    assert max_ulp(bits(c), want.view(np.uint16)) <= 1             # expf differs by at most an ulp of fp32


# ------------------------------------------------------------------ grouped matmul
def run_group(m, k, n, counts, kind, out, rng, with_bias, act, rows_cap=None):
    G = len(counts)
    x, w = rand_i8(rng, (m, k)), rand_i8(rng, (G, k, n))
    cs = rng.uniform(1e-4, 1e-2, (G, n)).astype(np.float32)
    ts = rng.uniform(1e-3, 1e-1, m).astype(np.float32)
    bias = orc.f32_to_bf16_bits(rng.standard_normal((G, n)).astype(np.float32)) if with_bias else None
    gl = np.asarray(counts, dtype=np.int64) if kind == abi.GROUP_LIST_COUNTS else np.cumsum(counts).astype(np.int64)
    y = torch.zeros((m, n), dtype=out, device=DEV)
    y.view(torch.int16).fill_(0x7E7E)
    ops.quant_group_matmul(y, to_dev(x), to_dev(w), to_dev(gl), to_dev(cs), to_dev(ts),
                           None if bias is None else to_dev(bias, "bf16"), kind, act)
    torch.cuda.synchronize()
    mm = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16 if out == torch.bfloat16 else abi.F16,
                        quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32, has_tok_scale=1,
                        bias_kind=abi.MM_BIAS_BF16_POST if with_bias else abi.MM_BIAS_NONE, activation=act)
    d = abi.GroupMatmulDesc(mm=mm, groups=G, group_list_kind=kind)
    orc.set_threads(16)
    want = orc.group_matmul_w8a8(d, x, w, bias, cs, ts, gl, fill=0x7E7E)
    return bits(y), (want.view(np.uint16) if want.dtype == np.float16 else want)


@pytest.mark.parametrize("kind", [abi.GROUP_LIST_COUNTS, abi.GROUP_LIST_PREFIX_SUM])
@pytest.mark.parametrize("counts", [[30, 0, 1, 45, 12], [256, 256], [0, 0, 700, 0], [1, 1, 1, 1, 1, 1, 1, 1],
                                    [513, 255, 0, 256]])
def test_group_matmul_edge_cases(kind, counts):
    announce("grouped matmul", kind, counts)
    rng = np.random.default_rng(sum(counts) + len(counts))
    m = sum(counts) + 8                                         # 8 rows belong to no group and stay untouched
    got, want = run_group(m, 256, 520, counts, kind, torch.bfloat16, rng, True, abi.MM_ACT_NONE)
    assert np.array_equal(got, want)
    assert np.all(got[sum(counts):] == 0x7E7E)


def test_group_matmul_reference_example_form():
    """The reference example's form: counts group list, no bias, FasterGelu, fp16 output."""
    announce("grouped matmul, example form")
    rng = np.random.default_rng(77)
    got, want = run_group(512, 256, 512, [128] * 4, abi.GROUP_LIST_COUNTS, torch.float16, rng, False,
                          abi.MM_ACT_FASTER_GELU)
    assert max_ulp(got, want) <= 1


def test_config5_moe_up_projection():
    """8 experts, 4096 tokens from a seeded multinomial, K=4096, N=14336, bf16 bias, prefix-sum group list."""
    announce("config 5")
    rng = np.random.default_rng(0xC5)
    counts = rng.multinomial(4096, [1 / 8] * 8).tolist()
    got, want = run_group(4096, 4096, 14336, counts, abi.GROUP_LIST_PREFIX_SUM, torch.bfloat16, rng, True,
                          abi.MM_ACT_NONE)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("counts,act", [([600, 40, 560], abi.MM_ACT_NONE), ([200, 0, 513, 129, 128, 1], abi.MM_ACT_FASTER_GELU),
                                        ([300, 300, 300, 300], abi.MM_ACT_SWIGLU)])
def test_group_matmul_all_tile_shapes(counts, act):
    """Enough 256-row tiles and tile columns that the launch holds a whole round of 256 x 256 tiles, a partial round
    of 256 x 128 tiles (the last of them 80 columns wide) and 128-row tiles for the groups' short remainders; groups
    with 128, 129 and 200 remainder rows sit on either side of the rule that picks the row-tile height."""
    announce("grouped matmul, every tile shape", counts, act)
    rng = np.random.default_rng(len(counts))
    m, k, n = sum(counts) + 3, 128, 16976
    out = torch.float16 if act == abi.MM_ACT_FASTER_GELU else torch.bfloat16
    if act == abi.MM_ACT_SWIGLU:
        x, w = rand_i8(rng, (m, k)), rand_i8(rng, (len(counts), k, n))
        cs = rng.uniform(1e-4, 1e-3, (len(counts), n)).astype(np.float32)
        ts = rng.uniform(1e-2, 1e-1, m).astype(np.float32)
        gl = np.asarray(counts, dtype=np.int64)
        y = torch.zeros((m, n // 2), dtype=out, device=DEV)
        y.view(torch.int16).fill_(0x7E7E)
        ops.quant_group_matmul(y, to_dev(x), to_dev(w), to_dev(gl), to_dev(cs), to_dev(ts), None, abi.GROUP_LIST_COUNTS,
                               act, act_beta=1.0)
        torch.cuda.synchronize()
        mm = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                            scale_format=abi.MM_SCALE_F32, has_tok_scale=1, activation=act, act_beta=1.0)
        orc.set_threads(16)
        want = orc.group_matmul_w8a8(abi.GroupMatmulDesc(mm=mm, groups=len(counts), group_list_kind=abi.GROUP_LIST_COUNTS),
                                     x, w, None, cs, ts, gl, fill=0x7E7E)
        got = bits(y)
        assert np.all(got[sum(counts):] == 0x7E7E)
        rows = sum(counts)
        assert max_ulp(got[:rows], want.view(np.uint16)[:rows], "bf16") <= 1  # expf differs by at most an ulp of fp32
        assert np.mean(got[:rows] == want.view(np.uint16)[:rows]) > 0.98
        return
    got, want = run_group(m, k, n, counts, abi.GROUP_LIST_COUNTS, out, rng, act == abi.MM_ACT_NONE, act)
    if act == abi.MM_ACT_NONE:
        assert np.array_equal(got, want)
    else:
        assert np.all(got[sum(counts):] == 0x7E7E)
        assert max_ulp(got[:sum(counts)], want[:sum(counts)]) <= 1


# ------------------------------------------------------------------ W4A16
def w4_case(rng, m, k, n, gs, has_offset):
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = rng.integers(-8, 8, (k, n)).astype(np.int8)
    sc = rng.uniform(1e-3, 1e-2, (k // gs, n)).astype(np.float16)
    of = rng.integers(-8, 8, (k // gs, n)).astype(np.float16) if has_offset else None
    return x, pack_int4(w), sc, of


@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 9, 16, 19, 32, 33, 37, 70])
@pytest.mark.parametrize("k,n,gs", [(512, 1024, 128), (1024, 544, 64), (256, 66, 128), (384, 512, 384)])
@pytest.mark.parametrize("has_offset", [True, False])
def test_w4a16_small(m, k, n, gs, has_offset):
    announce("w4a16", m, k, n, gs, has_offset)
    rng = np.random.default_rng(m + k + n)
    x, wp, sc, of = w4_case(rng, m, k, n, gs, has_offset)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.matmul_w4a16(y, to_dev(x), to_dev(wp), to_dev(sc), None if of is None else to_dev(of), gs)
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=gs, has_offset=int(has_offset))
    want = orc.matmul_w4a16(d, x, wp, sc, of)
    got = y.cpu().numpy()
    # fp32 accumulation in a different order than the oracle's: rel-err <= 1e-3 of the row scale, and <= 1 fp16 ulp
    # wherever the result is not close to a cancellation
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ref = np.abs(x.astype(np.float64)).sum(axis=1, keepdims=True) * 8 * 1e-2      # bound on sum |x||w|
    assert np.all(err <= 1e-3 * ref + 1e-6)
    assert np.mean(got.view(np.uint16) == want.view(np.uint16)) > 0.9


def w4_packed_reference(w_bytes, k, n):
    """The packed int4 layout restated in numpy: slabs of 16 columns, tiles of 128 k, lane l of a tile owns column l % 16
    and k 32 (l / 16) .. + 31, dword d holds k + 8 d .. + 7 with k offsets 0..7 in nibbles 0 4 1 5 2 6 3 7, nibbles stored as
    w + 8; 16 tiles of w = 0 behind the last slab."""
    slabs, ktiles = (n + 15) // 16, (k + 127) // 128
    u = np.full((ktiles * 128, slabs * 16), 8, dtype=np.uint32)                    # w = 0 where there is no weight
    lo, hi = w_bytes & 15, w_bytes >> 4
    nib = np.empty((k, n), dtype=np.uint32)
    nib[:, 0::2], nib[:, 1::2] = lo, hi
    u[:k, :n] = nib ^ 8
    u = u.reshape(ktiles, 4, 4, 8, slabs, 16)                                      # tile, g, d, e, slab, j
    pos = np.array([0, 4, 1, 5, 2, 6, 3, 7], dtype=np.uint32)                      # nibble of k offset e
    words = (u << (4 * pos)[None, None, None, :, None, None]).sum(axis=3, dtype=np.uint64).astype(np.uint32)
    words = words.transpose(3, 0, 1, 4, 2)                                         # slab, tile, g, j, d
    body = np.ascontiguousarray(words).reshape(-1)
    pad = np.full(16 * 256, 0x88888888, dtype=np.uint32)
    return np.concatenate([body, pad]).view(np.uint8)


@pytest.mark.parametrize("k,n", [(128, 16), (256, 40), (384, 1040), (1024, 272)])
def test_pack_weight_w4_layout(k, n):
    announce("pack w4", k, n)
    rng = np.random.default_rng(k + n)
    wp = pack_int4(rng.integers(-8, 8, (k, n)).astype(np.int8))
    got = ops.pack_weight_w4(to_dev(wp), k, n).cpu().numpy()
    assert np.array_equal(got, w4_packed_reference(wp, k, n))


def w4_check(got, want, x):
    # fp32 accumulation in a different order than the oracle's: rel-err <= 1e-3 of the row scale, and bit-identical
    # halves nearly everywhere (<= 1 fp16 ulp wherever the result is not close to a cancellation)
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ref = np.abs(x.astype(np.float64)).sum(axis=1, keepdims=True) * 8 * 1e-2      # bound on sum |x||w|
    assert np.all(err <= 1e-3 * ref + 1e-6)
    assert np.mean(got.view(np.uint16) == want.view(np.uint16)) > 0.9


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 9, 16, 17, 33])
@pytest.mark.parametrize("k,n,gs", [(512, 1024, 128), (1024, 544, 64), (256, 40, 32), (384, 512, 128), (2048, 272, 256),
                                     (2048, 64, 512), (128, 4112, 128)])
@pytest.mark.parametrize("offset", ["int", "frac", None])
def test_w4a16_packed_small(m, k, n, gs, offset):
    """The pre-packed weight path computes what the [k, n / 2] path computes (same oracle)."""
    announce("w4a16 packed", m, k, n, gs, offset)
    rng = np.random.default_rng(m + k + n)
    x, wp, sc, of = w4_case(rng, m, k, n, gs, offset is not None)
    if offset == "frac":
        of = (rng.standard_normal((k // gs, n)) * 3).astype(np.float16)
    w_gpu = ops.pack_weight_w4(to_dev(wp), k, n)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.matmul_w4a16_packed(y, to_dev(x), w_gpu, to_dev(sc), None if of is None else to_dev(of), gs)
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=gs, has_offset=int(of is not None))
    w4_check(y.cpu().numpy(), orc.matmul_w4a16(d, x, wp, sc, of), x)


def test_w4a16_packed_multi_pass_and_repeatable():
    """k too long for one pass of staged activations (several passes per wavefront), and two calls give identical bits."""
    m, k, n, gs = 4, 24576, 256, 128
    announce("w4a16 packed long k", m, k, n)
    rng = np.random.default_rng(5)
    x, wp, sc, of = w4_case(rng, m, k, n, gs, True)
    w_gpu = ops.pack_weight_w4(to_dev(wp), k, n)
    xs, scs, ofs = to_dev(x), to_dev(sc), to_dev(of)
    y1 = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    y2 = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.matmul_w4a16_packed(y1, xs, w_gpu, scs, ofs, gs)
    ops.matmul_w4a16_packed(y2, xs, w_gpu, scs, ofs, gs)
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=gs, has_offset=1)
    w4_check(y1.cpu().numpy(), orc.matmul_w4a16(d, x, wp, sc, of), x)
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("m,k,n,gs", [(7, 3200, 144, 64), (16, 5248, 48, 128), (12, 1024, 2320, 1024),
                                      (8, 8192, 64, 32)])
def test_w4a16_packed_more_than_four_rows(m, k, n, gs):
    """5 to 16 rows on packed weights: one wavefront per slab over all of k, activations shared chunk by chunk.  k of
    several chunks with a short last one, a last workgroup with idle wavefronts, one group per chunk; the last case has
    more quantisation groups than that kernel stages and runs the kernel of the few-row case in several passes.  Two
    calls give identical bits."""
    announce("w4a16 packed rows", m, k, n, gs)
    rng = np.random.default_rng(m * 131 + k + n)
    x, wp, sc, of = w4_case(rng, m, k, n, gs, True)
    w_gpu = ops.pack_weight_w4(to_dev(wp), k, n)
    xs, scs, ofs = to_dev(x), to_dev(sc), to_dev(of)
    y1 = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    y2 = torch.full((m, n), 7.0, dtype=torch.float16, device=DEV)
    ops.matmul_w4a16_packed(y1, xs, w_gpu, scs, ofs, gs)
    ops.matmul_w4a16_packed(y2, xs, w_gpu, scs, ofs, gs)
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=gs, has_offset=1)
    w4_check(y1.cpu().numpy(), orc.matmul_w4a16(d, x, wp, sc, of), x)
    assert torch.equal(y1, y2)


def config4_columns(m, n):
    """The oracle covers every column at M=1 (about 6 s on 16 threads); for more rows three slabs: the first and the last
    512 columns (the kernels' first and last column blocks) and one from the middle."""
    return [(0, n)] if m == 1 else [(0, 512), (n // 2 - 256, n // 2 + 256), (n - 512, n)]


def config4_check(got, x, wp, sc, of, d, cols):
    orc.set_threads(16)
    for c0, c1 in cols:
        want = orc.matmul_w4a16(d, x, wp, sc, of, cols=(c0, c1))[:, c0:c1]
        g = got[:, c0:c1]
        err = np.abs(g.astype(np.float64) - want.astype(np.float64))
        tol = 1e-3 * np.maximum(np.abs(want.astype(np.float64)), 1.0)          # fp32 epilogue rel-err <= 1e-3
        assert np.all(err <= tol + 2e-3)
        assert np.mean(g.view(np.uint16) == want.view(np.uint16)) > 0.99


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("m", [1, 4, 16])
def test_config4_w4a16_decode(m, packed):
    """fp16 [M,8192] x int4 [8192,28672], group 128, fp16 scale and offset; both weight layouts."""
    announce("config 4", m, "packed" if packed else "nd")
    rng = np.random.default_rng(0xC4 + m)
    k, n, gs = 8192, 28672, 128
    x, wp, sc, of = w4_case(rng, m, k, n, gs, True)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    if packed:
        ops.matmul_w4a16_packed(y, to_dev(x), ops.pack_weight_w4(to_dev(wp), k, n), to_dev(sc), to_dev(of), gs)
    else:
        ops.matmul_w4a16(y, to_dev(x), to_dev(wp), to_dev(sc), to_dev(of), gs)
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=gs, has_offset=1)
    config4_check(y.cpu().numpy(), x, wp, sc, of, d, config4_columns(m, n))


def w4_group_sum_gate(got, want):
    """The bar of a half output whose accumulation order is free, against the oracle's per-weight arithmetic: every
    element within one bfloat16 ulp of the expected value - where the expected value is small against its row (a
    cancellation), one bfloat16 ulp of the row's root mean square - and the error of a row as a whole within 1e-3 of the
    row.  No share of bit-identical elements is asked for: the group-sum form leaves out the per-weight roundings."""
    g, w = got.astype(np.float64), want.astype(np.float64)
    rms = np.sqrt(np.mean(w * w, axis=1, keepdims=True))
    ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(w), rms) + 1e-300)) - 7)
    assert np.all(np.abs(g - w) <= ulp)
    assert np.all(np.linalg.norm(g - w, axis=1) <= 1e-3 * np.linalg.norm(w, axis=1))


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 9, 16, 17, 33])
@pytest.mark.parametrize("k,n,gs", [(512, 1024, 128), (1024, 544, 64), (384, 512, 128), (2048, 272, 256), (2048, 64, 512),
                                     (128, 4112, 128), (3200, 144, 128)])
@pytest.mark.parametrize("offset", ["int", "frac", None])
def test_w4a16_packed_group_sum_small(m, k, n, gs, offset):
    """ASCQ_W4A16_GROUP_SUM: scale and offset applied once per quantisation group to fp32 sums.  Same oracle (the
    per-weight arithmetic), the tolerance of a half output; a group size that is no multiple of 128 runs the per-weight
    form and must pass the same gate.  Two calls give identical bits."""
    announce("w4a16 packed group sum", m, k, n, gs, offset)
    rng = np.random.default_rng(m * 7 + k + n)
    x, wp, sc, of = w4_case(rng, m, k, n, gs, offset is not None)
    if offset == "frac":
        of = (rng.standard_normal((k // gs, n)) * 3).astype(np.float16)
    w_gpu = ops.pack_weight_w4(to_dev(wp), k, n)
    xs, scs, ofs = to_dev(x), to_dev(sc), None if of is None else to_dev(of)
    y1 = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    y2 = torch.full((m, n), 7.0, dtype=torch.float16, device=DEV)
    ops.matmul_w4a16_packed(y1, xs, w_gpu, scs, ofs, gs, mode=abi.W4A16_GROUP_SUM)
    ops.matmul_w4a16_packed(y2, xs, w_gpu, scs, ofs, gs, mode=abi.W4A16_GROUP_SUM)
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=gs, has_offset=int(of is not None))
    w4_group_sum_gate(y1.cpu().numpy(), orc.matmul_w4a16(d, x, wp, sc, of))
    assert torch.equal(y1, y2)


def test_w4a16_packed_group_sum_is_the_real_number_value():
    """What the group-sum form computes, pinned without the oracle: on inputs whose products and sums are exact in
    fp32 (integer activations, power-of-two scales, integer offsets) it must give the exact value of
    sum_g scale_g (sum_k x_k w_k + offset_g sum_k x_k), computed here in Python integers."""
    m, k, n, gs = 3, 1024, 96, 128
    announce("w4a16 packed group sum exact", m, k, n)
    rng = np.random.default_rng(77)
    x = rng.integers(-4, 5, (m, k)).astype(np.float16)
    w = rng.integers(-8, 8, (k, n)).astype(np.int8)
    sc = (2.0 ** rng.integers(-6, -2, (k // gs, n))).astype(np.float16)
    of = rng.integers(-8, 8, (k // gs, n)).astype(np.float16)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.matmul_w4a16_packed(y, to_dev(x), ops.pack_weight_w4(to_dev(pack_int4(w)), k, n), to_dev(sc), to_dev(of), gs,
                            mode=abi.W4A16_GROUP_SUM)
    xg = x.astype(np.int64).reshape(m, k // gs, gs)
    wg = w.astype(np.int64).reshape(k // gs, gs, n)
    dots = np.einsum("mgk,gkn->mgn", xg, wg) + xg.sum(axis=2)[:, :, None] * of.astype(np.int64)[None]
    want = (dots.astype(np.float64) * sc.astype(np.float64)[None]).sum(axis=1)      # exact: multiples of 2^-6 below 2^24
    assert np.array_equal(y.cpu().numpy(), want.astype(np.float16))


@pytest.mark.parametrize("offset", ["int", "frac"])
@pytest.mark.parametrize("m", [1, 4, 16])
def test_config4_w4a16_decode_group_sum(m, offset):
    """Config 4 in the group-sum form: every column at M=1, three slabs of 512 columns at M=4 / 16, integer and
    fractional offsets, against the unchanged oracle."""
    announce("config 4 group sum", m, offset)
    rng = np.random.default_rng(0xC4 + m)
    k, n, gs = 8192, 28672, 128
    x, wp, sc, of = w4_case(rng, m, k, n, gs, True)
    if offset == "frac":
        of = (rng.standard_normal((k // gs, n)) * 3).astype(np.float16)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.matmul_w4a16_packed(y, to_dev(x), ops.pack_weight_w4(to_dev(wp), k, n), to_dev(sc), to_dev(of), gs,
                            mode=abi.W4A16_GROUP_SUM)
    d = abi.W4A16Desc(m=m, n=n, k=k, group_size=gs, has_offset=1)
    got = y.cpu().numpy()
    orc.set_threads(16)
    for c0, c1 in config4_columns(m, n):
        want = orc.matmul_w4a16(d, x, wp, sc, of, cols=(c0, c1))[:, c0:c1]
        w4_group_sum_gate(got[:, c0:c1], want)


# ------------------------------------------------------------------ W8A16 (Matmul anti-quant path)
def w8a16_check(got, want, x, out_f32):
    # fp32 accumulation in a different order than the oracle's wide one: error bounded relative to sum |x| |w| (w up
    # to 137 * 1e-2 in these cases), and bit-identical halves nearly everywhere
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ref = np.abs(x.astype(np.float64)).sum(axis=1, keepdims=True) * 1.4
    assert np.all(err <= 1e-5 * ref + 1e-6) if out_f32 else np.all(err <= 1e-3 * ref + 1e-6)
    if not out_f32:
        assert np.mean(got.view(np.uint16) == want.view(np.uint16)) > 0.9


@pytest.mark.parametrize("m", [1, 3, 16, 17, 32, 33, 40, 70, 97, 300])   # above 96 rows: transposed copy + tile GEMM
@pytest.mark.parametrize("k,n", [(256, 256), (512, 1040), (96, 48), (100, 30), (2048, 512), (192, 30)])
@pytest.mark.parametrize("mode", ["vector+offset", "vector", "scalar+offset", "scalar", "vector+intoffset"])
def test_w8a16_small(m, k, n, mode):
    announce("w8a16", m, k, n, mode)
    rng = np.random.default_rng(m * 7 + k + n)
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = rng.integers(-128, 128, (k, n)).astype(np.int8)
    per_tensor = mode.startswith("scalar")
    has_offset = "offset" in mode
    out_f32 = (m + k) % 2 == 1
    if per_tensor:
        sc, of = 0.0077, (2.5 if has_offset else None)
    else:
        sc = rng.uniform(1e-3, 1e-2, n).astype(np.float16)
        of = None
        if has_offset:
            of = (rng.integers(-9, 10, n) if "int" in mode else rng.uniform(-9, 9, n)).astype(np.float16)
    y = torch.zeros((m, n), dtype=torch.float32 if out_f32 else torch.float16, device=DEV)
    ops.matmul_w8a16(y, to_dev(x), to_dev(w), of if per_tensor else (None if of is None else to_dev(of)),
                     sc if per_tensor else to_dev(sc))
    d = abi.W8A16Desc(m=m, n=n, k=k, per_tensor=int(per_tensor), has_offset=int(has_offset),
                      scale=sc if per_tensor else 0.0, offset=of if per_tensor and has_offset else 0.0,
                      out_dtype=abi.F32 if out_f32 else abi.F16)
    want = orc.matmul_w8a16(d, x, w, None if per_tensor else of, None if per_tensor else sc)
    w8a16_check(y.cpu().numpy(), want, x, out_f32)


@pytest.mark.parametrize("m", [1, 16])
def test_w8a16_decode_shape(m):
    """fp16 [M,4096] x int8 [4096,11008], per-channel scale and offset (the W8A8 headline weight shape)."""
    announce("w8a16 decode", m)
    rng = np.random.default_rng(0xA16 + m)
    k, n = 4096, 11008
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = rng.integers(-128, 128, (k, n)).astype(np.int8)
    sc = rng.uniform(1e-3, 1e-2, n).astype(np.float16)
    of = rng.uniform(-9, 9, n).astype(np.float16)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.matmul_w8a16(y, to_dev(x), to_dev(w), to_dev(of), to_dev(sc))
    d = abi.W8A16Desc(m=m, n=n, k=k, per_tensor=0, has_offset=1, out_dtype=abi.F16)
    orc.set_threads(16)
    want = orc.matmul_w8a16(d, x, w, of, sc)
    w8a16_check(y.cpu().numpy(), want, x, False)


@pytest.mark.parametrize("m", [1, 4])
@pytest.mark.parametrize("mode", [abi.W8A16_PER_WEIGHT, abi.W8A16_CHANNEL_SUM])
def test_w8a16_decode_shape_weights_as_n_k(m, mode):
    """fp16 [M, 8192] x int8 [28672, 8192] kept as [n, k] (the benchmark's decode shape), per-channel scale and offset,
    on the stream kernel with the activations resident in LDS: the per-weight mode within the usual tolerance of a free
    accumulation order, the channel-sum mode within one bfloat16 ulp per element and 1e-3 per row."""
    announce("w8a16 decode [n, k]", m, mode)
    rng = np.random.default_rng(0xB16 + m)
    k, n = 8192, 28672
    x = rng.standard_normal((m, k)).astype(np.float16)
    wt = rng.integers(-128, 128, (n, k)).astype(np.int8)
    sc = rng.uniform(1e-3, 1e-2, n).astype(np.float16)
    of = rng.uniform(-9, 9, n).astype(np.float16)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.matmul_w8a16(y, to_dev(x), to_dev(wt), to_dev(of), to_dev(sc), workspace=torch.empty(4, device=DEV), trans_b=True,
                     mode=mode)
    d = abi.W8A16Desc(m=m, n=n, k=k, per_tensor=0, has_offset=1, out_dtype=abi.F16, trans_b=1)
    orc.set_threads(16)
    want = orc.matmul_w8a16(d, x, wt, of, sc)
    if mode == abi.W8A16_PER_WEIGHT:
        w8a16_check(y.cpu().numpy(), want, x, False)
    else:
        w4_group_sum_gate(y.cpu().numpy(), np.asarray(want))


@pytest.mark.parametrize("m", [2, 16])
def test_w8a16_exact_integers_full_size(m):
    """Small integer activations, power-of-two scales and integer offsets make every product and partial sum exact in
    fp32, so the result is independent of the accumulation order: bit-equal to plain integer arithmetic at full size."""
    announce("w8a16 exact", m)
    rng = np.random.default_rng(0xE8 + m)
    k, n = 4096, 11008
    xi = rng.integers(-2, 3, (m, k))
    w = rng.integers(-128, 128, (k, n)).astype(np.int8)
    sc = rng.choice([0.25, 0.5, 1.0], n)
    of = rng.integers(-9, 10, n)
    y = torch.zeros((m, n), dtype=torch.float32, device=DEV)
    ops.matmul_w8a16(y, to_dev(xi.astype(np.float16)), to_dev(w), to_dev(of.astype(np.float16)),
                     to_dev(sc.astype(np.float16)))
    want = (xi.astype(np.float64) @ (w.astype(np.float64) + of[None, :])) * sc[None, :]
    assert np.array_equal(y.cpu().numpy().astype(np.float64), want)

@pytest.mark.parametrize("m", [1, 3, 16, 17, 40, 49, 130, 300])
@pytest.mark.parametrize("k,n", [(128, 16), (256, 256), (512, 1040), (384, 30), (2048, 520), (8192, 144), (192, 40),
                                 (77, 23)])
@pytest.mark.parametrize("mode", ["vector+offset", "vector", "scalar+offset", "scalar"])
def test_w8a16_trans_b(m, k, n, mode):
    """B given as [n, k] (isTransposeB): one launch, no workspace; the whole-column kernel up to 48 rows, the
    de-quantising tile GEMM above, one lane per output element when k is no multiple of 128.  Against the oracle on
    the same transposed weights, and bit-equal between two calls (the summation order is fixed)."""
    announce("w8a16 [n, k]", m, k, n, mode)
    rng = np.random.default_rng(m * 5 + k + n)
    x = rng.standard_normal((m, k)).astype(np.float16)
    wt = rng.integers(-128, 128, (n, k)).astype(np.int8)
    per_tensor = mode.startswith("scalar")
    has_offset = "offset" in mode
    out_f32 = (m + k // 128) % 2 == 1
    if per_tensor:
        sc, of = 0.0077, (2.5 if has_offset else None)
    else:
        sc = rng.uniform(1e-3, 1e-2, n).astype(np.float16)
        of = rng.uniform(-9, 9, n).astype(np.float16) if has_offset else None
    ys = []
    for _ in range(2):
        y = torch.zeros((m, n), dtype=torch.float32 if out_f32 else torch.float16, device=DEV)
        y.view(torch.int16).fill_(0x7E7E)
        ops.matmul_w8a16(y, to_dev(x), to_dev(wt), of if per_tensor else (None if of is None else to_dev(of)),
                         sc if per_tensor else to_dev(sc), workspace=torch.empty(4, device=DEV), trans_b=True)
        ys.append(y.cpu().numpy())
    assert np.array_equal(ys[0].view(np.uint16), ys[1].view(np.uint16))
    d = abi.W8A16Desc(m=m, n=n, k=k, per_tensor=int(per_tensor), has_offset=int(has_offset),
                      scale=sc if per_tensor else 0.0, offset=of if per_tensor and has_offset else 0.0,
                      out_dtype=abi.F32 if out_f32 else abi.F16, trans_b=1)
    want = orc.matmul_w8a16(d, x, wt, None if per_tensor else of, None if per_tensor else sc)
    w8a16_check(ys[0], want, x, out_f32)
    # the oracle's own transposed indexing: the same answer from the [k, n] form
    d.trans_b = 0
    assert np.array_equal(np.asarray(want).view(np.uint8),
                          np.asarray(orc.matmul_w8a16(d, x, np.ascontiguousarray(wt.T), None if per_tensor else of,
                                                      None if per_tensor else sc)).view(np.uint8))


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("k,n", [(128, 16), (256, 256), (512, 1040), (384, 30), (2048, 520), (8192, 144)])
@pytest.mark.parametrize("mode", ["vector+offset", "vector", "scalar+offset", "scalar"])
def test_w8a16_trans_b_channel_sum(m, k, n, mode):
    """ASCQ_W8A16_CHANNEL_SUM on [n, k] weights: scale and offset applied once per output to fp32 sums.  Same oracle
    (the per-weight arithmetic), the tolerance of a half output: every element within one bfloat16 ulp, the row error
    within 1e-3; 5 rows run the per-weight kernel and pass the same gate.  Two calls give identical bits."""
    announce("w8a16 [n, k] channel sum", m, k, n, mode)
    rng = np.random.default_rng(m * 11 + k + n)
    x = rng.standard_normal((m, k)).astype(np.float16)
    wt = rng.integers(-128, 128, (n, k)).astype(np.int8)
    per_tensor = mode.startswith("scalar")
    has_offset = "offset" in mode
    if per_tensor:
        sc, of = 0.0077, (2.5 if has_offset else None)
    else:
        sc = rng.uniform(1e-3, 1e-2, n).astype(np.float16)
        of = rng.uniform(-9, 9, n).astype(np.float16) if has_offset else None
    ys = []
    for _ in range(2):
        y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
        y.view(torch.int16).fill_(0x7E7E)
        ops.matmul_w8a16(y, to_dev(x), to_dev(wt), of if per_tensor else (None if of is None else to_dev(of)),
                         sc if per_tensor else to_dev(sc), workspace=torch.empty(4, device=DEV), trans_b=True,
                         mode=abi.W8A16_CHANNEL_SUM)
        ys.append(y.cpu().numpy())
    assert np.array_equal(ys[0].view(np.uint16), ys[1].view(np.uint16))
    d = abi.W8A16Desc(m=m, n=n, k=k, per_tensor=int(per_tensor), has_offset=int(has_offset),
                      scale=sc if per_tensor else 0.0, offset=of if per_tensor and has_offset else 0.0,
                      out_dtype=abi.F16, trans_b=1)
    want = orc.matmul_w8a16(d, x, wt, None if per_tensor else of, None if per_tensor else sc)
    w4_group_sum_gate(ys[0], np.asarray(want))


def test_w8a16_channel_sum_is_the_real_number_value():
    """The channel-sum form rounds the exact value of the quantised product once; the per-weight form carries two
    roundings per weight.  Against float64 arithmetic on the same quantised inputs the channel-sum result is at least
    as close, on average, as the per-weight one."""
    announce("w8a16 channel sum against float64")
    rng = np.random.default_rng(91)
    m, k, n = 4, 4096, 1024
    x = rng.standard_normal((m, k)).astype(np.float16)
    wt = rng.integers(-128, 128, (n, k)).astype(np.int8)
    sc = rng.uniform(1e-3, 1e-2, n).astype(np.float16)
    of = rng.uniform(-9, 9, n).astype(np.float16)
    exact = (x.astype(np.float64) @ (wt.astype(np.float64).T + of.astype(np.float64)[None, :])) * sc.astype(np.float64)[None, :]
    errs = []
    for mode in (abi.W8A16_PER_WEIGHT, abi.W8A16_CHANNEL_SUM):
        y = torch.zeros((m, n), dtype=torch.float32, device=DEV)
        ops.matmul_w8a16(y, to_dev(x), to_dev(wt), to_dev(of), to_dev(sc), workspace=torch.empty(4, device=DEV), trans_b=True,
                         mode=mode)
        errs.append(np.abs(y.cpu().numpy().astype(np.float64) - exact).mean())
    assert errs[1] <= errs[0]
    assert errs[1] <= 1e-5 * np.abs(exact).mean()


@pytest.mark.parametrize("m", [1, 16])
def test_w8a16_trans_b_exact_integers_full_size(m):
    """K=8192, N=28672 as [n, k]: small integer activations, power-of-two scales and integer offsets make every partial
    sum exact in fp32, so the result must equal plain integer arithmetic bit for bit on every column."""
    announce("w8a16 [n, k] exact", m)
    rng = np.random.default_rng(0xE9 + m)
    k, n = 8192, 28672
    xi = rng.integers(-2, 3, (m, k))
    wt = rng.integers(-128, 128, (n, k)).astype(np.int8)
    sc = rng.choice([0.25, 0.5, 1.0], n)
    of = rng.integers(-9, 10, n)
    y = torch.zeros((m, n), dtype=torch.float32, device=DEV)
    ops.matmul_w8a16(y, to_dev(xi.astype(np.float16)), to_dev(wt), to_dev(of.astype(np.float16)),
                     to_dev(sc.astype(np.float16)), trans_b=True)
    want = ((wt.astype(np.float32) + of[:, None].astype(np.float32)) @ xi.T.astype(np.float32)).T * sc[None, :]
    assert np.array_equal(y.cpu().numpy().astype(np.float64), want.astype(np.float64))


# ------------------------------------------------------------------ fractal (NZ) weights
def to_nz(w):
    """[.., k, n] -> [.., n/32, k/16, 16, 32], as the reference example packs its weights
    (quant_group_matmul_high_performance/scripts/gen_data.py:62-65)."""
    *lead, k, n = w.shape
    nd = len(lead)
    perm = list(range(nd)) + [nd + 2, nd + 0, nd + 1, nd + 3]
    return np.ascontiguousarray(w.reshape(*lead, k // 16, 16, n // 32, 32).transpose(perm))


@pytest.mark.parametrize("m,n,k", [(1, 64, 128), (48, 160, 256), (200, 544, 384), (513, 288, 128), (2048, 2848, 256)])
@pytest.mark.parametrize("out", [torch.int32, torch.bfloat16])
def test_matmul_nz_weights(m, n, k, out):
    """The same product from fractal weights: bit-equal to the oracle on the row-major weights."""
    announce("nz weights", m, n, k, out)
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    c = torch.zeros((m, n), dtype=out, device=DEV)
    mm = ops.Matmul(m, n, k)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b(to_dev(to_nz(w)), nz=True)
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.I32)
    cs = ts = None
    if out != torch.int32:
        cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
        ts = rng.uniform(1e-3, 1e-1, m).astype(np.float32)
        mm.set_quant_vector(to_dev(cs))
        mm.set_token_scale(to_dev(ts))
        d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                           scale_format=abi.MM_SCALE_F32, has_tok_scale=1)
    mm.iterate_all(c)
    orc.set_threads(16)
    want = orc.matmul_w8a8(d, a, w, None, cs, ts)
    assert np.array_equal(bits(c), want)


@pytest.mark.parametrize("m,kernel", [(1, abi.MM_KERNEL_STREAM), (100, abi.MM_KERNEL_DMA_128),
                                      (700, abi.MM_KERNEL_DMA_256)])
def test_matmul_plan_then_call(m, kernel):
    """The plan query names the kernel family and launches nothing; the call that follows is unaffected."""
    announce("plan", m)
    rng = np.random.default_rng(m)
    n, k = 544, 384
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    c = torch.full((m, n), -7, dtype=torch.int32, device=DEV)
    mm = ops.Matmul(m, n, k)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b(to_dev(w))
    plan = mm.plan(c)
    torch.cuda.synchronize()
    assert plan.kernel == kernel and plan.launches >= 1 and plan.workgroups >= 1
    assert bool((c == -7).all())                      # nothing ran
    mm.iterate_all(c)
    assert np.array_equal(c.cpu().numpy(), a.astype(np.int32) @ w.astype(np.int32))


@pytest.mark.parametrize("g,k,n", [(1, 16, 32), (1, 128, 160), (3, 208, 544), (2, 4096, 1024), (1, 80, 11008)])
def test_pack_weight_nz(g, k, n):
    """The device-side packer against the reference script's reshape / transpose, and its error paths."""
    announce("pack nz", g, k, n)
    rng = np.random.default_rng(g + k + n)
    w = rng.integers(-128, 128, (g, k, n)).astype(np.int8)
    got = ops.pack_weight_nz(to_dev(w)).cpu().numpy()
    assert np.array_equal(got, to_nz(w))
    if g == 1:
        got2 = ops.pack_weight_nz(to_dev(w[0])).cpu().numpy()
        assert got2.shape == (n // 32, k // 16, 16, 32) and np.array_equal(got2, to_nz(w[0]))


def test_pack_weight_nz_feeds_the_matmul():
    """ND weights packed on the device give the product of the ND weights, bit for bit."""
    announce("pack nz + matmul")
    rng = np.random.default_rng(0x4E5A)
    m, n, k = 300, 544, 384
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    c = torch.zeros((m, n), dtype=torch.int32, device=DEV)
    mm = ops.Matmul(m, n, k)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b(ops.pack_weight_nz(to_dev(w)), nz=True)
    mm.iterate_all(c)
    assert np.array_equal(c.cpu().numpy(), a.astype(np.int32) @ w.astype(np.int32))


def test_pack_weight_nz_rejects():
    announce("pack nz rejects")
    w = torch.zeros((24, 32), dtype=torch.int8, device=DEV)
    with pytest.raises(ops.AscqError, match="k % 16"):
        ops.pack_weight_nz(w)
    w = torch.zeros((16, 48), dtype=torch.int8, device=DEV)
    with pytest.raises(ops.AscqError, match="n % 32"):
        ops.pack_weight_nz(w)
    w = torch.zeros((16, 32), dtype=torch.int8, device=DEV)
    with pytest.raises(ops.AscqError, match="same buffer"):
        ops.pack_weight_nz(w, out=w)


def test_group_matmul_nz_weights_as_the_reference_example_packs_them():
    """The example's configuration in small: counts group list, fractal weights, FasterGelu, fp16 out."""
    announce("group nz")
    rng = np.random.default_rng(0x6E7A)
    groups, k, n = 4, 256, 320
    counts = [100, 0, 257, 31]
    m = sum(counts)
    x = rng.integers(-10, 10, (m, k)).astype(np.int8)
    w = rng.integers(-10, 10, (groups, k, n)).astype(np.int8)
    sc = rng.normal(0, 0.01, (groups, n)).astype(np.float32)
    ts = rng.normal(0, 0.01, m).astype(np.float32)
    y = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    gl = torch.tensor(counts, dtype=torch.int64, device=DEV)
    ops.quant_group_matmul(y, to_dev(x), to_dev(to_nz(w)), gl, to_dev(sc), to_dev(ts),
                           activation=abi.MM_ACT_FASTER_GELU, weight_nz=True)
    mmd = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.F16, quant_mode=abi.MM_QUANT_VECTOR,
                         scale_format=abi.MM_SCALE_F32, has_tok_scale=1, activation=abi.MM_ACT_FASTER_GELU)
    gd = abi.GroupMatmulDesc(mm=mmd, groups=groups, group_list_kind=abi.GROUP_LIST_COUNTS)
    want = orc.group_matmul_w8a8(gd, x, w, None, sc, ts, np.array(counts, dtype=np.int64))
    got = bits(y)
    assert max_ulp(got, want.view(np.uint16), "f16") <= 1


def test_group_matmul_example_full_size_nz_equals_nd():
    """The reference example's own size (8 groups x 1024 tokens, k=1024, n=8192, FasterGelu, fp16): the result from
    the fractal weights is bit-equal to the one from row-major weights (which the other tests tie to the oracle), and
    a sample of rows is checked against the example's golden formula in float64."""
    announce("group example full size")
    rng = np.random.default_rng(0xE8A)
    groups, m, k, n = 8, 8192, 1024, 8192
    counts = [1024] * groups
    x = rng.integers(-10, 10, (m, k)).astype(np.int8)
    w = rng.integers(-10, 10, (groups, k, n)).astype(np.int8)
    sc = rng.normal(0, 0.01, (groups, n)).astype(np.float32)
    ts = rng.normal(0, 0.01, m).astype(np.float32)
    gl = torch.tensor(counts, dtype=torch.int64, device=DEV)
    xd, scd, tsd = to_dev(x), to_dev(sc), to_dev(ts)
    y_nd = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    y_nz = torch.zeros((m, n), dtype=torch.float16, device=DEV)
    ops.quant_group_matmul(y_nd, xd, to_dev(w), gl, scd, tsd, activation=abi.MM_ACT_FASTER_GELU)
    ops.quant_group_matmul(y_nz, xd, to_dev(to_nz(w)), gl, scd, tsd, activation=abi.MM_ACT_FASTER_GELU, weight_nz=True)
    assert torch.equal(y_nd.view(torch.int16), y_nz.view(torch.int16))
    rows = rng.choice(m, 64, replace=False)
    got = y_nz[torch.from_numpy(rows).to(DEV)].float().cpu().numpy().astype(np.float64)
    for i, r in enumerate(rows):
        g = r // 1024
        v = (x[r].astype(np.float64) @ w[g].astype(np.float64)) * sc[g].astype(np.float64) * float(ts[r])
        gold = v / (1.0 + np.exp(-1.702 * v))                       # the example's FastGelu, in closed form
        assert np.all(np.abs(got[i] - gold) <= 2e-3 * np.abs(gold) + 1e-6)

# ------------------------------------------------------------------ SwiGLU epilogue
def swiglu_close(got_bits, want_bits, fmt):
    # expf of the device library against libm: the activation may differ by an ulp of the output type
    assert max_ulp(got_bits, want_bits, fmt) <= 1
    assert np.mean(got_bits == want_bits) > 0.98


@pytest.mark.parametrize("m,n,k", [(1, 64, 128), (16, 1040, 2048), (33, 144, 128), (200, 528, 384), (600, 528, 640),
                                   (1100, 784, 384), (19, 22, 77), (2048, 2832, 384)])
@pytest.mark.parametrize("out,bias", [(torch.bfloat16, None), (torch.float16, "f32"), (torch.float32, "bf16")])
def test_matmul_swiglu_epilogue(m, n, k, out, bias):
    """Columns 2j / 2j + 1 -> output column j; every kernel family (weight streams, K-split tiles, large tiles with the
    in-register form, generic) against the oracle."""
    announce("swiglu", m, n, k, out, bias)
    rng = np.random.default_rng(m * 3 + n + k)
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    cs = rng.uniform(1e-4, 4e-4, n).astype(np.float32)
    ts = rng.uniform(0.5, 2.0, m).astype(np.float32)
    bv = None
    if bias == "f32":
        bv = (rng.standard_normal(n).astype(np.float32), None)
    elif bias == "bf16":
        bv = (orc.f32_to_bf16_bits(rng.standard_normal(n).astype(np.float32)), "bf16")
    mm = ops.Matmul(m, n, k)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b(to_dev(b))
    mm.set_quant_vector(to_dev(cs))
    mm.set_token_scale(to_dev(ts))
    if bv is not None:
        mm.set_bias(to_dev(bv[0], bv[1]))
    mm.set_activation(abi.MM_ACT_SWIGLU, 1.0 if m % 2 else 1.702)
    c = torch.zeros((m, n // 2), dtype=out, device=DEV)
    mm.iterate_all(c)
    want = oracle_mm(mm.desc, a, b, bv, cs, ts)
    if out == torch.float32:
        got = c.cpu().numpy()
        assert np.all(np.abs(got - want) <= 4 * np.spacing(np.abs(want)) + 1e-30)
    else:
        fmt = "bf16" if out == torch.bfloat16 else "f16"
        swiglu_close(bits(c), want.view(np.uint16), fmt)


def test_group_matmul_swiglu_and_dynamic_linear():
    """The grouped matmul (MoE gate / up projection with interleaved columns) and the fused quantise + linear call."""
    announce("group swiglu")
    rng = np.random.default_rng(0x51)
    groups, m, k, n = 4, 700, 256, 544
    counts = np.array([300, 0, 1, 399], dtype=np.int64)
    x, w = rand_i8(rng, (m, k)), rand_i8(rng, (groups, k, n))
    sc = rng.uniform(1e-4, 4e-4, (groups, n)).astype(np.float32)
    ts = rng.uniform(0.5, 2.0, m).astype(np.float32)
    y = torch.zeros((m, n // 2), dtype=torch.bfloat16, device=DEV)
    ops.quant_group_matmul(y, to_dev(x), to_dev(w), to_dev(counts), to_dev(sc), to_dev(ts),
                           activation=abi.MM_ACT_SWIGLU, act_beta=1.0)
    mmd = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                         has_tok_scale=1, activation=abi.MM_ACT_SWIGLU, act_beta=1.0)
    gd = abi.GroupMatmulDesc(mm=mmd, groups=groups, group_list_kind=abi.GROUP_LIST_COUNTS)
    want = orc.group_matmul_w8a8(gd, x, w, None, sc, ts, counts)
    swiglu_close(bits(y), want.view(np.uint16), "bf16")
    # dynamic quantisation + linear + SwiGLU in one call, decode and prefill sizes
    for mm_rows in (3, 640):
        xa = orc.f32_to_bf16_bits(rng.standard_normal((mm_rows, k)).astype(np.float32))
        wl = rand_i8(rng, (k, n))
        cs = rng.uniform(1e-4, 4e-4, n).astype(np.float32)
        c = torch.zeros((mm_rows, n // 2), dtype=torch.bfloat16, device=DEV)
        ops.linear_w8a8_dynamic(c, to_dev(xa, "bf16"), to_dev(wl), to_dev(cs), activation=abi.MM_ACT_SWIGLU)
        q, tsn = orc.dynamic_quant_per_token(abi.BF16, xa)
        d = abi.MatmulDesc(m=mm_rows, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                           scale_format=abi.MM_SCALE_F32, has_tok_scale=1, activation=abi.MM_ACT_SWIGLU, act_beta=1.0)
        swiglu_close(bits(c), orc.matmul_w8a8(d, q, wl, None, cs, tsn).view(np.uint16), "bf16")


@pytest.mark.parametrize("m", [1, 5, 16, 17, 64, 130, 300])
@pytest.mark.parametrize("n,k", [(22, 128), (1040, 2048), (528, 384), (96, 4096), (64, 8192), (48, 11008)])
@pytest.mark.parametrize("out,bias", [(torch.bfloat16, None), (torch.float16, "f32"), (torch.float32, "bf16")])
def test_matmul_swiglu_in_the_decode_kernels(m, n, k, out, bias):
    """SwiGLU on [n, k] and on packed weights: the decode kernels (activations resident in LDS up to 16 rows, weights
    held in registers beyond, also in chunks of a longer k) pair the columns of a row through neighbouring lanes in
    their own epilogue - one launch, no raw accumulators; [n, k] weights past 224 rows (64 or 48 at k above 4096) take the
    tile kernels.  Against the oracle."""
    announce("swiglu decode", m, n, k, out, bias)
    rng = np.random.default_rng(m * 5 + n + k)
    a, b = rand_i8(rng, (m, k)), rand_i8(rng, (k, n))
    cs = rng.uniform(1e-4, 4e-4, n).astype(np.float32)
    ts = rng.uniform(0.5, 2.0, m).astype(np.float32)
    bv = None
    if bias == "f32":
        bv = (rng.standard_normal(n).astype(np.float32), None)
    elif bias == "bf16":
        bv = (orc.f32_to_bf16_bits(rng.standard_normal(n).astype(np.float32)), "bf16")
    beta = 1.0 if m % 2 else 1.702
    want = None
    for packed in (False, True):
        mm = ops.Matmul(m, n, k, False, not packed)
        mm.set_tensor_a(to_dev(a))
        if packed:
            mm.set_tensor_b_packed(ops.pack_weight_w8(to_dev(b), k, n))
        else:
            mm.set_tensor_b(to_dev(np.ascontiguousarray(b.T)))
        mm.set_quant_vector(to_dev(cs))
        mm.set_token_scale(to_dev(ts))
        if bv is not None:
            mm.set_bias(to_dev(bv[0], bv[1]))
        mm.set_activation(abi.MM_ACT_SWIGLU, beta)
        c = torch.zeros((m, n // 2), dtype=out, device=DEV)
        mm.iterate_all(c)
        if want is None:
            d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=mm.desc.out_dtype, quant_mode=abi.MM_QUANT_VECTOR,
                               scale_format=abi.MM_SCALE_F32, has_tok_scale=1, bias_kind=mm.desc.bias_kind,
                               activation=abi.MM_ACT_SWIGLU, act_beta=beta)
            want = oracle_mm(d, a, b, bv, cs, ts)
        if out == torch.float32:
            assert np.all(np.abs(c.cpu().numpy() - want) <= 4 * np.spacing(np.abs(want)) + 1e-30)
        else:
            swiglu_close(bits(c), want.view(np.uint16), "bf16" if out == torch.bfloat16 else "f16")


@pytest.mark.parametrize("m", [1, 3, 8, 12, 40])
def test_linear_dynamic_swiglu_in_one_launch(m):
    """The gate / up projection of a decode step in one call: per-token quantisation, int8 matmul on [n, k] or packed
    weights, SwiGLU of the column pairs (up to 8 rows inside one kernel).  Against the oracle of the steps."""
    announce("linear dynamic swiglu", m)
    rng = np.random.default_rng(0x5E + m)
    k, n = 512, 736
    xa = orc.f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    w = rand_i8(rng, (k, n))
    cs = rng.uniform(1e-4, 4e-4, n).astype(np.float32)
    q, tsn = orc.dynamic_quant_per_token(abi.BF16, xa)
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                       has_tok_scale=1, activation=abi.MM_ACT_SWIGLU, act_beta=1.0)
    want = orc.matmul_w8a8(d, q, w, None, cs, tsn).view(np.uint16)
    c = torch.zeros((m, n // 2), dtype=torch.bfloat16, device=DEV)
    ops.linear_w8a8_dynamic(c, to_dev(xa, "bf16"), to_dev(np.ascontiguousarray(w.T)), to_dev(cs), trans_b=True,
                            activation=abi.MM_ACT_SWIGLU)
    swiglu_close(bits(c), want, "bf16")
    c2 = torch.zeros((m, n // 2), dtype=torch.bfloat16, device=DEV)
    ops.linear_w8a8_dynamic_packed(c2, to_dev(xa, "bf16"), ops.pack_weight_w8(to_dev(w), k, n), n, to_dev(cs),
                                   activation=abi.MM_ACT_SWIGLU)
    swiglu_close(bits(c2), want, "bf16")
    assert torch.equal(c, c2)


# ------------------------------------------------------------------ workspace contract, determinism
@pytest.mark.parametrize("m", [1, 5, 16, 19, 130])
def test_workspaces_need_no_initialisation_and_results_repeat(m):
    """The scratch of the weight-stream and split-K paths may hold anything (here: all-ones bytes = NaN / -1) and two
    calls give the same bits."""
    announce("workspace garbage", m)
    rng = np.random.default_rng(0x5C + m)
    k, n = 1024, 1056
    # W8A8 (stream kernel for m <= 32, split-K tiles above)
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    mm = ops.Matmul(m, n, k)
    mm.set_tensor_a(to_dev(a))
    mm.set_tensor_b(to_dev(w))
    mm.set_quant_vector(to_dev(cs))
    c1 = torch.zeros((m, n), dtype=torch.bfloat16, device=DEV)
    mm.iterate_all(c1)
    if mm._ws is not None:
        mm._ws.fill_(-1)
    c2 = torch.zeros((m, n), dtype=torch.bfloat16, device=DEV)
    mm.iterate_all(c2)
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32)
    want = orc.matmul_w8a8(d, a, w, None, cs, None)
    assert np.array_equal(bits(c1), want) and np.array_equal(bits(c2), want)
    # W4A16 and W8A16
    x = rng.standard_normal((m, k)).astype(np.float16)
    xw, wp, sc, of = w4_case(rng, m, k, n, 128, True)
    garbage = torch.full((1 << 22,), float("nan"), dtype=torch.float32, device=DEV)
    outs = []
    for ws in (None, garbage, garbage):
        y4 = torch.zeros((m, n), dtype=torch.float16, device=DEV)
        ops.matmul_w4a16(y4, to_dev(xw), to_dev(wp), to_dev(sc), to_dev(of), 128, workspace=ws)
        y8 = torch.zeros((m, n), dtype=torch.float16, device=DEV)
        ops.matmul_w8a16(y8, to_dev(x), to_dev(w), to_dev(of[0]), to_dev(sc[0]), workspace=ws)
        outs.append((bits(y4), bits(y8)))
        garbage.fill_(float("nan"))
    for y4, y8 in outs[1:]:
        assert np.array_equal(y4, outs[0][0]) and np.array_equal(y8, outs[0][1])
    assert not np.isnan(outs[0][0].view(np.float16)).any() and not np.isnan(outs[0][1].view(np.float16)).any()

# ------------------------------------------------------------------ fused dynamic quantisation + matmul
@pytest.mark.parametrize("m", [1, 2, 5, 8, 9, 40])
@pytest.mark.parametrize("k,n", [(256, 128), (1024, 1056), (4096, 2064), (320, 48)])
@pytest.mark.parametrize("xdt", [torch.bfloat16, torch.float16, torch.float32])
def test_linear_w8a8_dynamic_equals_quantise_then_matmul(m, k, n, xdt):
    """One call = per-token quantisation followed by the matmul, bit for bit (oracle of the two steps)."""
    announce("linear dynamic", m, k, n, xdt)
    rng = np.random.default_rng(m * 3 + k + n)
    xf = rng.standard_normal((m, k)).astype(np.float32) * rng.uniform(0.1, 30.0, (m, 1)).astype(np.float32)
    if m > 2:
        xf[1] = 0.0                                       # an all-zero row: scale 1, zeros
    x = torch.from_numpy(xf).to(DEV).to(xdt)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c = torch.zeros((m, n), dtype=torch.bfloat16, device=DEV)
    ops.linear_w8a8_dynamic(c, x, to_dev(w), to_dev(cs), to_dev(bias))
    xdt_abi = {torch.bfloat16: abi.BF16, torch.float16: abi.F16, torch.float32: abi.F32}[xdt]
    q, ts = orc.dynamic_quant_per_token(xdt_abi, bits(x))
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                       has_tok_scale=1, bias_kind=abi.MM_BIAS_F32_POST)
    want = orc.matmul_w8a8(d, q, w, bias, cs, ts)
    assert np.array_equal(bits(c), want)


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 7, 8, 9, 17])
@pytest.mark.parametrize("k,n", [(64, 16), (192, 40), (256, 128), (1024, 1056), (4096, 2064), (320, 48), (5632, 100),
                                 (8192, 100), (11008, 272), (12288, 16)])
@pytest.mark.parametrize("xdt,odt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                     (torch.bfloat16, torch.float32)])
def test_linear_w8a8_dynamic_on_n_k_weights(m, k, n, xdt, odt):
    """Weights kept as [n, k] (isTransposeB): up to 8 rows are quantised inside the weight-streaming kernel, more rows
    by the two kernels; either way the bits of quantise-then-matmul (oracle of the two steps)."""
    announce("linear dynamic [n, k]", m, k, n, xdt, odt)
    rng = np.random.default_rng(m * 7 + k + n)
    xf = rng.standard_normal((m, k)).astype(np.float32) * rng.uniform(0.1, 30.0, (m, 1)).astype(np.float32)
    if m > 2:
        xf[1] = 0.0
        xf[2, : k // 2] = 0.0                              # the row's maximum lies in the upper half of k only
    x = torch.from_numpy(xf).to(DEV).to(xdt)
    w = rng.integers(-127, 128, (n, k)).astype(np.int8)
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c = torch.zeros((m, n), dtype=odt, device=DEV)
    ops.linear_w8a8_dynamic(c, x, to_dev(w), to_dev(cs), to_dev(bias), trans_b=True)
    xdt_abi = {torch.bfloat16: abi.BF16, torch.float16: abi.F16}[xdt]
    odt_abi = {torch.bfloat16: abi.BF16, torch.float16: abi.F16, torch.float32: abi.F32}[odt]
    q, ts = orc.dynamic_quant_per_token(xdt_abi, bits(x))
    d = abi.MatmulDesc(m=m, n=n, k=k, trans_b=1, out_dtype=odt_abi, quant_mode=abi.MM_QUANT_VECTOR,
                       scale_format=abi.MM_SCALE_F32, has_tok_scale=1, bias_kind=abi.MM_BIAS_F32_POST)
    want = orc.matmul_w8a8(d, q, w, bias, cs, ts)
    assert np.array_equal(bits(c), gpu_util.as_bits(want))


@pytest.mark.parametrize("m", [1, 3, 4, 5, 8, 9, 33])
@pytest.mark.parametrize("k,n", [(64, 16), (192, 40), (1024, 1056), (4096, 2064), (11008, 272)])
@pytest.mark.parametrize("xdt,src_nk", [(torch.bfloat16, False), (torch.float16, True), (torch.float32, False)])
def test_linear_w8a8_dynamic_on_packed_weights(m, k, n, xdt, src_nk):
    """ascq_linear_w8a8_dynamic_packed: up to 8 rows of half / bfloat16 x in one launch, anything else quantiser +
    packed matmul; either way the bits of quantise-then-matmul (oracle of the two steps)."""
    announce("linear dynamic packed", m, k, n, xdt, src_nk)
    rng = np.random.default_rng(m * 11 + k + n)
    xf = rng.standard_normal((m, k)).astype(np.float32) * rng.uniform(0.1, 30.0, (m, 1)).astype(np.float32)
    if m > 2:
        xf[1] = 0.0
    x = torch.from_numpy(xf).to(DEV).to(xdt)
    w = rng.integers(-127, 128, (k, n)).astype(np.int8)
    wp = ops.pack_weight_w8(to_dev(np.ascontiguousarray(w.T)) if src_nk else to_dev(w), k, n, src_nk)
    cs = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    c = torch.zeros((m, n), dtype=torch.bfloat16, device=DEV)
    ops.linear_w8a8_dynamic_packed(c, x, wp, n, to_dev(cs), to_dev(bias))
    xdt_abi = {torch.bfloat16: abi.BF16, torch.float16: abi.F16, torch.float32: abi.F32}[xdt]
    q, ts = orc.dynamic_quant_per_token(xdt_abi, bits(x))
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                       has_tok_scale=1, bias_kind=abi.MM_BIAS_F32_POST)
    want = orc.matmul_w8a8(d, q, w, bias, cs, ts)
    assert np.array_equal(bits(c), want)


@pytest.mark.parametrize("m", [2, 9])
def test_prepared_linear_object_equals_the_function(m):
    """ops.DynamicLinear (descriptor and scratch prepared once) gives what ops.linear_w8a8_dynamic gives, on [k, n],
    [n, k] and packed weights."""
    k, n = 512, 208
    rng = np.random.default_rng(m)
    x = torch.from_numpy(rng.standard_normal((m, k)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    w = to_dev(rng.integers(-127, 128, (k, n)).astype(np.int8))
    wt = w.t().contiguous()
    cs, bias = to_dev(rng.uniform(1e-4, 1e-2, n).astype(np.float32)), to_dev(rng.standard_normal(n).astype(np.float32))
    want = ops.linear_w8a8_dynamic(torch.zeros((m, n), dtype=torch.bfloat16, device=DEV), x, w, cs, bias)
    for lin in (ops.DynamicLinear(m, k, w, cs, bias), ops.DynamicLinear(m, k, wt, cs, bias, trans_b=True),
                ops.DynamicLinear(m, k, ops.pack_weight_w8(w, k, n), cs, bias, packed_n=n)):
        for _ in range(2):
            got = lin(torch.zeros((m, n), dtype=torch.bfloat16, device=DEV), x)
            assert torch.equal(got, want)


# ------------------------------------------------------------------ Matmul<int4b_t, int4b_t, C>
def ref_pack_int4(x):
    """The packing of the reference example's script (matmul_int4/scripts/gen_data.py:32-42): byte j of a row is
    (x[2j+1] << 4) + (x[2j] & 0x0F), kept in int8."""
    return ((x[..., 1::2].astype(np.int32) << 4) + (x[..., 0::2].astype(np.int32) & 0x0F)).astype(np.int8)


def test_matmul_int4_reference_example():
    """The example at its own size and with its own data recipe: M=256, N=7680, K=128, values from
    uniform(-5, 5) cast to int8, int32 bias, int32 out (matmul_int4/scripts/gen_data.py:20-31)."""
    announce("int4 example")
    rng = np.random.default_rng(0x14)
    m, n, k = 256, 7680, 128
    x1 = rng.uniform(-5, 5, (m, k)).astype(np.int8)
    x2 = rng.uniform(-5, 5, (k, n)).astype(np.int8)
    bias = rng.uniform(-5, 5, n).astype(np.int32)
    golden = x1.astype(np.int32) @ x2.astype(np.int32) + bias
    c = torch.zeros((m, n), dtype=torch.int32, device=DEV)
    mm = ops.MatmulInt4(m, n, k)
    mm.set_tensor_a(to_dev(ref_pack_int4(x1)))
    mm.set_tensor_b(to_dev(ref_pack_int4(x2)))
    mm.set_bias(to_dev(bias))
    mm.iterate_all(c)
    assert np.array_equal(c.cpu().numpy(), golden)


@pytest.mark.parametrize("m,n,k,trans_b", [(1, 64, 128, False), (33, 160, 96, False), (200, 544, 384, True),
                                           (513, 34, 130, False), (70, 33, 64, True)])
@pytest.mark.parametrize("out", [torch.int32, torch.float16])
def test_matmul_int4_full_range(m, n, k, trans_b, out):
    """Every nibble value, both B orientations, int32 and the half output the reference allows (through the
    fixpipe scale words), bit-equal to the int8 oracle on the widened operands."""
    announce("int4", m, n, k, trans_b, out)
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-8, 8, (m, k)).astype(np.int8)
    b = rng.integers(-8, 8, (n, k) if trans_b else (k, n)).astype(np.int8)
    c = torch.zeros((m, n), dtype=out, device=DEV)
    mm = ops.MatmulInt4(m, n, k, trans_b=trans_b)
    mm.set_tensor_a(to_dev(pack_int4(a)))
    mm.set_tensor_b(to_dev(pack_int4(b)))
    d = abi.MatmulDesc(m=m, n=n, k=k, trans_b=int(trans_b), out_dtype=abi.I32)
    qv = None
    if out != torch.int32:
        qv = np.array([ops.pack_quant_param(s) for s in rng.uniform(1e-3, 1e-1, n)], dtype=np.uint64)
        mm.set_quant_vector(to_dev(qv.view(np.int64)))
        d = abi.MatmulDesc(m=m, n=n, k=k, trans_b=int(trans_b), out_dtype=abi.F16, quant_mode=abi.MM_QUANT_VECTOR,
                           scale_format=abi.MM_SCALE_U64)
    mm.iterate_all(c)
    want = orc.matmul_w8a8(d, a, b, None, qv, None)
    assert np.array_equal(bits(c), want if out == torch.int32 else want.view(np.uint16))


@pytest.mark.parametrize("count", [2, 30, 32, 4096 + 34, 1 << 20])
def test_unpack_int4(count):
    announce("unpack int4", count)
    rng = np.random.default_rng(count)
    v = rng.integers(-8, 8, count).astype(np.int8)
    got = ops.unpack_int4(to_dev(pack_int4(v))).cpu().numpy()
    assert got.dtype == np.int8 and np.array_equal(got, v)
    assert np.array_equal(ops.unpack_int4(to_dev(ref_pack_int4(v))).cpu().numpy(), v)


def test_matmul_int4_rejects():
    announce("int4 rejects")
    z = torch.zeros(64, dtype=torch.int8, device=DEV)
    c = torch.zeros((4, 4), dtype=torch.int32, device=DEV)
    for kw, msg in [(dict(m=4, n=4, k=3), "k 3 must be even"), (dict(m=4, n=3, k=4), "n 3 must be even"),
                    (dict(m=4, n=4, k=4, trans_a=True), "cannot be transposed")]:
        mm = ops.MatmulInt4(**kw)
        mm.set_tensor_a(z)
        mm.set_tensor_b(z)
        with pytest.raises(ops.AscqError, match=msg):
            mm.iterate_all(c)
