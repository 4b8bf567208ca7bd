"""Block-scaled (MX) matmul through the C ABI against the oracle's float64 golden."""
import ctypes as C

import numpy as np
import pytest
import torch

import orc
from ascq import _abi as abi
from ascq import ops
from gpu_util import DEV, announce, to_dev
from test_oracle_ops import mx_random_operand, mx_values

pytestmark = pytest.mark.gpu

E4, E5, F2, F1 = abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2, abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2
NP_OUT = {torch.float32: np.float32, torch.bfloat16: np.int16, torch.float16: np.float16}


def mx_case(rng, m, n, k, fa, fb, sk=None, bias=False, lo=118, hi=137):
    sk = sk or -(-((k + 31) // 32) // 2) * 2          # the reference rounds ceil(k / 32) up to an even number
    a, b = mx_random_operand(rng, m, k, fa), mx_random_operand(rng, n, k, fb)
    sa, sb = rng.integers(lo, hi, (m, sk)).astype(np.uint8), rng.integers(lo, hi, (n, sk)).astype(np.uint8)
    bv = rng.integers(-10, 10, n).astype(np.float32) if bias else None
    return a, b, sa, sb, bv


def run_mx(m, n, k, a, b, sa, sb, fa, fb, out=torch.float32, bias=None):
    c = torch.zeros((m, n), dtype=out, device=DEV)
    ops.matmul_mx(c, to_dev(a), to_dev(b), to_dev(sa), to_dev(sb), fa, fb, k, None if bias is None else to_dev(bias))
    return c


def mx_abs_dot(a, b, sa, sb, k, fa, fb):
    """sum_k |A[i, k] B[j, k]|: what the rounding error of a sum in another order is measured against"""
    blk = np.arange(k) // 32
    af = np.abs(mx_values(a, k, fa)) * np.power(2.0, sa.astype(np.float64) - 127.0)[:, blk]
    bf = np.abs(mx_values(b, k, fb)) * np.power(2.0, sb.astype(np.float64) - 127.0)[:, blk]
    return af @ bf.T


def mx_check(got, want, absdot, eight_bit):
    """Against the float64 golden rounded to fp32.  4-bit operands: the products are exact and the matrix core's fp32
    sums differ from the golden by the additions' rounding, a few 2^-24 of the sum of the terms' magnitudes.  8-bit
    operands: the matrix core aligns the 64 products of an instruction before it adds them and drops what falls below
    (measured: up to 2.3e-4 of the sum of magnitudes, median 1e-5, whatever the scales), so the bound is 1e-3 of that
    sum.  Either way, where nothing cancels the result is inside the reference's criterion rtol = 1e-3
    (verify_result.py); the scale bytes span 2^19 per operand here, so an element may be far smaller than its terms."""
    g, w = got.astype(np.float64), want.astype(np.float64)
    assert np.all(np.abs(g - w) <= (1e-3 if eight_bit else 4e-6) * absdot + 1e-30)
    plain = np.abs(w) > (0.5 if eight_bit else 0.01) * absdot
    assert np.all(np.abs(g - w)[plain] <= 2e-3 * np.abs(w)[plain])


def is8(fa, fb):
    return not (fa == F2 and fb == F2)     # every pair but e2m1 x e2m1 runs (or is widened to) 8-bit operands


@pytest.mark.parametrize("fa,fb", [(F1, F2), (F2, F1), (E4, E5), (E5, E4), (E4, E4), (F2, F2), (E5, F1)])
@pytest.mark.parametrize("bias", [False, True])
def test_mx_reference_example_shape(fa, fb, bias):
    """[40, 70] x [50, 70], the shape and the format pairs of the reference's MmadMx example: k is no multiple of 32,
    so the kernel with one lane per output element runs."""
    announce("mx example", fa, fb, bias)
    rng = np.random.default_rng(fa * 16 + fb + 100 * bias)
    m, n, k = 40, 50, 70
    a, b, sa, sb, bv = mx_case(rng, m, n, k, fa, fb, bias=bias)
    d = abi.MxDesc(m=m, n=n, k=k, scale_k=sa.shape[1], a_format=fa, b_format=fb, out_dtype=abi.F32, has_bias=int(bias))
    got = run_mx(m, n, k, a, b, sa, sb, fa, fb, bias=bv).cpu().numpy()
    mx_check(got - (bv if bias else 0), orc.matmul_mx(d, a, b, sa, sb, bv) - (bv if bias else 0),
             mx_abs_dot(a, b, sa, sb, k, fa, fb) + (np.abs(bv) if bias else 0), False)


@pytest.mark.parametrize("m,n,k", [(256, 256, 256), (64, 64, 1024), (300, 520, 512), (513, 272, 768), (1024, 256, 2048)])
@pytest.mark.parametrize("fa,fb", [(E4, E4), (E4, E5), (E5, E4), (E5, E5), (F2, F2), (F1, F1), (F2, F1), (E4, F2), (F1, E5)])
def test_mx_tile_kernel(m, n, k, fa, fb):
    """The tile kernel on the scaled matrix instruction: the four 8-bit pairs and e2m1 x e2m1 straight from the given
    buffers, the other pairs with their 4-bit operands widened to e4m3 first; row and column tails, odd and even
    numbers of K steps."""
    announce("mx tiles", m, n, k, fa, fb)
    rng = np.random.default_rng(m + n + k + fa * 16 + fb)
    a, b, sa, sb, _ = mx_case(rng, m, n, k, fa, fb)
    d = abi.MxDesc(m=m, n=n, k=k, scale_k=sa.shape[1], a_format=fa, b_format=fb, out_dtype=abi.F32, has_bias=0)
    orc.set_threads(16)
    want = orc.matmul_mx(d, a, b, sa, sb)
    mx_check(run_mx(m, n, k, a, b, sa, sb, fa, fb).cpu().numpy(), want, mx_abs_dot(a, b, sa, sb, k, fa, fb), is8(fa, fb))


@pytest.mark.parametrize("m,n,k,sk", [(128, 128, 256, 16), (128, 192, 128, 16), (256, 256, 1280, 40), (200, 136, 640, 24),
                                      (256, 256, 1024, 40), (320, 256, 2304, 72), (256, 256, 256, 8)])
@pytest.mark.parametrize("fa,fb", [(E4, E5), (F2, F2), (F1, E4)])
def test_mx_tile_kernel_scale_rows(m, n, k, sk, fa, fb):
    """The tile kernel fetches 16 scale bytes per row for every two K steps and moves the last fetch back to stay inside
    the row: rows of scale bytes that end in half a fetch, rows longer than k / 32, a single K step, odd numbers of
    steps; rows shorter than one fetch (the last case) go through the element-wise kernel."""
    announce("mx scale rows", m, n, k, sk, fa, fb)
    rng = np.random.default_rng(m + 3 * n + 5 * k + 7 * sk + fa * 16 + fb)
    a, b, sa, sb, _ = mx_case(rng, m, n, k, fa, fb, sk=sk)
    d = abi.MxDesc(m=m, n=n, k=k, scale_k=sk, a_format=fa, b_format=fb, out_dtype=abi.F32, has_bias=0)
    orc.set_threads(16)
    want = orc.matmul_mx(d, a, b, sa, sb)
    mx_check(run_mx(m, n, k, a, b, sa, sb, fa, fb).cpu().numpy(), want, mx_abs_dot(a, b, sa, sb, k, fa, fb), is8(fa, fb))


@pytest.mark.parametrize("n", [320, 257])
@pytest.mark.parametrize("out", [torch.bfloat16, torch.float16])
def test_mx_sixteen_bit_outputs_and_bias(out, n):
    """e2m1 operands (exact products, fp32 sums): a 16-bit result is the golden's or its neighbour.  An even n leaves
    the tile kernel as one dword per lane, an odd n element by element."""
    announce("mx 16-bit out", out, n)
    rng = np.random.default_rng(5)
    m, k = 256, 512
    a, b, sa, sb, bv = mx_case(rng, m, n, k, F2, F2, bias=True, lo=124, hi=130)
    dt = abi.BF16 if out == torch.bfloat16 else abi.F16
    d = abi.MxDesc(m=m, n=n, k=k, scale_k=sa.shape[1], a_format=F2, b_format=F2, out_dtype=dt, has_bias=1)
    want = orc.matmul_mx(d, a, b, sa, sb, bv).view(np.int16).astype(np.int32)
    got = run_mx(m, n, k, a, b, sa, sb, F2, F2, out=out, bias=bv).view(torch.int16).cpu().numpy().astype(np.int32)
    assert np.abs(got - want).max() <= 1 and np.mean(got == want) > 0.99


def test_mx_reference_data_distribution_and_criterion():
    """Operands drawn as the reference's data scripts draw them (uniform values cast to the format, scale bytes
    127..129: mmad_mx/scripts/gen_data.py:104-111, 161-165) and judged as its verify script judges (|out - golden| <=
    1e-3 + 1e-3 |golden| with at most one element in a thousand outside, verify_result.py).  e2m1 operands meet it
    (their products are exact and never far enough apart to be dropped).  fp8 operands on the scaled matrix
    instruction do not at this k: the instruction drops every product more than 2^13 below the largest of its 64 and
    truncates the others to that window, so sums in which the terms cancel carry an error of up to 2.3e-4 of the
    terms' magnitudes; about five elements in a thousand fall outside, and the bound asserted is one in a hundred."""
    announce("mx reference criterion")
    rng = np.random.default_rng(9)
    m, n, k = 512, 512, 1024
    sa, sb = rng.integers(127, 130, (m, k // 32)).astype(np.uint8), rng.integers(127, 130, (n, k // 32)).astype(np.uint8)
    orc.set_threads(16)

    def outside(a, b, fa, fb):
        d = abi.MxDesc(m=m, n=n, k=k, scale_k=k // 32, a_format=fa, b_format=fb, out_dtype=abi.F32, has_bias=0)
        want = orc.matmul_mx(d, a, b, sa, sb).astype(np.float64)
        got = run_mx(m, n, k, a, b, sa, sb, fa, fb).cpu().numpy().astype(np.float64)
        return (np.abs(got - want) > 1e-3 + 1e-3 * np.abs(want)).mean()

    a4, b4 = mx_random_operand(rng, m, k, F2), mx_random_operand(rng, n, k, F2)
    assert outside(a4, b4, F2, F2) == 0.0
    xa = torch.from_numpy(rng.uniform(-10, 10, (m, k)).astype(np.float32))
    xb = torch.from_numpy(rng.uniform(-10, 10, (n, k)).astype(np.float32))
    a8 = xa.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    b8 = xb.to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert outside(a8, b8, E4, E5) <= 1e-2


def test_mx_scale_byte_selection():
    """Every block of 32 k gets its own scale byte: the operands are all ones and one scale byte at a time is raised,
    which must add exactly 32 (8-bit) to one row or column of the result - whatever lane half, sub-step and K step
    the block falls into."""
    announce("mx scale bytes")
    m = n = 256
    for fmt, one, per_byte in ((E4, 0x38, 1), (F2, 0x22, 2)):
        k = 1024
        a = np.full((m, k // per_byte), one, np.uint8)
        b = np.full((n, k // per_byte), one, np.uint8)
        for blk in range(k // 32):
            sa, sb = np.full((m, k // 32), 127, np.uint8), np.full((n, k // 32), 127, np.uint8)
            sa[37 + blk, blk] = 128
            sb[200 - blk, blk] = 126
            want = np.full((m, n), float(k), np.float32)
            want[37 + blk, :] += 32
            want[:, 200 - blk] -= 16
            want[37 + blk, 200 - blk] = k - 32 + 32 * 2 * 0.5
            got = run_mx(m, n, k, a, b, sa, sb, fmt, fmt).cpu().numpy()
            assert np.array_equal(got, want), (fmt, blk)


def test_mx_reference_benchmark_shape_sampled():
    """m = n = k = 8192 (the shape of the reference's high-performance MxFP4 example, bfloat16 output) in e2m1 and in
    e1m2, which that example uses: rows from the first, a middle and the last tile against the oracle."""
    announce("mx 8192^3")
    rng = np.random.default_rng(8192)
    m = n = k = 8192
    orc.set_threads(16)
    for fmt in (F2, F1):
        a, b, sa, sb, _ = mx_case(rng, m, n, k, fmt, fmt, lo=127, hi=130)     # scales as in the example's data script
        got = run_mx(m, n, k, a, b, sa, sb, fmt, fmt, out=torch.bfloat16).view(torch.int16).cpu().numpy()
        d = abi.MxDesc(m=m, n=n, k=k, scale_k=sa.shape[1], a_format=fmt, b_format=fmt, out_dtype=abi.BF16, has_bias=0)
        for r0 in (0, 4093, 8188):
            want = orc.matmul_mx(d, a, b, sa, sb, rows=(r0, r0 + 4))[r0:r0 + 4].view(np.int16)
            diff = np.abs(got[r0:r0 + 4].astype(np.int32) - want.astype(np.int32))
            assert diff.max() <= 1 and np.mean(diff == 0) > 0.99


def test_mx_rejects_what_it_cannot_compute():
    lib = abi.load_library()
    need = C.c_size_t(0)
    d = abi.MxDesc(m=4, n=4, k=63, scale_k=2, a_format=F2, b_format=E4, out_dtype=abi.F32, has_bias=0)
    assert lib.ascq_matmul_mx_workspace_size(C.byref(d), C.byref(need)) == abi.EINVAL       # odd k with a 4-bit operand
    d = abi.MxDesc(m=4, n=4, k=64, scale_k=1, a_format=E4, b_format=E4, out_dtype=abi.F32, has_bias=0)
    assert lib.ascq_matmul_mx_workspace_size(C.byref(d), C.byref(need)) == abi.EINVAL       # scale rows too short
    d = abi.MxDesc(m=4, n=4, k=64, scale_k=2, a_format=abi.QDST_I8, b_format=E4, out_dtype=abi.F32, has_bias=0)
    assert lib.ascq_matmul_mx_workspace_size(C.byref(d), C.byref(need)) == abi.EINVAL
    d = abi.MxDesc(m=256, n=256, k=512, scale_k=16, a_format=F1, b_format=E4, out_dtype=abi.F32, has_bias=0)
    assert lib.ascq_matmul_mx_workspace_size(C.byref(d), C.byref(need)) == abi.OK and need.value == 256 * 512
