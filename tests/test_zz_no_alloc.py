"""The entry point that allocates nothing (ascq_linear_w8a8_dynamic_noalloc) against the workspace form it is a variant
of (ascq_linear_w8a8_dynamic), through the C ABI: bit-identical outputs on two calls in a row, the second with a
smaller input, at a decode shape (partial sums in the scratch), a split-K shape and a large-M shape (quantised
activations in the scratch).  The scratch is shared by every call on the GPU and keeps the previous call's contents."""
import ctypes as C

import numpy as np
import pytest
import torch

import orc
from ascq import _abi as abi
from gpu_util import DEV, announce

pytestmark = pytest.mark.gpu
L = abi.load_library()


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def desc(m, n, k, bias):
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32)
    if bias is not None:
        d.bias_kind = abi.MM_BIAS_F32_POST
    return d


def both(m, n, k, seed, with_bias):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    x = torch.randn((m, k), device=DEV, generator=g).to(torch.bfloat16)
    w = torch.randint(-127, 128, (k, n), dtype=torch.int8, device=DEV, generator=g)
    cs = torch.rand(n, device=DEV, generator=g) * 1e-2 + 1e-4
    bias = torch.randn(n, device=DEV, generator=g) if with_bias else None
    d = desc(m, n, k, bias)
    need = C.c_size_t(0)
    assert L.ascq_linear_w8a8_dynamic_workspace_size(C.byref(d), C.byref(need)) == abi.OK
    ws = torch.empty(max(need.value, 16), dtype=torch.uint8, device=DEV)
    want = torch.full((m, n), -1.0, dtype=torch.bfloat16, device=DEV)
    got = torch.full((m, n), -2.0, dtype=torch.bfloat16, device=DEV)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = L.ascq_linear_w8a8_dynamic(C.byref(d), abi.BF16, ptr(want), ptr(x), ptr(w), ptr(bias), ptr(cs), ptr(ws),
                                    ws.numel(), stream)
    assert rc == abi.OK, L.ascq_last_error().decode()
    rc = L.ascq_linear_w8a8_dynamic_noalloc(C.byref(d), abi.BF16, ptr(got), ptr(x), ptr(w), ptr(bias), ptr(cs), stream)
    assert rc == abi.OK, L.ascq_last_error().decode()
    torch.cuda.synchronize()
    return got, want, (x, w, cs, bias, d)


@pytest.mark.parametrize("first,second", [((16, 1040, 2048), (3, 528, 1024)),        # weight-stream kernels: partial sums
                                           ((128, 2064, 1024), (40, 528, 512)),        # 128-row tiles, K split over workgroups
                                           ((600, 528, 640), (300, 272, 512))])        # large tiles: q and token scales only
def test_noalloc_equals_workspace_form_two_calls(first, second):
    for i, (m, n, k) in enumerate((first, second)):
        announce("noalloc", m, n, k)
        got, want, _ = both(m, n, k, seed=100 + i, with_bias=bool(i))
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"call {i}: differs from the workspace form"


def test_noalloc_against_oracle_small():
    m, n, k = 5, 272, 256
    announce("noalloc oracle", m, n, k)
    got, _, (x, w, cs, bias, d) = both(m, n, k, seed=7, with_bias=False)
    xb = x.view(torch.int16).cpu().numpy().view(np.uint16)
    q, ts = orc.dynamic_quant_per_token(abi.BF16, xb)
    dd = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32,
                        has_tok_scale=1)
    want = orc.matmul_w8a8(dd, q, w.cpu().numpy(), None, cs.cpu().numpy(), ts)
    assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want)


def test_noalloc_rejects_shapes_beyond_its_buffer():
    d = desc(32, 11008, 4096, None)                 # 32 MiB of partial sums
    rc = L.ascq_linear_w8a8_dynamic_noalloc(C.byref(d), abi.BF16, C.c_void_p(0x1000), C.c_void_p(0x1000),
                                            C.c_void_p(0x1000), None, C.c_void_p(0x1000), None)
    assert rc == abi.EINVAL and "built-in buffer" in L.ascq_last_error().decode()


@pytest.mark.parametrize("m,n,k", [(7, 544, 512), (300, 544, 512)])
def test_noalloc_wrapper_with_swiglu(m, n, k):
    """The Python wrapper takes n from the weight (with SwiGLU the output has n / 2 columns) and passes act_beta on: its
    result is that of the workspace form's wrapper, bit for bit."""
    from ascq import ops
    announce("noalloc swiglu wrapper", m, n, k)
    g = torch.Generator(device=DEV)
    g.manual_seed(31)
    x = torch.randn((m, k), device=DEV, generator=g).to(torch.bfloat16)
    w = torch.randint(-127, 128, (k, n), dtype=torch.int8, device=DEV, generator=g)
    cs = torch.rand(n, device=DEV, generator=g) * 1e-2 + 1e-4
    want = torch.full((m, n // 2), -1.0, dtype=torch.bfloat16, device=DEV)
    got = torch.full((m, n // 2), -2.0, dtype=torch.bfloat16, device=DEV)
    ops.linear_w8a8_dynamic(want, x, w, cs, activation=abi.MM_ACT_SWIGLU, act_beta=1.702)
    ops.linear_w8a8_dynamic_noalloc(got, x, w, cs, activation=abi.MM_ACT_SWIGLU, act_beta=1.702)
    plain = torch.empty_like(want)
    ops.linear_w8a8_dynamic(plain, x, w, cs, activation=abi.MM_ACT_SWIGLU, act_beta=1.0)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert not torch.equal(plain.view(torch.int16), want.view(torch.int16)), "act_beta had no effect"
