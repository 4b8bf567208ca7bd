"""The library allocates nothing and clears scratch with kernels, so its calls can be captured into a HIP graph.
Replays (with eager work of the same kind between them) must reproduce the eager result bit for bit."""
import numpy as np
import pytest
import torch

from ascq import ops
from gpu_util import DEV, announce

pytestmark = pytest.mark.gpu


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()                                   # warm-up on the stream that will capture: the wrappers key their scratch
    torch.cuda.current_stream().wait_stream(side)  # buffers by stream, so those the capture uses exist afterwards
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        fn()
    torch.cuda.synchronize()
    return graph


@pytest.mark.parametrize("m", [1, 48, 300])
def test_quant_linear_step_replays_like_eager(m):
    announce("graph: quant + w8a8", m)
    k, n = 1024, 1056
    gen = torch.Generator(device=DEV)
    gen.manual_seed(m)
    x = torch.randn((m, k), device=DEV, generator=gen).to(torch.bfloat16)
    w = torch.randint(-127, 128, (k, n), dtype=torch.int8, device=DEV, generator=gen)
    cs = torch.rand(n, device=DEV, generator=gen) * 1e-2 + 1e-4
    q = torch.empty((m, k), dtype=torch.int8, device=DEV)
    ts = torch.empty(m, dtype=torch.float32, device=DEV)
    c = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    mm = ops.Matmul(m, n, k)
    mm.set_tensor_a(q)
    mm.set_tensor_b(w)
    mm.set_quant_vector(cs)
    mm.set_token_scale(ts)

    def step():
        ops.dynamic_quant_per_token(x, q, ts)
        mm.iterate_all(c)

    step()
    torch.cuda.synchronize()
    want = c.clone()
    graph = _capture(step)
    for _ in range(3):
        x2 = torch.randn((m, k), device=DEV, generator=gen).to(torch.bfloat16)
        x.copy_(x2)
        step()                                  # eager, new activations
        torch.cuda.synchronize()
        eager = c.clone()
        c.zero_()
        graph.replay()                          # the graph reads the same buffers: must give the same output
        torch.cuda.synchronize()
        assert torch.equal(c.view(torch.int16), eager.view(torch.int16))
    assert not torch.equal(want.view(torch.int16), c.view(torch.int16))      # the inputs did change


@pytest.mark.parametrize("m", [1, 16])
def test_w4a16_replays_like_eager(m):
    announce("graph: w4a16", m)
    k, n, gs = 1024, 2048, 128
    gen = torch.Generator(device=DEV)
    gen.manual_seed(100 + m)
    x = torch.randn((m, k), device=DEV, generator=gen).to(torch.float16)
    w = torch.randint(0, 256, (k, n // 2), dtype=torch.uint8, device=DEV, generator=gen)
    sc = (torch.rand((k // gs, n), device=DEV, generator=gen) * 9e-3 + 1e-3).to(torch.float16)
    of = torch.randint(-8, 8, (k // gs, n), device=DEV, generator=gen).to(torch.float16)
    y = torch.empty((m, n), dtype=torch.float16, device=DEV)

    def step():
        ops.matmul_w4a16(y, x, w, sc, of, gs)

    graph = _capture(step)
    for _ in range(3):
        x.copy_(torch.randn((m, k), device=DEV, generator=gen).to(torch.float16))
        step()
        torch.cuda.synchronize()
        eager = y.clone()
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), eager.view(torch.int16))


def test_grouped_and_whole_column_kernels_replay_like_eager():
    """The persistent grouped kernel (its plan lives in LDS, nothing in global memory), the whole-column kernels on [n, k]
    weights, the packed W4A16 GEMV and the W8A16 tile GEMM in one captured sequence."""
    announce("graph: grouped + [n, k] + packed")
    from ascq import _abi as abi
    gen = torch.Generator(device=DEV)
    gen.manual_seed(7)
    ri = lambda lo, hi, shape, dt=torch.int8: torch.randint(lo, hi, shape, dtype=dt, device=DEV, generator=gen)
    # grouped
    G, T, K, N = 3, 700, 256, 4352
    gl = torch.tensor([300, 10, 390], dtype=torch.int64, device=DEV)
    xg, wg = ri(-127, 128, (T, K)), ri(-127, 128, (G, K, N))
    cs = torch.rand((G, N), device=DEV, generator=gen) * 1e-2 + 1e-4
    ts = torch.rand(T, device=DEV, generator=gen) + 0.5
    yg = torch.empty((T, N), dtype=torch.bfloat16, device=DEV)
    # int8 decode on [n, k]
    a8, w8 = ri(-127, 128, (5, 512)), ri(-127, 128, (1040, 512))
    cs8 = torch.rand(1040, device=DEV, generator=gen) * 1e-2 + 1e-4
    c8 = torch.empty((5, 1040), dtype=torch.bfloat16, device=DEV)
    mm = ops.Matmul(5, 1040, 512, False, True)
    mm.set_tensor_a(a8)
    mm.set_tensor_b(w8)
    mm.set_quant_vector(cs8)
    # W8A16 on [n, k]: decode and tile GEMM
    xh = torch.randn((3, 512), device=DEV, generator=gen).to(torch.float16)
    xh2 = torch.randn((200, 512), device=DEV, generator=gen).to(torch.float16)
    sc16 = (torch.rand(1040, device=DEV, generator=gen) * 9e-3 + 1e-3).to(torch.float16)
    y16 = torch.empty((3, 1040), dtype=torch.float16, device=DEV)
    y16b = torch.empty((200, 1040), dtype=torch.float16, device=DEV)
    # packed W4A16
    k4, n4, gs = 512, 1024, 128
    w4 = ops.pack_weight_w4(ri(0, 256, (k4, n4 // 2), torch.uint8), k4, n4)
    sc4 = (torch.rand((k4 // gs, n4), device=DEV, generator=gen) * 9e-3 + 1e-3).to(torch.float16)
    x4 = torch.randn((2, k4), device=DEV, generator=gen).to(torch.float16)
    y4 = torch.empty((2, n4), dtype=torch.float16, device=DEV)
    outs = (yg, c8, y16, y16b, y4)

    def step():
        ops.quant_group_matmul(yg, xg, wg, gl, cs, ts, None, abi.GROUP_LIST_COUNTS)
        mm.iterate_all(c8)
        ops.matmul_w8a16(y16, xh, w8, None, sc16, trans_b=True)
        ops.matmul_w8a16(y16b, xh2, w8, None, sc16, trans_b=True)
        ops.matmul_w4a16_packed(y4, x4, w4, sc4, None, gs)

    graph = _capture(step)
    for _ in range(3):
        xg.copy_(ri(-127, 128, (T, K)))
        a8.copy_(ri(-127, 128, (5, 512)))
        xh.copy_(torch.randn((3, 512), device=DEV, generator=gen).to(torch.float16))
        xh2.copy_(torch.randn((200, 512), device=DEV, generator=gen).to(torch.float16))
        x4.copy_(torch.randn((2, k4), device=DEV, generator=gen).to(torch.float16))
        step()
        torch.cuda.synchronize()
        eager = [o.clone() for o in outs]
        for o in outs:
            o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for o, e in zip(outs, eager):
            assert torch.equal(o.view(torch.int16), e.view(torch.int16))
