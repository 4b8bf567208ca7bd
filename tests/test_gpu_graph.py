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
        fn()                                   # warm-up on a side stream: lazily created workspaces exist afterwards
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
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
