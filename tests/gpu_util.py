"""Helpers for the GPU parity tests: numpy <-> device tensors by bit pattern, seeded inputs, ulp distance."""
import sys

import numpy as np
import torch

from ascq import _abi as abi

DEV = "cuda:0"


def announce(*what):
    """Name the case before the GPU step runs, so that a fault can be attributed."""
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def to_dev(a, kind=None):
    """numpy array -> device tensor.  kind 'bf16' / 'f16' reinterpret uint16 bit patterns."""
    a = np.ascontiguousarray(a)
    if kind == "bf16":
        return torch.from_numpy(a.view(np.int16)).to(DEV).view(torch.bfloat16)
    if kind == "f16" and a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).to(DEV).view(torch.float16)
    if a.dtype == np.uint64:
        return torch.from_numpy(a.view(np.int64)).to(DEV)
    return torch.from_numpy(a).to(DEV)


def bits(t):
    """device tensor -> numpy array of its raw bit pattern (uint16 for 16-bit floats)."""
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def as_bits(a):
    return a.view(np.uint16) if a.dtype == np.float16 else a


def ordered(u16, fmt):
    """Map 16-bit float bit patterns to integers whose difference is the distance in ulps."""
    u = u16.astype(np.int32)
    return np.where(u & 0x8000, -(u & 0x7FFF), u)


def max_ulp(got_bits, want_bits, fmt="bf16"):
    return int(np.abs(ordered(got_bits, fmt) - ordered(want_bits, fmt)).max()) if got_bits.size else 0


def src_array(rng, shape, dtype, scale=1.0):
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    if dtype == abi.F32:
        return x, to_dev(x)
    import orc
    if dtype == abi.F16:
        h = x.astype(np.float16)
        return h, to_dev(h)
    b = orc.f32_to_bf16_bits(x)
    return b, to_dev(b, "bf16")


def param_array(rng, shape, dtype, lo, hi):
    return src_array_uniform(rng, shape, dtype, lo, hi)


def src_array_uniform(rng, shape, dtype, lo, hi):
    x = rng.uniform(lo, hi, shape).astype(np.float32)
    if dtype == abi.F32:
        return x, to_dev(x)
    import orc
    if dtype == abi.F16:
        h = x.astype(np.float16)
        return h, to_dev(h)
    b = orc.f32_to_bf16_bits(x)
    return b, to_dev(b, "bf16")


def pack_int4(w):
    """int array in [-8, 7], last axis even -> uint8, element 2j in the low nibble."""
    flat = w.reshape(-1).astype(np.uint8) & 0xF
    return (flat[0::2] | (flat[1::2] << 4)).astype(np.uint8).reshape(*w.shape[:-1], w.shape[-1] // 2)
