"""Writes tests/golden/hif8_vectors.npz: inputs and outputs of the hifloat8 conversions that ship with the reference
as a Python script (examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_fp8/scripts/hif8.py).  No document table
or test vector in the reference fixes the hifloat8 encoding, so the script's functions are run once, here, and their
results kept as data:

  decode      float32[256]   cvt_hifuint8_to_float(code) for every code (over_mode True: 128 is NaN, 111 / 239 +-inf)
  f32_in      float32[n]     inputs of the float32 encoder: every code's value, the midpoints between neighbouring
                             values and their float32 neighbours, powers of two around the range ends, random values
  f32_round   uint8[n]       cvt_float32_to_hifuint8(x, "round", over_mode=False)
  f32_hybrid  uint8[n]       cvt_float32_to_hifuint8(x, "hybrid", over_mode=False)
  f32_round_inf uint8[n]     cvt_float32_to_hifuint8(x, "round", over_mode=True)
  f16_round   uint8[65536]   cvt_float16_to_hifuint8(h, "round", over_mode=False) for every float16 bit pattern
  f16_hybrid  uint8[65536]   the same with "hybrid"

Run from the repository root with the reference checked out at /root/reference:  python3 tests/golden/make_hif8_vectors.py
"""
import importlib.util
import os
import sys

import numpy as np

REF = "/root/reference/examples/01_simd_cpp_api/04_advanced_api/00_matmul/matmul_fp8/scripts/hif8.py"


def main():
    spec = importlib.util.spec_from_file_location("ref_hif8", REF)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)

    decode = np.array([ref.cvt_hifuint8_to_float(c) for c in range(256)], dtype=np.float32)
    finite = np.unique(np.abs(decode[np.isfinite(decode)]))
    mids = (finite[:-1].astype(np.float64) + finite[1:].astype(np.float64)) / 2
    pts = [finite, mids.astype(np.float32)]
    for base in (finite, mids.astype(np.float32)):
        pts.append(np.nextafter(base, np.float32(np.inf)).astype(np.float32))
        pts.append(np.nextafter(base, np.float32(0)).astype(np.float32))
    pts.append(np.array([2.0 ** e for e in range(-26, 18)], dtype=np.float32))
    pts.append(np.array([1.25 * 2 ** 15, 1.2499 * 2 ** 15, 1.5 * 2 ** 15, 3.0e38, 1e-30, 1.5 * 2 ** -23, 1.4999 * 2 ** -23],
                        dtype=np.float32))
    rng = np.random.default_rng(0x41F8)
    pts.append((rng.standard_normal(6000) * np.exp2(rng.integers(-24, 16, 6000))).astype(np.float32))
    pos = np.concatenate(pts).astype(np.float32)
    f32_in = np.concatenate([pos, -pos, np.array([0.0, -0.0, np.inf, -np.inf, np.nan], dtype=np.float32)])

    def enc32(mode, over):
        with np.errstate(all="ignore"):
            return np.array([ref.cvt_float32_to_hifuint8(np.float32(x), mode, over) for x in f32_in]).astype(np.uint8)

    halves = np.arange(65536, dtype=np.uint16).view(np.float16)

    def enc16(mode):
        out = np.zeros(65536, dtype=np.uint8)
        bad = np.zeros(65536, dtype=bool)
        with np.errstate(all="ignore"):
            for i, h in enumerate(halves):
                try:
                    out[i] = int(ref.cvt_float16_to_hifuint8(h, mode, False)) & 0xFF
                except Exception:                       # the script raises on a few inputs; they are marked, not used
                    bad[i] = True
        return out, bad

    f16_round, bad_round = enc16("round")
    f16_hybrid, bad_hybrid = enc16("hybrid")
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hif8_vectors.npz")
    np.savez_compressed(out, decode=decode, f32_in=f32_in, f32_round=enc32("round", False), f32_hybrid=enc32("hybrid", False),
                        f32_round_inf=enc32("round", True), f16_round=f16_round, f16_hybrid=f16_hybrid,
                        f16_round_raised=bad_round, f16_hybrid_raised=bad_hybrid)
    print("wrote", out, os.path.getsize(out), "bytes;", f32_in.size, "float32 inputs;", int(bad_round.sum()),
          int(bad_hybrid.sum()), "float16 inputs on which the script raised")


if __name__ == "__main__":
    sys.exit(main())
