"""No-GPU checks of the C ABI: the library loads, exports every symbol include/ascq.h declares, rejects bad
descriptors with the documented status before touching the GPU, and answers the host tiling queries with the
reference's known answers (tests/api/adv_api/tiling/test_tiling.cpp:6539-6703 of the reference)."""
import ctypes as C
import os
import re

import pytest

from ascq import _abi as abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
L = abi.load_library()
FAKE = C.c_void_p(0x1000)          # never dereferenced: validation fails first


def err():
    return L.ascq_last_error().decode()


def test_every_declared_symbol_is_exported_and_bound():
    header = open(os.path.join(ROOT, "include", "ascq.h")).read()
    declared = set(re.findall(r"\b(ascq_[a-z0-9_]+)\s*\(", header))
    assert declared == set(abi.SIGNATURES), declared ^ set(abi.SIGNATURES)
    for name in declared:
        assert hasattr(L, name)
    assert b"gfx950" in L.ascq_version()


def test_struct_sizes_match_the_header():
    # field-by-field layout is 4-byte scalars; the matmul descriptor ends with an 8-byte word
    assert C.sizeof(abi.QuantDesc) == 14 * 4
    assert C.sizeof(abi.DequantDesc) == 11 * 4
    assert C.sizeof(abi.AntiQuantDesc) == 13 * 4
    assert C.sizeof(abi.MatmulDesc) == 11 * 4 + 4 + 8 + 8
    assert C.sizeof(abi.GroupMatmulDesc) == C.sizeof(abi.MatmulDesc) + 8
    assert C.sizeof(abi.W4A16Desc) == 6 * 4
    assert C.sizeof(abi.W8A16Desc) == 10 * 4
    assert C.sizeof(abi.AntiQuantPolicyDesc) == 14 * 4
    assert C.sizeof(abi.MxDesc) == 8 * 4


def q(**kw):
    d = abi.QuantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.F16, scale_dtype=abi.F16, compute=abi.COMPUTE_F16,
                      round_mode=abi.CAST_RINT, offset_kind=abi.OFFSET_SCALAR, k_dim=1, n=64, cal_count=640)
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def test_quant_rejections():
    call = lambda d, dst=FAKE, src=C.c_void_p(0x100000), sc=FAKE, of=FAKE: L.ascq_quant(C.byref(d), dst, src, sc, of, None)
    assert L.ascq_quant(None, FAKE, FAKE, FAKE, FAKE, None) == abi.ENULL
    assert call(q(), dst=None) == abi.ENULL
    assert call(q(), sc=None) == abi.ENULL
    assert call(q(offset_kind=abi.OFFSET_TENSOR), of=None) == abi.ENULL
    assert call(q(policy=9)) == abi.EINVAL
    assert call(q(cal_count=650)) == abi.EINVAL and "integer multiple" in err()      # calCount % scaleCount != 0
    assert call(q(n=0)) == abi.EINVAL
    assert call(q(src_dtype=abi.I8)) == abi.EUNSUPPORTED
    assert call(q(round_mode=6)) == abi.EUNSUPPORTED                                   # CAST_ODD has no int8 form
    assert call(q(dst_format=3)) == abi.EUNSUPPORTED                                   # int8 / fp8_e4m3fn / fp8_e5m2 only
    assert call(q(dst_format=abi.QDST_FP8_E5M2)) == abi.EUNSUPPORTED                   # the fp16 contract is int8 only
    assert call(q(policy=abi.PER_TOKEN)) == abi.EUNSUPPORTED                           # fp16 compute is tensor/channel only
    assert call(q(scale_dtype=abi.F32)) == abi.EUNSUPPORTED                            # legacy: scale dtype == src dtype
    tok = dict(policy=abi.PER_TOKEN, compute=abi.COMPUTE_SCALE_T, m=10, n=288, cal_count=2880)
    assert call(q(src_dtype=abi.F32, scale_dtype=abi.F16, **tok)) == abi.EUNSUPPORTED  # (float, half) is not a legal pair
    assert call(q(**dict(tok, cal_count=2881))) == abi.EINVAL
    assert call(q(**dict(tok, m=9))) == abi.EINVAL                                     # calCount > m*n
    assert call(q(**dict(tok, n=24, cal_count=240))) == abi.EALIGN                     # 48-byte rows
    grp = dict(tok, policy=abi.PER_GROUP, n=256, cal_count=2560)
    assert call(q(group_size=48, **grp)) == abi.EINVAL and "multiple of 32" in err()
    assert call(q(group_size=0, **grp)) == abi.EINVAL
    assert call(q(group_size=64, k_dim=2, **grp)) == abi.EINVAL
    assert call(q(), dst=C.c_void_p(0x100010)) == abi.EINVAL and "overlaps" in err()
    assert call(q(cal_count=0)) == abi.OK                                              # nothing to do, nothing launched


def test_in_place_calls_are_rejected():
    """The reference lets AscendQuant's destination reuse the source's memory; the GPU kernels cannot (other wavefronts
    still have to read what an output byte would cover), so dst == src, or any intersection of the byte ranges, is
    ASCQ_EINVAL before anything is launched."""
    src = C.c_void_p(0x100000)
    for dst in (src, C.c_void_p(0x100000 + 2 * 640 - 1), C.c_void_p(0x100000 - 639)):
        assert L.ascq_quant(C.byref(q()), dst, src, FAKE, FAKE, None) == abi.EINVAL and "overlaps" in err()
    dq = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.BF16,
                         mode=abi.DEQUANT_WITH_MULTI_ROW, m=4, n=64, cal_count=64)
    assert L.ascq_dequant(C.byref(dq), src, src, FAKE, None) == abi.EINVAL and "overlaps" in err()
    aq = abi.AntiQuantDesc(src_dtype=abi.I8, dst_dtype=abi.F16, has_offset=1, k=64, n=128, scale_height=1,
                           scale_width=128, offset_height=1, offset_width=128)
    assert L.ascq_antiquant(C.byref(aq), src, src, FAKE, FAKE, None) == abi.EINVAL and "overlaps" in err()


def test_dequant_rejections():
    def d(**kw):
        x = abi.DequantDesc(policy=abi.PER_CHANNEL, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.BF16,
                            mode=abi.DEQUANT_WITH_MULTI_ROW, m=4, n=64, cal_count=64)
        for k, v in kw.items():
            setattr(x, k, v)
        return x
    call = lambda x, sc=FAKE: L.ascq_dequant(C.byref(x), FAKE, C.c_void_p(0x100000), sc, None)
    assert call(d(), sc=None) == abi.ENULL
    assert call(d(n=60, cal_count=60)) == abi.EALIGN                                   # 240-byte rows
    assert call(d(cal_count=65)) == abi.EINVAL
    assert call(d(dst_dtype=abi.F16)) == abi.EUNSUPPORTED                              # half out needs uint64 scale
    assert call(d(scale_dtype=abi.U64, dst_dtype=abi.BF16)) == abi.EUNSUPPORTED
    assert call(d(policy=abi.PER_TENSOR, dst_dtype=abi.F16)) == abi.EUNSUPPORTED
    assert call(d(src_dtype=abi.F32)) == abi.EUNSUPPORTED
    assert call(d(policy=abi.PER_GROUP, group_size=40, k_dim=1)) == abi.EINVAL
    assert call(d(m=0)) == abi.EINVAL
    assert L.ascq_dequant_dst_stride(abi.BF16, 40) == 48 and L.ascq_dequant_dst_stride(abi.F32, 40) == 40


def test_antiquant_rejections():
    def d(**kw):
        x = abi.AntiQuantDesc(src_dtype=abi.I8, dst_dtype=abi.F16, has_offset=1, k=64, n=128, scale_height=1,
                              scale_width=128, offset_height=1, offset_width=128)
        for k, v in kw.items():
            setattr(x, k, v)
        return x
    call = lambda x, of=FAKE, sc=FAKE: L.ascq_antiquant(C.byref(x), FAKE, C.c_void_p(0x100000), of, sc, None)
    assert call(d(), sc=None) == abi.ENULL
    assert call(d(), of=None) == abi.ENULL
    assert call(d(src_dtype=abi.F16)) == abi.EUNSUPPORTED
    assert call(d(dst_dtype=abi.F32)) == abi.EUNSUPPORTED
    assert call(d(scale_height=3)) == abi.EINVAL                                       # k % groups != 0
    assert call(d(offset_height=2, scale_height=4)) == abi.EINVAL
    assert call(d(is_transpose=1, k=48, scale_width=1, scale_height=128, offset_width=1, offset_height=128)) == abi.EALIGN  # k not 32-byte aligned
    assert call(d(k=0)) == abi.EINVAL


def test_matmul_rejections():
    def d(**kw):
        x = abi.MatmulDesc(m=32, n=64, k=64, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                           scale_format=abi.MM_SCALE_F32)
        for k, v in kw.items():
            setattr(x, k, v)
        return x
    call = lambda x, bias=None, qv=FAKE, tok=None: L.ascq_matmul_w8a8(C.byref(x), FAKE, FAKE, FAKE, bias, qv, tok,
                                                                     None, 0, None)
    assert call(d(), qv=None) == abi.ENULL
    assert call(d(bias_kind=abi.MM_BIAS_F32_POST)) == abi.ENULL
    assert call(d(has_tok_scale=1)) == abi.ENULL
    assert call(d(k=0)) == abi.EINVAL
    assert call(d(out_dtype=abi.I32)) == abi.EUNSUPPORTED
    assert call(d(out_dtype=abi.I8)) == abi.EUNSUPPORTED                               # requant needs the uint64 words
    assert call(d(quant_mode=abi.MM_QUANT_NONE)) == abi.EUNSUPPORTED                   # int32 out only
    assert call(d(quant_mode=abi.MM_QUANT_NONE, out_dtype=abi.I32, has_tok_scale=1), tok=FAKE) == abi.EUNSUPPORTED
    g = abi.GroupMatmulDesc(mm=d(), groups=0, group_list_kind=abi.GROUP_LIST_COUNTS)
    gcall = lambda x, gl=FAKE: L.ascq_group_matmul_w8a8(C.byref(x), FAKE, FAKE, FAKE, None, FAKE, None, gl, None)
    assert gcall(g) == abi.EINVAL
    g.groups = 4
    assert gcall(g, gl=None) == abi.ENULL
    g.mm.scale_format = abi.MM_SCALE_U64
    assert gcall(g) == abi.EUNSUPPORTED
    g.mm.scale_format, g.mm.k = abi.MM_SCALE_F32, 72
    assert gcall(g) == abi.EALIGN


def test_w4a16_rejections_and_workspace():
    d = abi.W4A16Desc(m=1, n=1024, k=512, group_size=128, has_offset=1)
    n = C.c_size_t(0)
    assert L.ascq_matmul_w4a16_workspace_size(C.byref(d), C.byref(n)) == abi.OK and n.value % (1024 * 4) == 0
    assert L.ascq_matmul_w4a16(C.byref(d), FAKE, FAKE, FAKE, FAKE, None, FAKE, 1 << 30, None) == abi.ENULL
    assert L.ascq_matmul_w4a16(C.byref(d), FAKE, FAKE, FAKE, FAKE, FAKE, None, 0, None) == abi.EINVAL
    assert "workspace" in err()
    d.group_size = 96
    assert L.ascq_matmul_w4a16_workspace_size(C.byref(d), C.byref(n)) == abi.EINVAL
    d.group_size, d.n = 128, 1023
    assert L.ascq_matmul_w4a16_workspace_size(C.byref(d), C.byref(n)) == abi.EINVAL


def sizes(fn, *args):
    mx, mn = C.c_uint32(0), C.c_uint32(0)
    rc = fn(*args, C.byref(mx), C.byref(mn))
    return rc, mx.value, mn.value


def u32(*v):
    return (C.c_uint32 * len(v))(*v)


def test_tiling_known_answers():
    # TestAscendQuantTiling: {512} x 2 bytes -> min 2*256, max 2*512
    assert sizes(L.ascq_get_ascend_quant_max_min_tmp_size, u32(512), 1, 2) == (abi.OK, 1024, 512)
    # TestAscendDequantTiling (the reference passes typeSize 2: reported, sizes still produced)
    rc, mx, mn = sizes(L.ascq_get_ascend_dequant_max_min_tmp_size, u32(10, 32), 2, 2)
    assert (mx, mn) == (4 * (64 + 32 * 10 + 40), 4 * (64 + 32 + 40)) and rc == abi.EUNSUPPORTED
    assert sizes(L.ascq_get_ascend_dequant_max_min_tmp_size, u32(320), 1, 4) == (abi.OK, 4 * (64 + 320 + 328),
                                                                                4 * (64 + 320 + 328))
    aq = L.ascq_get_ascend_antiquant_max_min_tmp_size
    # TestAntiquantTilingNoTransposePerChannelHalf / ...PerChannel / ...PerTensor / TransposePerChannel
    assert sizes(aq, u32(640, 5120), 2, u32(1, 5120), 2, 0, abi.I8, abi.F16) == (abi.OK, 0, 0)
    exp = 5120 * 2 * 4 + 64 * 640 * 4
    assert sizes(aq, u32(640, 5120), 2, u32(1, 5120), 2, 0, abi.I8, abi.BF16) == (abi.OK, exp, exp)
    assert sizes(aq, u32(640, 5120), 2, u32(1), 1, 0, abi.I8, abi.BF16) == (abi.OK, 640 * 5120 * 4, 1024)
    assert sizes(aq, u32(64, 512), 2, u32(64, 1), 2, 1, abi.I8, abi.BF16) == (abi.OK, 80 * 64 * 4, 80 * 64 * 4)
    assert sizes(aq, u32(640, 5120), 2, u32(1), 1, 1, abi.I8, abi.BF16) == (abi.OK, 640 * 5120 * 4, 1024)


def test_pack_quant_param():
    import numpy as np
    w = L.ascq_pack_quant_param(0.1, 5, 1)
    assert (w & 0xFFFFFFFF) == int(np.float32(0.1).view(np.uint32)) and (w >> 37) & 0x1FF == 5 and (w >> 46) & 1 == 1


def test_cpp_host_mirror_header_compiles_standalone(tmp_path):
    """include/ascq_ascendc.hpp is plain C++17 on top of ascq.h: it must compile with the host compiler alone."""
    import subprocess
    src = tmp_path / "t.cpp"
    src.write_text('#include "ascq_ascendc.hpp"\n'
                   'int main() { ascq::Matmul<ascq::bfloat16_t> mm(1, 1, 1); return mm.Desc().m == 1 ? 0 : 1; }\n')
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "include")
    subprocess.check_call(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", inc, str(src)])


def _plan(m, n, k, a=0x10000, b=0x20000, ws=True, **kw):
    d = abi.MatmulDesc(m=m, n=n, k=k, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                       scale_format=abi.MM_SCALE_F32, has_tok_scale=1, **kw)
    need = C.c_size_t(0)
    assert L.ascq_matmul_w8a8_workspace_size(C.byref(d), C.byref(need)) == abi.OK
    p = abi.MatmulPlan()
    have = need.value if ws else 0
    rc = L.ascq_matmul_w8a8_plan(C.byref(d), C.c_void_p(0x30000), C.c_void_p(a), C.c_void_p(b), None,
                                 C.c_void_p(0x40000), C.c_void_p(0x50000), C.c_void_p(0x60000) if have else None,
                                 have, C.byref(p))
    assert rc == abi.OK, err()
    return p, need.value


def test_matmul_plan_of_the_benchmark_shapes():
    """The plan query answers without a GPU (pointers are only inspected) and names what the dispatcher does."""
    assert C.sizeof(abi.MatmulPlan) == 10 * 4 + 8
    # M=2048, K=4096, N=11008: 8 x 43 tiles of 256 x 256 = 344 = one full round of 256 + 88; the last 11 tile columns
    # (2816 columns of C) go to further workgroups of the same launch with 256 x 128 tiles
    p, _ = _plan(2048, 11008, 4096)
    assert (p.kernel, p.tile_m, p.tile_n, p.tile_k) == (abi.MM_KERNEL_DMA_256, 256, 256, 128)
    assert (p.workgroups, p.narrow_tile_n, p.narrow_workgroups, p.launches) == (256, 128, 176, 1)
    assert p.k_splits == 1 and p.workspace_bytes == 0 and p.lds_bytes == 2 * (256 * 128 * 2) + 1024
    # decode: weight streams, one per SIMD of 256 compute units, and a kernel that adds their pieces
    p, need = _plan(1, 11008, 4096)
    assert (p.kernel, p.tile_m, p.tile_n, p.tile_k) == (abi.MM_KERNEL_STREAM, 32, 128, 64)
    assert p.workgroups == 256 and p.launches == 2 and p.k_splits > 1 and p.workspace_bytes == need > 0
    # without the workspace the same call cannot run the streams: 128 x 128 tiles, no K split
    p, _ = _plan(1, 11008, 4096, ws=False)
    assert (p.kernel, p.k_splits, p.launches, p.workspace_bytes) == (abi.MM_KERNEL_DMA_128, 1, 1, 0)
    # M=128: 86 tiles of 128 x 128, K split 4 ways to put some 300 workgroups on the chip
    p, need = _plan(128, 11008, 4096)
    assert (p.kernel, p.tile_m, p.tile_n) == (abi.MM_KERNEL_DMA_128, 128, 128)
    assert (p.k_splits, p.workgroups, p.launches) == (4, 88 * 4, 2) and p.workspace_bytes == 4 * 128 * 11008 * 4
    # two or more row tiles cover most of the compute units by themselves: no split
    p, need = _plan(300, 11008, 4096)
    assert (p.kernel, p.k_splits, p.workgroups, p.launches, p.workspace_bytes) == (abi.MM_KERNEL_DMA_128, 1, 264, 1, 0)
    # B as [n, k] runs the same direct-to-LDS tiles at every m; a K that is no multiple of 128 the register-staged kernel
    p, _ = _plan(2048, 11008, 4096, trans_b=1)
    assert (p.kernel, p.tile_m, p.tile_n, p.narrow_tile_n, p.launches) == (abi.MM_KERNEL_DMA_256, 256, 256, 128, 1)
    p, _ = _plan(300, 11008, 4096, trans_b=1)
    assert (p.kernel, p.tile_m, p.tile_n, p.k_splits, p.launches) == (abi.MM_KERNEL_DMA_128, 128, 128, 1, 1)
    # 17 to 224 rows on [n, k] weights (k up to 4096): weights held in registers, activations streamed, no scratch
    p, need = _plan(100, 11008, 4096, trans_b=1)
    assert (p.kernel, p.k_splits, p.launches, p.workgroups) == (abi.MM_KERNEL_STREAM, 1, 1, 256)
    assert p.workspace_bytes == need == 0
    p, need = _plan(100, 11008, 8192, trans_b=1)
    assert (p.kernel, p.k_splits, p.launches) == (abi.MM_KERNEL_DMA_128, 4, 2) and p.workspace_bytes == need
    p, _ = _plan(300, 11008, 4096 + 64, trans_b=1)
    assert (p.kernel, p.launches) == (abi.MM_KERNEL_STAGED, 1)
    # odd addresses fall to the generic kernel
    p, _ = _plan(2048, 11008, 4096, a=0x10001)
    assert (p.kernel, p.launches) == (abi.MM_KERNEL_GENERIC, 1)
    # a rejected descriptor is rejected by the plan query as by the call
    d = abi.MatmulDesc(m=0, n=8, k=16, out_dtype=abi.I32)
    assert L.ascq_matmul_w8a8_plan(C.byref(d), FAKE, FAKE, FAKE, None, None, None, None, 0,
                                   C.byref(abi.MatmulPlan())) == abi.EINVAL
    assert L.ascq_matmul_w8a8_plan(C.byref(d), FAKE, FAKE, FAKE, None, None, None, None, 0, None) == abi.ENULL


def test_missing_library_is_a_loud_error_with_no_fallback(monkeypatch, tmp_path):
    """The package has no CPU path: without libascq.so the first call raises instead of computing something else."""
    monkeypatch.setattr(abi, "_lib", None)
    monkeypatch.setattr(abi, "LIB_PATH", str(tmp_path / "libascq.so"))
    with pytest.raises(RuntimeError, match="is missing"):
        abi.load_library()
    from ascq import ops
    with pytest.raises(RuntimeError, match="is missing"):
        ops.dequant_dst_stride("float16", 40)


def test_inline_assembly_kernels_have_no_scratch_frame():
    """The build records every kernel's register / scratch figures (asc-devkit_amd/csrc/check_resources.py).  Kernels
    that load through inline assembly and wait by hand must have no scratch frame and no spills: the compiler does not
    know that their destination registers are still being written."""
    import json
    path = os.path.join(ROOT, "asc-devkit_amd", "lib", "kernel_resources.json")
    assert os.path.exists(path), "build the library first (make -C asc-devkit_amd/csrc writes this file)"
    rec = json.load(open(path))
    guarded = [k for k in rec["kernels"] if k["guarded"]]
    seen = {k["name"].replace("void ", "").split("<")[0].split("(")[0] for k in guarded}
    for name in ("w4a16_gemv_kernel", "w4a16_tile_kernel", "w8a16_tile_kernel", "gemm_stream_kernel", "gemm_dma_kernel",
                 "gemm_dma_dual_kernel", "gemm_dma_group_kernel", "w4a16_packed_kernel"):
        assert name in seen, f"{name} is missing from the build record"
    assert set(rec["guarded_names"]) == seen, "a guarded name that matches no kernel guards nothing"
    for k in guarded:
        assert k["scratch_bytes_per_lane"] == 0 and k["vgpr_spills"] == 0, k   # scalar spills go to reserved lanes
        assert k["vgprs"] + k["agprs"] <= 512 and k["lds_bytes"] <= 160 * 1024, k


def test_resource_checker_rejects_a_guarded_kernel_with_scratch(tmp_path):
    import subprocess
    import sys
    remarks = tmp_path / "fake.remarks"
    lines = ["Function Name: _ZN4ascq12_GLOBAL__N_118gemm_stream_kernelENS0_12StreamParamsE", "    TotalSGPRs: 10",
             "    VGPRs: 256", "    AGPRs: 0", "    ScratchSize [bytes/lane]: 100", "    Occupancy [waves/SIMD]: 1",
             "    SGPRs Spill: 0", "    VGPRs Spill: 25", "    LDS Size [bytes/block]: 0"]
    remarks.write_text("".join(f"x.hip:1:1: remark: {l} [-Rpass-analysis=kernel-resource-usage]\n" for l in lines))
    r = subprocess.run([sys.executable, os.path.join(ROOT, "asc-devkit_amd", "csrc", "check_resources.py"), str(remarks)],
                       capture_output=True, text=True)
    assert r.returncode == 1 and "100 bytes of scratch" in r.stderr


def test_w4a16_packed_rejections_and_size():
    d = abi.W4A16Desc(m=1, n=64, k=256, group_size=128, has_offset=0)
    call = lambda d, y=FAKE, x=FAKE, w=FAKE, sc=FAKE, of=None: L.ascq_matmul_w4a16_packed(C.byref(d), y, x, w, sc, of, None)
    assert L.ascq_matmul_w4a16_packed(None, FAKE, FAKE, FAKE, FAKE, None, None) == abi.ENULL
    assert call(d, w=None) == abi.ENULL
    assert call(abi.W4A16Desc(m=1, n=64, k=256, group_size=128, has_offset=1)) == abi.ENULL       # offset missing
    assert call(abi.W4A16Desc(m=1, n=63, k=256, group_size=128, has_offset=0)) == abi.EINVAL
    assert call(abi.W4A16Desc(m=1, n=64, k=256, group_size=100, has_offset=0)) == abi.EINVAL      # k % group_size
    assert call(abi.W4A16Desc(m=1, n=64, k=160, group_size=32, has_offset=0)) == abi.EUNSUPPORTED  # k % 128
    assert call(abi.W4A16Desc(m=1, n=66, k=256, group_size=128, has_offset=0)) == abi.EUNSUPPORTED  # n % 8
    assert call(abi.W4A16Desc(m=1, n=64, k=384, group_size=96, has_offset=0)) == abi.EUNSUPPORTED  # 96 = 32 * 3
    assert call(d, x=C.c_void_p(0x1008)) == abi.EALIGN
    size = C.c_size_t(0)
    assert L.ascq_pack_weight_w4_size(8192, 28672, C.byref(size)) == abi.OK
    assert size.value == (28672 // 16 * (8192 // 128) + 16) * 1024               # slabs * tiles + 16 tiles of padding
    assert L.ascq_pack_weight_w4_size(100, 30, C.byref(size)) == abi.OK and size.value == (2 * 1 + 16) * 1024
    assert L.ascq_pack_weight_w4_size(128, 15, C.byref(size)) == abi.EINVAL
    assert L.ascq_pack_weight_w4(None, FAKE, 128, 16, None) == abi.ENULL


def test_noalloc_entry_point_rejects_before_touching_the_gpu():
    d = abi.MatmulDesc(m=32, n=11008, k=4096, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                       scale_format=abi.MM_SCALE_F32)
    rc = L.ascq_linear_w8a8_dynamic_noalloc(C.byref(d), abi.BF16, FAKE, FAKE, FAKE, None, FAKE, None)
    assert rc == abi.EINVAL and "built-in buffer" in err()
    assert L.ascq_linear_w8a8_dynamic_noalloc(None, abi.BF16, FAKE, FAKE, FAKE, None, FAKE, None) == abi.ENULL


def test_integration_snippet_matches_the_abi():
    """The ctypes struct printed in the integration notes has the fields of the struct the library reads."""
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = text[text.index("class QuantDesc(C.Structure)"):]
    block = block[:block.index("lib.ascq_quant.restype")]
    fields = re.findall(r'\("([a-z_]+)", C\.(c_[a-z0-9]+)\)', block)
    # compare names and the ctypes types themselves (c_int32 is an alias of c_int on this platform)
    got = [(n, getattr(C, t)) for n, t in fields]
    assert got == list(abi.QuantDesc._fields_), (got, abi.QuantDesc._fields_)


def test_combined_policies_are_rejected_by_name():
    FAKE2 = C.c_void_p(0x100000)
    for pol in (abi.PER_CHANNEL_PER_GROUP, abi.PER_TOKEN_PER_GROUP):
        assert L.ascq_quant(C.byref(q(policy=pol)), FAKE, FAKE2, FAKE, FAKE, None) == abi.EUNSUPPORTED
        assert "PER_CHANNEL_PER_GROUP" in err()
        dq = abi.DequantDesc(policy=pol, src_dtype=abi.I32, scale_dtype=abi.F32, dst_dtype=abi.F32, m=4, n=8, cal_count=32,
                             group_size=8)
        assert L.ascq_dequant(C.byref(dq), FAKE, FAKE2, FAKE, None) == abi.EUNSUPPORTED
        aq = abi.AntiQuantPolicyDesc(policy=pol, dst_dtype=abi.F16, scale_dtype=abi.F16, m=4, n=32, cal_count=128,
                                     group_size=8)
        assert L.ascq_antiquant_policy(C.byref(aq), FAKE, FAKE2, FAKE, None, None) == abi.EUNSUPPORTED
    assert L.ascq_quant(C.byref(q(policy=6)), FAKE, FAKE2, FAKE, FAKE, None) == abi.EINVAL
    from ascq import ops
    assert ops.AscendDeQuantPolicy.TO_ABI[ops.AscendDeQuantPolicy.PER_TOKEN] == abi.PER_TOKEN
    assert ops.AscendDeQuantPolicy.PER_TOKEN == 0 and ops.AscendDeQuantPolicy.PER_TOKEN_PER_GROUP == 3


def test_hifloat8_surface_and_refused_round_modes():
    """hifloat8 is a destination of ascq_quant and a source of ascq_antiquant_policy; CAST_HYBRID and CAST_ODD have
    the reference's values (kernel_utils_mode.h:94-109) and are refused by name; format 6 does not exist."""
    FAKE2 = C.c_void_p(0x100000)
    assert (abi.CAST_ODD, abi.CAST_HYBRID, abi.QDST_HIF8) == (6, 7, 5)
    for mode in (abi.CAST_ODD, abi.CAST_HYBRID):
        assert L.ascq_quant(C.byref(q(round_mode=mode, dst_format=abi.QDST_HIF8)), FAKE, FAKE2, FAKE, FAKE, None) == abi.EUNSUPPORTED
        assert "CAST_HYBRID" in err()
    assert L.ascq_quant(C.byref(q(dst_format=6)), FAKE, FAKE2, FAKE, FAKE, None) == abi.EUNSUPPORTED and "hifloat8" in err()
    aq = abi.AntiQuantPolicyDesc(policy=abi.PER_TOKEN, src_format=6, dst_dtype=abi.F16, scale_dtype=abi.F16, m=4, n=32,
                                 cal_count=128)
    assert L.ascq_antiquant_policy(C.byref(aq), FAKE, FAKE2, FAKE, None, None) == abi.EUNSUPPORTED and "hifloat8" in err()
    hdr = open(os.path.join(ROOT, "include", "ascq.h")).read()
    assert "ASCQ_QDST_HIF8 = 5" in hdr and "ASCQ_CAST_HYBRID = 7" in hdr


def test_w8a16_transposed_weights_surface():
    """[n, k] weights: no workspace at any k (a k off the kernels' 128-element steps runs the one-lane-per-output
    kernel, which needs none either); the descriptor carries trans_b as its last field."""
    assert C.sizeof(abi.W8A16Desc) == 10 * 4 and abi.W8A16Desc._fields_[-2][0] == "trans_b"
    assert abi.W8A16Desc._fields_[-1][0] == "mode" and (abi.W8A16_PER_WEIGHT, abi.W8A16_CHANNEL_SUM) == (0, 1)
    need = C.c_size_t(77)
    d = abi.W8A16Desc(m=4, n=64, k=256, per_tensor=1, scale=0.5, out_dtype=abi.F16, trans_b=1)
    assert L.ascq_matmul_w8a16_workspace_size(C.byref(d), C.byref(need)) == abi.OK and need.value == 0
    d.k = 192
    need.value = 77
    assert L.ascq_matmul_w8a16_workspace_size(C.byref(d), C.byref(need)) == abi.OK and need.value == 0


def test_quant_word_with_pre_shift_bit_passes_validation():
    """The mode-control bit 36 of a quant word (pre-shift by bits [35:32]) is part of the supported domain: the
    descriptor is accepted (the call then fails on the NULL output, which is checked after the descriptor)."""
    d = abi.MatmulDesc(m=16, n=32, k=64, out_dtype=abi.F16, quant_mode=abi.MM_QUANT_SCALAR, scale_format=abi.MM_SCALE_U64,
                       quant_scalar=(1 << 36) | (3 << 32) | (0x3F800000 & 0xFFFFE000))
    rc = L.ascq_matmul_w8a8(C.byref(d), None, FAKE, FAKE, None, None, None, None, 0, None)
    assert rc == abi.ENULL and "bit 36" not in err()


def test_linear_dynamic_packed_argument_checks():
    """ascq_linear_w8a8_dynamic_packed refuses what the packed layout cannot serve before anything is launched, and its
    scratch need is covered by ascq_linear_w8a8_dynamic_workspace_size."""
    def d(**kw):
        x = abi.MatmulDesc(m=4, n=64, k=128, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR, scale_format=abi.MM_SCALE_F32)
        for key, v in kw.items():
            setattr(x, key, v)
        return x
    big = C.c_void_p(0x200000)
    call = lambda x, dt=abi.BF16, ws=big, nbytes=1 << 20: L.ascq_linear_w8a8_dynamic_packed(
        C.byref(x), dt, FAKE, FAKE, FAKE, None, FAKE, ws, nbytes, None)
    assert L.ascq_linear_w8a8_dynamic_packed(None, abi.BF16, FAKE, FAKE, FAKE, None, FAKE, big, 1 << 20, None) == abi.ENULL
    assert call(d(), dt=abi.I8) == abi.EUNSUPPORTED and "x dtype" in err()
    assert call(d(k=100)) == abi.EUNSUPPORTED and "multiple of 64" in err()
    assert call(d(trans_a=1)) == abi.EUNSUPPORTED
    assert call(d(activation=abi.MM_ACT_SWIGLU, n=63)) == abi.EINVAL and "must be even" in err()   # SwiGLU pairs columns
    assert call(d(quant_mode=abi.MM_QUANT_NONE)) == abi.EUNSUPPORTED
    assert call(d(out_dtype=abi.I8)) == abi.EUNSUPPORTED
    assert call(d(), ws=None) == abi.ENULL
    assert call(d(), ws=C.c_void_p(0x200004)) == abi.EALIGN
    assert call(d(), nbytes=256) == abi.EINVAL and "workspace" in err()
    need = C.c_size_t(0)
    assert L.ascq_linear_w8a8_dynamic_workspace_size(C.byref(d()), C.byref(need)) == abi.OK
    assert need.value >= 4 * 128 + 4 * 4


def test_tmp_buffer_factor_sizes_known_answers():
    """tests/api/adv_api/tiling/test_tiling.cpp:6549-6553, 6565-6569, 6583-6608, 6621-6625, 6643-6647, 6662-6666,
    6684-6688 of the reference."""
    U = C.c_uint32
    live, extra = U(9), U(9)
    assert L.ascq_get_ascend_quant_tmp_buffer_factor_size(C.byref(live), C.byref(extra)) == abi.OK
    assert (live.value, extra.value) == (2, 0)
    shape = (U * 2)(10, 32)
    assert L.ascq_get_ascend_dequant_tmp_buffer_factor_size(shape, 2, C.byref(live), C.byref(extra)) == abi.OK
    assert (live.value, extra.value) == (1, 104)
    shape1 = (U * 1)(320)
    assert L.ascq_get_ascend_dequant_tmp_buffer_factor_size(shape1, 1, C.byref(live), C.byref(extra)) == abi.OK
    assert (live.value, extra.value) == (2, 72)
    shape3 = (U * 3)(2, 3, 4)
    assert L.ascq_get_ascend_dequant_tmp_buffer_factor_size(shape3, 3, C.byref(live), C.byref(extra)) == abi.OK
    assert (live.value, extra.value) == (0, 0)

    def aq(src, scale, transpose, out):
        s, c = (U * len(src))(*src), (U * len(scale))(*scale)
        assert L.ascq_get_ascend_antiquant_tmp_buffer_factor_size(s, len(src), c, len(scale), int(transpose), 0, out,
                                                                  C.byref(live), C.byref(extra)) == abi.OK
        return live.value, extra.value
    assert aq((640, 5120), (1, 5120), False, abi.F16) == (0, 0)
    assert aq((640, 5120), (1, 5120), False, abi.BF16) == (0, 5120 * 2 * 4 + 64 * 640 * 4)
    assert aq((640, 5120), (1,), False, abi.BF16) == (1, 0)
    assert aq((64, 512), (64, 1), True, abi.BF16) == (0, 80 * 64 * 4)
    assert aq((640, 5120), (1,), True, abi.BF16) == (1, 0)


def test_swiglu_rejections_and_workspace():
    mk = lambda **kw: abi.MatmulDesc(**{**dict(m=16, n=64, k=128, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                                               scale_format=abi.MM_SCALE_F32, activation=abi.MM_ACT_SWIGLU, act_beta=1.0), **kw})
    call = lambda d, ws=None, nb=0: L.ascq_matmul_w8a8(C.byref(d), FAKE, FAKE, FAKE, None, FAKE, None, ws, nb, None)
    assert call(mk(n=63)) == abi.EINVAL and "even" in err()
    assert call(mk(out_dtype=abi.I8, scale_format=abi.MM_SCALE_U64)) == abi.EUNSUPPORTED
    assert call(mk(quant_mode=abi.MM_QUANT_NONE, out_dtype=abi.I32)) == abi.EUNSUPPORTED
    assert call(mk(act_beta=float("inf"))) == abi.EINVAL
    assert call(mk(activation=3)) == abi.EINVAL
    need = C.c_size_t(0)
    assert L.ascq_matmul_w8a8_workspace_size(C.byref(mk()), C.byref(need)) == abi.OK
    assert need.value >= 16 * 64 * 4                                  # the int32 accumulators of the pairwise epilogue
    assert call(mk()) == abi.EINVAL and "workspace" in err()          # small m: not the large tile kernel


def test_mx_matmul_surface_without_a_gpu():
    """Descriptor checks and the workspace rule of the block-scaled matmul answer on the host."""
    lib = abi.load_library()
    need = C.c_size_t(7)
    e4, e5, f2, f1 = abi.QDST_FP8_E4M3FN, abi.QDST_FP8_E5M2, abi.QDST_FP4_E2M1, abi.QDST_FP4_E1M2
    mk = lambda **kw: abi.MxDesc(**{**dict(m=512, n=512, k=1024, scale_k=32, a_format=e4, b_format=e5,
                                           out_dtype=abi.BF16, has_bias=0), **kw})
    for d, want in [(mk(), 0), (mk(a_format=f2, b_format=f2), 0),                      # straight from the given buffers
                    (mk(a_format=f1, b_format=f1), 2 * 512 * 1024),                    # e1m2: both widened to e4m3
                    (mk(a_format=f2), 512 * 1024),                                     # 4-bit beside 8-bit: a widened
                    (mk(a_format=f1, k=70, scale_k=4), 0)]:                            # one lane per output: no scratch
        assert lib.ascq_matmul_mx_workspace_size(C.byref(d), C.byref(need)) == abi.OK and need.value == want
    for d, msg in [(mk(k=63, a_format=f2), "even"), (mk(scale_k=31), "scale_k"), (mk(a_format=abi.QDST_I8), "a_format"),
                   (mk(out_dtype=abi.I8), "out_dtype"), (mk(m=0), "greater than 0")]:
        assert lib.ascq_matmul_mx_workspace_size(C.byref(d), C.byref(need)) == abi.EINVAL
        assert msg in lib.ascq_last_error().decode()
    assert lib.ascq_matmul_mx(C.byref(mk()), None, None, None, None, None, None, None, 0, None) == abi.ENULL
