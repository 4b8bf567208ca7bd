#!/usr/bin/env python3
"""Benchmark of the quantized-inference hot path on one MI355X.

Headline (the `value` of the JSON line): the W8A8 LLM linear at M=2048, K=4096, N=11008 - one step = dynamic
per-token quantisation of the bf16 activations + the int8 MFMA GEMM with the fused dequant epilogue to bf16 - reported
as int8 TOPS (2*M*K*N per step).  The same line carries the roofline of the dominant kernel (the GEMM, timed alone with
events on the launch stream), the CPU baseline (the oracle, timed on the host cores), the W4A16 decode GEMV as HBM GB/s
and, unless --quick, the other workloads of the path (elementwise ops, small-M linears, W4A16 M=4/16, the MoE grouped
matmul) under "others".

Inputs are synthetic, seeded and resident in HBM before the timed region.  Memory-bound workloads rotate among
several buffer sets larger than the 256 MB Infinity Cache so that their input is read from HBM every iteration.

The default of 1000 timed steps after 100 warm-up steps keeps the GPU busy for about 0.1 s.  After an idle period the
clocks take a few milliseconds of load to reach their sustained state: a 50-step region (6 ms) measured 124 us per
step and 108 us per GEMM, a 1000-step region 102-106 us per step and 95 us per GEMM, on the same box minutes apart.
For the same reason `--settle` untimed steps (300, about 30 ms; reported as config.settle_steps) run before the W
warm-up steps of every workload, the headline and the others alike, so that a caller's short --steps/--warmup is
measured at the sustained clock as well; the workloads under "others" time at least 100 steps.

Besides the workloads the line carries "ceilings": the figures the stand-alone program asc-devkit_amd/lib/machine_probe
measures on this GPU in the same run (matrix-pipe rate with constant and with random int8 operands and the shader clock
during each, HBM copy / read / fill, LDS read rate), and "roofline.same_kernel_zero_operands": the headline GEMM
launched on all-zero operands, which shows what the same instruction stream reaches when the operands do not toggle
the multipliers (the power management then leaves the clock at its maximum).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "asc-devkit_amd"), os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

# MI355X published peaks (dense int8 matrix TOP/s, HBM3E GB/s, dense f16 matrix TFLOP/s): peaks.json beside this file
# holds them together with the ceilings measured on the machine
with open(os.path.join(ROOT, "peaks.json")) as _f:
    _PEAKS = json.load(_f)["published"]
PEAK_INT8_TOPS = float(_PEAKS["int8_dense_tops"])
PEAK_HBM_GBS = float(_PEAKS["hbm_gbs"])
PEAK_F16_TFLOPS = float(_PEAKS["f16_dense_tflops"])
PEAK_FP8_TFLOPS = float(_PEAKS["fp8_dense_tflops"])
PEAK_FP4_TFLOPS = float(_PEAKS["fp4_dense_tflops"])
# Bytes that left / entered the L2 caches per launch, from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of
# `bench.py --quick --no-cpu --copy-probe`; each counter is scaled by its reading for the 1 GiB copy of the same run
# (FETCH_SIZE reads 0.5 per KiB there, WRITE_SIZE 1.0 per KiB).  Measured offline and recorded here; a run of this
# file does not re-measure them.
GEMM_TRAFFIC_BYTES = 228293837   # M=2048 GEMM, both tile shapes: 183.2 MB fetched + 45.1 MB written
GEMV_TRAFFIC_BYTES = 133853594   # W4A16 M=1 GEMV, [k, n / 2] layout, stream + sum kernels: 129.5 MB fetched + 4.3 MB written
GEMV_PACKED_TRAFFIC_BYTES = 125_108_224   # the same on packed weights in the group-sum mode, one launch: 125.05 MB fetched + 0.06 MB written (profiles/w4a16_packed_group_sum_gemv_m1_trace_and_counters.md)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--settle", type=int, default=300,
                    help="untimed steps of the headline workload before its warm-up, so that short --steps/--warmup "
                         "runs are also measured at the sustained clock (0 disables)")
    ap.add_argument("--quick", action="store_true", help="headline + W4A16 GEMV only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="", help="run a single workload: w8a8 | w4a16 | w4a16_per_weight | w4a16_per_weight_m4 | w4a16_per_weight_m16 | w4a16_nd | w4a16_m4 | w4a16_m16 | w4a16_nd_m4 | w4a16_nd_m16 | "
                         "w8a8_zeros | w8a8_m1 | w8a8_m8 | w8a8_m16 | w8a8_m128 | w8a8_m512 | w8a8_m8192 | w8a8_packed_m1 | w8a8_packed_m8 | w8a8_packed_m16 | w8a8_packed_m32 | w8a8_packed_m64 | w8a8_packed_m128 | w8a8_packed_down_m16 | w8a8_packed_down_m64 | w8a8_nk_down_m16 | w8a8_nk_m32 | w8a8_nk_m64 | w8a8_m32 | w8a8_nk_m1 | w8a8_nk_m16 | w8a8_nk_m128 | w8a8_linear_nk_m1 | w8a8_linear_nk_m4 | w8a8_linear_nk_m16 | w8a8_linear_packed_m1 | w8a8_linear_packed_m4 | w8a8_linear_packed_swiglu_m1 | w8a8_linear_nk_swiglu_m1 | w8a8_decode_layer_packed_m1 | w8a8_decode_layer_packed_m4 | w8a8_decode_layer_packed_m16 | w8a8_decode_layer_nk_m1 | w8a16_m1 | w8a16_m16 | w8a16_nk_m1 | w8a16_nk_m4 | w8a16_nk_sum_m1 | w8a16_nk_sum_m4 | "
                         "w8a16_nk_m16 | w8a16_m2048 | w8a16_nk_m2048 | quant | dequant | antiquant | group | group_example | mx_fp4 | mx_fp4_e1m2 | mx_fp8 (a W4A16 name without _nd "
                         "is the packed-weight path, in the group-sum form unless it says per_weight; _nk: weights kept as [n, k])")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one device-to-device copy of 1 GiB: the known-size kernel that calibrates the "
                         "FETCH_SIZE / WRITE_SIZE counters when this command runs under rocprofv3 --pmc")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU; run it with --gpus 1 (the path shards over output columns, rows "
              "or experts without any communication, so N GPUs are N independent copies of this run).",
              file=sys.stderr)
        sys.exit(2)

    # The stand-alone probe of the machine's ceilings runs first, in a process of its own, before this process has
    # touched the GPU.
    ceilings = None
    if not (args.quick or args.only):
        import subprocess
        exe = os.path.join(ROOT, "asc-devkit_amd", "lib", "machine_probe")
        if not os.path.exists(exe):
            ceilings = {"error": "asc-devkit_amd/lib/machine_probe is not built"}
        else:
            try:
                r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
                ceilings = json.loads(r.stdout) if r.returncode == 0 else {"error": r.stderr.strip()[-200:]}
            except Exception as e:     # the probe is evidence, not part of the measurement: report and go on
                ceilings = {"error": str(e)}

    import numpy as np
    import torch
    from ascq import _abi as abi
    from ascq import ops

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = "cuda:0"
    torch.cuda.set_device(0)
    abi.load_library()           # fail loudly if the HIP library is missing
    gen = torch.Generator(device=dev)
    gen.manual_seed(0xA5C0)

    def rand_i8(*shape):
        return torch.randint(-127, 128, shape, dtype=torch.int8, device=dev, generator=gen)

    def timed(fn, steps, warmup, settle=None):
        """Times `steps` calls of fn(i, None, None) after `settle` + `warmup` untimed ones by the host clock between two
        synchronizes, then the same `steps` calls again between one pair of events on the launch stream.  Returns (ms
        per step by the host clock, ms per step by the events).  No event is recorded inside either region: a record
        between two launches idles the queue for 3-6 us, which is a tenth of a 35 us decode step."""
        for i in range(args.settle if settle is None else settle):
            fn(i, None, None)
        for i in range(warmup):
            fn(i, None, None)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            fn(warmup + i, None, None)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for i in range(steps):
            fn(warmup + i, None, None)
        ev1.record()
        torch.cuda.synchronize()
        return wall_ms, ev0.elapsed_time(ev1) / steps

    def bracket(starts, stops, call):
        if starts is None:
            call()
            return
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        call()
        b.record()
        starts.append(a)
        stops.append(b)

    if args.copy_probe:
        a = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        b = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        b.copy_(a)
        torch.cuda.synchronize()
        del a, b
        torch.cuda.empty_cache()

    # ------------------------------------------------------------------ W8A8 linear (config 3)
    def w8a8(M, steps, warmup, sets=1, settle=None, zero=False, gauss=False, b_nk=False, packed=False,
             shape=(4096, 11008)):
        """`sets` > 1 rotates the weights over several copies (together larger than the Infinity Cache) so that the
        weight-bound small-M cases read them from HBM.  The weights are uniform over [-127, 127] unless `gauss`: then
        they are normal weights quantised per output channel by their absolute maximum, as a checkpoint's would be.
        b_nk: the weights are kept as [n, k] (isTransposeB).  packed: the weights in the layout of ascq_pack_weight_w8
        (packed once, outside the timed region) and the one-launch kernel for few rows.  shape: (K, N), by default the
        up projection's; (11008, 4096) is the down projection of the same layer."""
        K, N = shape
        x = torch.randn((M, K), device=dev, generator=gen).to(torch.bfloat16)
        if gauss:
            ws = []
            for _ in range(sets):
                wf = torch.randn((K, N), device=dev, generator=gen)
                ws.append(torch.round(wf / wf.abs().amax(dim=0, keepdim=True) * 127).clamp(-127, 127).to(torch.int8))
                del wf
        else:
            ws = [rand_i8(N, K) if b_nk else rand_i8(K, N) for _ in range(sets)]
        if zero:          # all-zero activations and weights: the same launches, nothing toggles in the multipliers
            x.zero_()
            for wj in ws:
                wj.zero_()
        w = ws[0]
        cs = torch.rand(N, device=dev, generator=gen) * (1e-2 - 1e-4) + 1e-4
        q = torch.empty((M, K), dtype=torch.int8, device=dev)
        ts = torch.empty(M, dtype=torch.float32, device=dev)
        c = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        mms = []
        for wj in ws:
            mm = ops.Matmul(M, N, K, False, b_nk and not packed)
            mm.set_tensor_a(q)
            if packed:
                mm.set_tensor_b_packed(ops.pack_weight_w8(wj, K, N, b_nk))
            else:
                mm.set_tensor_b(wj)
            mm.set_quant_vector(cs)
            mm.set_token_scale(ts)
            mms.append(mm)

        def step(i, starts, stops):
            ops.dynamic_quant_per_token(x, q, ts)
            bracket(starts, stops, lambda: mms[i % sets].iterate_all(c))

        # The timed region proper is quant + GEMM per step.  Then the GEMM launches of the same steps run back to
        # back between one pair of events on the launch stream, which gives the average duration of the GEMM launch.
        ms, _ = timed(lambda i, a, b: step(i, None, None), steps, warmup, settle)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        ev0.record()
        for i in range(steps):
            mms[i % sets].iterate_all(c)
        ev1.record()
        torch.cuda.synchronize()
        kern_ms = ev0.elapsed_time(ev1) / steps
        # the same launches once more in blocks of 20, one pair of events per block: median and minimum over blocks
        blocks = []
        for b0 in range(0, steps - steps % 20, 20):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(b0, b0 + 20):
                mms[i % sets].iterate_all(c)
            e1.record()
            blocks.append((e0, e1))
        torch.cuda.synchronize()
        per_block = sorted(e0.elapsed_time(e1) / 20 for e0, e1 in blocks)
        flops = 2.0 * M * K * N
        bytes_ = M * K + K * N + 4 * N + 4 * M + 2 * M * N
        return {"ms_per_step": ms, "gemm_kernel_ms": kern_ms, "tops": flops / (ms * 1e-3) / 1e12,
                "gemm_kernel_ms_median": per_block[len(per_block) // 2] if per_block else None,
                "gemm_kernel_ms_min": per_block[0] if per_block else None,
                "gemm_tops": flops / (kern_ms * 1e-3) / 1e12, "gemm_gbs": bytes_ / (kern_ms * 1e-3) / 1e9,
                "ops": flops, "bytes": bytes_, "tensors": (x, w, cs)}

    def w8a8_linear(M, steps, warmup, sets=7, packed=False, swiglu=False):
        """The whole W8A8 linear as one call on weights kept as [n, k] (ascq_linear_w8a8_dynamic) or packed once
        (ascq_linear_w8a8_dynamic_packed): up to 8 rows the per-token quantisation happens inside the weight-streaming
        kernel, one launch per step."""
        K, N = 4096, 11008
        x = torch.randn((M, K), device=dev, generator=gen).to(torch.bfloat16)
        ws = [rand_i8(N, K) for _ in range(sets)]
        cs = torch.rand(N, device=dev, generator=gen) * (1e-2 - 1e-4) + 1e-4
        act = abi.MM_ACT_SWIGLU if swiglu else abi.MM_ACT_NONE   # SwiGLU: column pairs -> [M, N / 2]
        c = torch.empty((M, N // 2 if swiglu else N), dtype=torch.bfloat16, device=dev)
        if packed:
            lins = [ops.DynamicLinear(M, K, ops.pack_weight_w8(w, K, N, True), cs, packed_n=N, activation=act) for w in ws]
        else:
            lins = [ops.DynamicLinear(M, K, w, cs, trans_b=True, activation=act) for w in ws]
        ms, kern_ms = timed(lambda i, a, b: lins[i % sets](c, x), steps, warmup)
        bytes_ = 2 * M * K + K * N + 4 * N + 2 * M * N
        return {"ms_per_step": ms, "kernel_ms": kern_ms, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9, "bytes": bytes_,
                "tops": 2.0 * M * K * N / (kern_ms * 1e-3) / 1e12, "tensors": (x, ws[0], cs)}

    def w8a8_decode_layer(M, steps, warmup, sets=2, packed=True):
        """The four W8A8 linears of one decoder layer (hidden 4096, feed-forward 11008) at M rows, one call each: QKV
        (4096 -> 12288), attention output (4096 -> 4096), gate / up with SwiGLU (4096 -> 2 x 11008 -> 11008) and down
        (11008 -> 4096), the last one on the output of the one before.  The attention between the first two is not part
        of this library: its output is a fixed random tensor.  The 202 MB of weights rotate over `sets` copies."""
        H, F = 4096, 11008
        x = torch.randn((M, H), device=dev, generator=gen).to(torch.bfloat16)
        attn = torch.randn((M, H), device=dev, generator=gen).to(torch.bfloat16)
        qkv = torch.empty((M, 3 * H), dtype=torch.bfloat16, device=dev)
        h = torch.empty((M, H), dtype=torch.bfloat16, device=dev)
        g = torch.empty((M, F), dtype=torch.bfloat16, device=dev)
        y = torch.empty((M, H), dtype=torch.bfloat16, device=dev)
        plan = (("qkv", H, 3 * H, abi.MM_ACT_NONE), ("o", H, H, abi.MM_ACT_NONE), ("gate_up", H, 2 * F, abi.MM_ACT_SWIGLU),
                ("down", F, H, abi.MM_ACT_NONE))
        layers = []
        for _ in range(sets):
            lin = {}
            for name, K, N, act in plan:
                w = rand_i8(N, K)
                cs = torch.rand(N, device=dev, generator=gen) * (2e-4 - 1e-4) + 1e-4
                if packed:
                    lin[name] = ops.DynamicLinear(M, K, ops.pack_weight_w8(w, K, N, True), cs, packed_n=N, activation=act)
                    del w
                else:
                    lin[name] = ops.DynamicLinear(M, K, w, cs, trans_b=True, activation=act)
            layers.append(lin)

        def step(i, starts, stops):
            lin = layers[i % sets]
            lin["qkv"](qkv, x)
            lin["o"](h, attn)
            lin["gate_up"](g, h)
            lin["down"](y, g)

        ms, kern_ms = timed(step, steps, warmup)
        bytes_ = sum(K * N + 4 * N + 2 * M * K + 2 * M * (N // 2 if act == abi.MM_ACT_SWIGLU else N) for _, K, N, act in plan)
        return {"ms_per_step": ms, "kernel_ms": kern_ms, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9, "bytes": bytes_,
                "launches": 4 if M <= 8 else None, "tensors": (x, attn)}

    # ------------------------------------------------------------------ W4A16 decode (config 4)
    def w4a16(M, steps, warmup, sets=4, packed=False, mode=abi.W4A16_PER_WEIGHT):
        """packed: the weights in the layout of ascq_pack_weight_w4 (packed once, outside the timed region) and the
        one-launch kernel; otherwise the [k, n / 2] layout and the stream + sum kernels.  mode (packed only):
        abi.W4A16_PER_WEIGHT = AscendAntiQuant's two roundings to half per weight, abi.W4A16_GROUP_SUM = scale and offset
        applied once per quantisation group to fp32 sums."""
        K, N, gs = 8192, 28672, 128
        xs = torch.randn((M, K), device=dev, generator=gen).to(torch.float16)
        ws = [torch.randint(0, 256, (K, N // 2), dtype=torch.uint8, device=dev, generator=gen) for _ in range(sets)]
        sc = [(torch.rand((K // gs, N), device=dev, generator=gen) * 9e-3 + 1e-3).to(torch.float16) for _ in range(sets)]
        of = [torch.randint(-8, 8, (K // gs, N), device=dev, generator=gen).to(torch.float16) for _ in range(sets)]
        y = torch.empty((M, N), dtype=torch.float16, device=dev)
        wps = [ops.pack_weight_w4(w, K, N) for w in ws] if packed else None

        def step(i, starts, stops):
            j = i % sets
            if packed:
                bracket(starts, stops, lambda: ops.matmul_w4a16_packed(y, xs, wps[j], sc[j], of[j], gs, mode=mode))
            else:
                bracket(starts, stops, lambda: ops.matmul_w4a16(y, xs, ws[j], sc[j], of[j], gs))

        ms, kern_ms = timed(step, steps, warmup)
        bytes_ = K * N // 2 + 2 * (K // gs) * N * 2 + M * K * 2 + M * N * 2
        return {"ms_per_step": ms, "kernel_ms": kern_ms, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9, "bytes": bytes_,
                "tops": 2.0 * M * K * N / (kern_ms * 1e-3) / 1e12, "tensors": (xs, ws[0], sc[0], of[0])}

    # ------------------------------------------------------------------ W8A16 decode (Matmul anti-quant path)
    def w8a16(M, steps, warmup, sets=3, b_nk=False, mode=abi.W8A16_PER_WEIGHT):
        K, N = 8192, 28672
        xs = torch.randn((M, K), device=dev, generator=gen).to(torch.float16)
        ws = [rand_i8(N, K) if b_nk else rand_i8(K, N) for _ in range(sets)]
        sc = [(torch.rand((N,), device=dev, generator=gen) * 9e-3 + 1e-3).to(torch.float16) for _ in range(sets)]
        of = [(torch.rand((N,), device=dev, generator=gen) * 18 - 9).to(torch.float16) for _ in range(sets)]
        y = torch.empty((M, N), dtype=torch.float16, device=dev)

        def step(i, starts, stops):
            j = i % sets
            bracket(starts, stops, lambda: ops.matmul_w8a16(y, xs, ws[j], of[j], sc[j], trans_b=b_nk, mode=mode))

        ms, kern_ms = timed(step, steps, warmup, settle=min(args.settle, 300 if M <= 64 else 20))
        bytes_ = K * N + 2 * N * 2 + M * K * 2 + M * N * 2
        return {"ms_per_step": ms, "kernel_ms": kern_ms, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9, "bytes": bytes_,
                "tflops": 2.0 * M * K * N / (kern_ms * 1e-3) / 1e12}

    # ------------------------------------------------------------------ elementwise (config 2)
    def quant2a(steps, warmup, sets=3):
        m, n = 8192, 4096
        xs = [(torch.randn((m, n), device=dev, generator=gen) * 2).to(torch.float16) for _ in range(sets)]
        ss = [(127.0 / x.float().abs().amax(dim=0)).to(torch.float16) for x in xs]
        dst = [torch.empty((m, n), dtype=torch.int8, device=dev) for _ in range(sets)]

        def step(i, starts, stops):
            j = i % sets
            bracket(starts, stops, lambda: ops.ascend_quant(dst[j], xs[j], ss[j], 0.0))

        ms, kern_ms = timed(step, steps, warmup)
        bytes_ = m * n * 3 + n * 2
        return {"kernel_ms": kern_ms, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9, "bytes": bytes_, "tensors": (xs[0], ss[0])}

    def dequant2b(steps, warmup, sets=2):
        m, n = 8192, 4096
        src = [torch.randint(-2**20, 2**20 + 1, (m, n), dtype=torch.int32, device=dev, generator=gen) for _ in range(sets)]
        sc = torch.rand(n, device=dev, generator=gen) * (1e-3 - 1e-5) + 1e-5
        dst = [torch.empty((m, n), dtype=torch.bfloat16, device=dev) for _ in range(sets)]
        prm = ops.DequantParams(m, n, n)

        def step(i, starts, stops):
            j = i % sets
            bracket(starts, stops, lambda: ops.ascend_dequant(dst[j], src[j], sc, prm, abi.DEQUANT_WITH_MULTI_ROW))

        ms, kern_ms = timed(step, steps, warmup)
        bytes_ = m * n * 6 + n * 4
        return {"kernel_ms": kern_ms, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9, "bytes": bytes_}

    def antiquant2c(steps, warmup, sets=3):
        k, n = 4096, 11008
        w = [rand_i8(k, n) for _ in range(sets)]
        sc = (torch.rand((1, n), device=dev, generator=gen) * (1e-1 - 1e-3) + 1e-3).to(torch.float16)
        of = torch.randint(-8, 9, (1, n), device=dev, generator=gen).to(torch.float16)
        dst = [torch.empty((k, n), dtype=torch.float16, device=dev) for _ in range(sets)]
        info = ops.AntiQuantShapeInfo(1, n, 1, n)

        def step(i, starts, stops):
            j = i % sets
            bracket(starts, stops, lambda: ops.ascend_antiquant(dst[j], w[j], of, sc, k, info))

        ms, kern_ms = timed(step, steps, warmup)
        bytes_ = k * n * 3 + 2 * n * 2
        return {"kernel_ms": kern_ms, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9, "bytes": bytes_}

    # ------------------------------------------------------------------ grouped matmul (config 5)
    def group5(steps, warmup):
        G, T, K, N = 8, 4096, 4096, 14336
        rng = np.random.default_rng(0xC5)
        counts = rng.multinomial(T, [1.0 / G] * G)
        gl = torch.from_numpy(np.cumsum(counts).astype(np.int64)).to(dev)
        x = rand_i8(T, K)
        w = rand_i8(G, K, N)
        cs = torch.rand((G, N), device=dev, generator=gen) * (1e-2 - 1e-4) + 1e-4
        ts = torch.rand(T, device=dev, generator=gen) * (1e-1 - 1e-3) + 1e-3
        bias = torch.randn((G, N), device=dev, generator=gen).to(torch.bfloat16)
        y = torch.empty((T, N), dtype=torch.bfloat16, device=dev)

        def step(i, starts, stops):
            bracket(starts, stops, lambda: ops.quant_group_matmul(y, x, w, gl, cs, ts, bias, abi.GROUP_LIST_PREFIX_SUM))

        ms, kern_ms = timed(step, steps, warmup)
        flops = 2.0 * T * K * N
        bytes_ = T * K + G * K * N + G * N * 4 + T * 4 + G * N * 2 + T * N * 2 + G * 8
        return {"kernel_ms": kern_ms, "tops": flops / (kern_ms * 1e-3) / 1e12, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9,
                "ops": flops, "bytes": bytes_}

    def group_example(steps, warmup):
        """The reference example's own shape and options (quant_group_matmul_high_performance: 8 groups x 1024 tokens,
        k = 1024, n = 8192, weights in the fractal NZ layout, FasterGelu, fp16 output; data as its gen_data.py draws
        them).  Its README reports 204.129 us and mac_ratio 0.887 on an Ascend 950PR (context only)."""
        G, T, K, N = 8, 8192, 1024, 8192
        gl = torch.full((G,), T // G, dtype=torch.int64, device=dev)
        x = torch.randint(-10, 10, (T, K), dtype=torch.int8, device=dev, generator=gen)
        w = ops.pack_weight_nz(torch.randint(-10, 10, (G, K, N), dtype=torch.int8, device=dev, generator=gen))
        cs = torch.randn((G, N), device=dev, generator=gen) * 0.01
        ts = torch.randn(T, device=dev, generator=gen) * 0.01
        y = torch.empty((T, N), dtype=torch.float16, device=dev)

        def step(i, starts, stops):
            bracket(starts, stops, lambda: ops.quant_group_matmul(y, x, w, gl, cs, ts, None, abi.GROUP_LIST_COUNTS,
                                                                  abi.MM_ACT_FASTER_GELU, True))

        ms, kern_ms = timed(step, steps, warmup)
        flops = 2.0 * T * K * N
        bytes_ = T * K + G * K * N + G * N * 4 + T * 4 + T * N * 2 + G * 8
        return {"kernel_ms": kern_ms, "tops": flops / (kern_ms * 1e-3) / 1e12, "gbs": bytes_ / (kern_ms * 1e-3) / 1e9,
                "ops": flops, "bytes": bytes_, "reference_published_us_ascend_950pr": 204.129,
                "reference_published_mac_ratio": 0.887}

    def mx(fmt, steps, warmup):
        """The shape of the reference's high-performance MxFP4 example (m = n = k = 8192, bfloat16 output, scale bytes
        127..129 as its gen_data.py draws them; its README reports 681.056 us on an Ascend 950PR for fp4 e1m2 operands,
        context only).  fmt: "fp4" = e2m1 x e2m1 straight on the scaled matrix instruction, "fp4_e1m2" = the example's
        own format (repacked as 6-bit e2m3 codes first, inside the timed call), "fp8" = e4m3 x e4m3."""
        M = N = K = 8192
        f = {"fp4": abi.QDST_FP4_E2M1, "fp4_e1m2": abi.QDST_FP4_E1M2, "fp8": abi.QDST_FP8_E4M3FN}[fmt]
        rb = K if fmt == "fp8" else K // 2
        a = torch.randint(0, 256, (M, rb), dtype=torch.uint8, device=dev, generator=gen)
        b = torch.randint(0, 256, (N, rb), dtype=torch.uint8, device=dev, generator=gen)
        if fmt == "fp8":    # no NaN codes
            a[(a & 0x7F) == 0x7F] = 0
            b[(b & 0x7F) == 0x7F] = 0
        sa = torch.randint(127, 130, (M, K // 32), dtype=torch.uint8, device=dev, generator=gen)
        sb = torch.randint(127, 130, (N, K // 32), dtype=torch.uint8, device=dev, generator=gen)
        c = torch.empty((M, N), dtype=torch.bfloat16, device=dev)

        def step(i, starts, stops):
            bracket(starts, stops, lambda: ops.matmul_mx(c, a, b, sa, sb, f, f, K))

        ms, kern_ms = timed(step, steps, warmup)
        flops = 2.0 * M * N * K
        # two e1m2 operands run as 6-bit e2m3 codes, which the matrix core takes at the 4-bit rate
        peak = PEAK_FP8_TFLOPS if fmt == "fp8" else PEAK_FP4_TFLOPS
        return {"kernel_ms": kern_ms, "tflops": flops / (kern_ms * 1e-3) / 1e12,
                "mfma_frac": flops / (kern_ms * 1e-3) / 1e12 / peak, "peak_tflops": peak,
                "reference_published_us_ascend_950pr_fp4_e1m2": 681.056}

    def strip(d):
        return {k: v for k, v in d.items() if k != "tensors"}

    only = args.only
    if only and only != "w8a8":
        gsum = abi.W4A16_GROUP_SUM
        fn = {"w4a16": lambda: w4a16(1, args.steps, args.warmup, packed=True, mode=gsum),
              "w4a16_per_weight": lambda: w4a16(1, args.steps, args.warmup, packed=True),
              "w4a16_per_weight_m4": lambda: w4a16(4, args.steps, args.warmup, packed=True),
              "w4a16_per_weight_m16": lambda: w4a16(16, args.steps, args.warmup, packed=True),
              "w4a16_nd": lambda: w4a16(1, args.steps, args.warmup),
              "group_example": lambda: group_example(args.steps, args.warmup),
              "mx_fp4": lambda: mx("fp4", args.steps, args.warmup),
              "mx_fp4_e1m2": lambda: mx("fp4_e1m2", args.steps, args.warmup),
              "mx_fp8": lambda: mx("fp8", args.steps, args.warmup),
              "w4a16_m4": lambda: w4a16(4, args.steps, args.warmup, packed=True, mode=gsum),
              "w4a16_m16": lambda: w4a16(16, args.steps, args.warmup, packed=True, mode=gsum),
              "w4a16_nd_m4": lambda: w4a16(4, args.steps, args.warmup),
              "w4a16_nd_m16": lambda: w4a16(16, args.steps, args.warmup),
              "w8a8_m1": lambda: w8a8(1, args.steps, args.warmup, sets=7),
              "w8a8_m8": lambda: w8a8(8, args.steps, args.warmup, sets=7),
              "w8a8_m16": lambda: w8a8(16, args.steps, args.warmup, sets=7),
              "w8a8_m512": lambda: w8a8(512, args.steps, args.warmup, sets=7),
              "w8a8_m8192": lambda: w8a8(8192, max(20, args.steps // 10), 5, settle=40),
              "w8a8_nk_m128": lambda: w8a8(128, args.steps, args.warmup, sets=7, b_nk=True),
              "w8a8_m128": lambda: w8a8(128, args.steps, args.warmup, sets=7),
              "w8a8_packed_m1": lambda: w8a8(1, args.steps, args.warmup, sets=7, packed=True),
              "w8a8_packed_m8": lambda: w8a8(8, args.steps, args.warmup, sets=7, packed=True),
              "w8a8_packed_m16": lambda: w8a8(16, args.steps, args.warmup, sets=7, packed=True),
              "w8a8_packed_m32": lambda: w8a8(32, args.steps, args.warmup, sets=7, packed=True),
              "w8a8_packed_m64": lambda: w8a8(64, args.steps, args.warmup, sets=7, packed=True),
              "w8a8_packed_m128": lambda: w8a8(128, args.steps, args.warmup, sets=7, packed=True),
              "w8a8_nk_m64": lambda: w8a8(64, args.steps, args.warmup, sets=7, b_nk=True),
              "w8a8_packed_down_m16": lambda: w8a8(16, args.steps, args.warmup, sets=7, packed=True, shape=(11008, 4096)),
              "w8a8_packed_down_m64": lambda: w8a8(64, args.steps, args.warmup, sets=7, packed=True, shape=(11008, 4096)),
              "w8a8_nk_down_m16": lambda: w8a8(16, args.steps, args.warmup, sets=7, b_nk=True, shape=(11008, 4096)),
              "w8a8_nk_m32": lambda: w8a8(32, args.steps, args.warmup, sets=7, b_nk=True),
              "w8a8_m32": lambda: w8a8(32, args.steps, args.warmup, sets=7),
              "w8a8_linear_nk_m1": lambda: w8a8_linear(1, args.steps, args.warmup),
              "w8a8_linear_nk_m4": lambda: w8a8_linear(4, args.steps, args.warmup),
              "w8a8_linear_nk_m16": lambda: w8a8_linear(16, args.steps, args.warmup),
              "w8a8_linear_packed_m1": lambda: w8a8_linear(1, args.steps, args.warmup, packed=True),
              "w8a8_linear_packed_m4": lambda: w8a8_linear(4, args.steps, args.warmup, packed=True),
              "w8a8_linear_packed_swiglu_m1": lambda: w8a8_linear(1, args.steps, args.warmup, packed=True, swiglu=True),
              "w8a8_linear_nk_swiglu_m1": lambda: w8a8_linear(1, args.steps, args.warmup, swiglu=True),
              "w8a8_decode_layer_packed_m1": lambda: w8a8_decode_layer(1, args.steps, args.warmup),
              "w8a8_decode_layer_packed_m4": lambda: w8a8_decode_layer(4, args.steps, args.warmup),
              "w8a8_decode_layer_packed_m16": lambda: w8a8_decode_layer(16, args.steps, args.warmup),
              "w8a8_decode_layer_nk_m1": lambda: w8a8_decode_layer(1, args.steps, args.warmup, packed=False),
              "w8a8_nk_m1": lambda: w8a8(1, args.steps, args.warmup, sets=7, b_nk=True),
              "w8a8_nk_m16": lambda: w8a8(16, args.steps, args.warmup, sets=7, b_nk=True),
              "w8a16_nk_m1": lambda: w8a16(1, args.steps, args.warmup, b_nk=True),
              "w8a16_nk_sum_m1": lambda: w8a16(1, args.steps, args.warmup, b_nk=True, mode=abi.W8A16_CHANNEL_SUM),
              "w8a16_nk_sum_m4": lambda: w8a16(4, args.steps, args.warmup, b_nk=True, mode=abi.W8A16_CHANNEL_SUM),
              "w8a16_nk_m4": lambda: w8a16(4, args.steps, args.warmup, b_nk=True),
              "w8a16_nk_m16": lambda: w8a16(16, args.steps, args.warmup, b_nk=True),
              "w8a16_nk_m2048": lambda: w8a16(2048, min(args.steps, 30), min(args.warmup, 5), sets=1, b_nk=True),
              "w8a16_m2048": lambda: w8a16(2048, min(args.steps, 30), min(args.warmup, 5), sets=1),
              "w8a16_m1": lambda: w8a16(1, args.steps, args.warmup),
              "w8a16_m16": lambda: w8a16(16, args.steps, args.warmup), "quant": lambda: quant2a(args.steps, args.warmup),
              "dequant": lambda: dequant2b(args.steps, args.warmup),
              "antiquant": lambda: antiquant2c(args.steps, args.warmup),
              "w8a8_zeros": lambda: w8a8(2048, args.steps, args.warmup, zero=True),
              "group": lambda: group5(args.steps, args.warmup)}[only]
        print(json.dumps({only: strip(fn())}))
        return

    head = w8a8(2048, args.steps, args.warmup, settle=args.settle)
    out = {
        "metric": "w8a8_linear_int8_tops_m2048_k4096_n11008",
        "value": head["tops"],
        "unit": "TOPS",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[2] (W8A8 LLM linear) at M=2048: bf16 x [2048,4096] -> dynamic "
                               "per-token int8 quant -> int8 GEMM with W [4096,11008] -> fused (channel x token) "
                               "dequant to bf16; one step = quant kernel + GEMM kernel",
                   "m": 2048, "k": 4096, "n": 11008, "ops_per_step": head["ops"],
                   "settle_steps": args.settle},
        # The GEMM is one launch that runs two tile shapes: 256x256 tiles for the full round of 256 workgroups and
        # 256x128 tiles for the last partial round; `achieved` is the 2*M*K*N operations over the average duration of
        # the launch, from one pair of events around `steps` back-to-back GEMMs.  `traffic` is HBM bytes per GEMM from
        # rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of `bench.py --only w8a8 --copy-probe`, each counter scaled by
        # its reading for the 1 GiB copy; it is a constant measured offline, not re-measured by this run.
        "roofline": {"bound": "mfma", "kernel": "gemm_dma_dual_kernel (256x256 tiles, then 256x128 tiles for the last partial round)",
                     "achieved": head["gemm_tops"], "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": head["gemm_tops"] / PEAK_INT8_TOPS, "traffic": GEMM_TRAFFIC_BYTES,
                     "avg_kernel_ms": head["gemm_kernel_ms"], "median_kernel_ms_blocks_of_20": head["gemm_kernel_ms_median"],
                     "min_kernel_ms_blocks_of_20": head["gemm_kernel_ms_min"], "ops_per_launch": head["ops"],
                     "algorithmic_bytes": head["bytes"]},
    }
    if only == "w8a8":
        print(json.dumps(out))
        return
    if not args.quick:
        z = w8a8(2048, min(args.steps, 300), min(args.warmup, 50), zero=True)
        out["roofline"]["same_kernel_zero_operands"] = {
            "avg_kernel_ms": z["gemm_kernel_ms"], "achieved": z["gemm_tops"], "frac": z["gemm_tops"] / PEAK_INT8_TOPS,
            "note": "the same GEMM launches on all-zero activations and weights: the instruction stream, tiling and "
                    "memory traffic are those of the headline, only the operand values differ"}
        del z
        torch.cuda.empty_cache()
        g = w8a8(2048, min(args.steps, 300), min(args.warmup, 50), gauss=True)
        out["roofline"]["same_kernel_normal_weights"] = {
            "avg_kernel_ms": g["gemm_kernel_ms"], "achieved": g["gemm_tops"], "frac": g["gemm_tops"] / PEAK_INT8_TOPS,
            "note": "the same GEMM launches on normally distributed weights quantised per output channel by their "
                    "absolute maximum (the headline's weights are uniform over [-127, 127], the most switching "
                    "activity a weight matrix can cause)"}
        del g
        torch.cuda.empty_cache()
    if ceilings is not None:
        out["ceilings"] = ceilings

    # The other workloads run a bounded number of steps so that the whole file finishes in about a minute.
    side_steps, side_warmup = max(100, min(args.steps, 500)), min(args.warmup, 50)
    gemv = w4a16(1, side_steps, side_warmup, packed=True, mode=abi.W4A16_GROUP_SUM)
    gemv_pw = w4a16(1, side_steps, side_warmup, packed=True)
    gemv_nd = w4a16(1, side_steps, side_warmup)
    out["w4a16_gemv"] = {"metric": "w4a16_decode_gemv_hbm_gbs_m1_k8192_n28672", "value": gemv["gbs"], "unit": "GB/s",
                         "workload": "BASELINE configs[3] at M=1 in the mode ASCQ_W4A16_GROUP_SUM (scale and offset "
                                     "applied once per quantisation group to fp32 sums; fp16 output within one bf16 ulp "
                                     "of the per-weight arithmetic), weights pre-packed by ascq_pack_weight_w4 (outside "
                                     "the timed region), 4 rotating weight sets (500 MB > Infinity Cache)",
                         "ms_per_step": gemv["ms_per_step"],
                         "roofline": {"bound": "hbm", "kernel": "w4a16_packed_kernel<offset, 8, 4, group sum> (one launch)",
                                      "achieved": gemv["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                      "frac": gemv["gbs"] / PEAK_HBM_GBS, "traffic": GEMV_PACKED_TRAFFIC_BYTES,
                                      "avg_kernel_ms": gemv["kernel_ms"], "bytes_per_launch": gemv["bytes"]},
                         "per_weight_mode": {"kernel": "w4a16_packed_kernel<offset, 8, 4, per weight> (one launch)",
                                             "workload": "the same GEMV in the default mode ASCQ_W4A16_PER_WEIGHT: "
                                                         "AscendAntiQuant's two roundings to half per weight",
                                             "avg_kernel_ms": gemv_pw["kernel_ms"], "gbs": gemv_pw["gbs"],
                                             "hbm_frac": gemv_pw["gbs"] / PEAK_HBM_GBS},
                         "nd_layout": {"kernel": "w4a16_gemv_kernel<1, offset> + stream_sum_kernel<1>",
                                       "workload": "the same GEMV on the reference's [k, n / 2] weight layout",
                                       "avg_kernel_ms": gemv_nd["kernel_ms"], "gbs": gemv_nd["gbs"],
                                       "hbm_frac": gemv_nd["gbs"] / PEAK_HBM_GBS, "traffic": GEMV_TRAFFIC_BYTES}}
    del gemv_nd, gemv_pw
    torch.cuda.empty_cache()

    if not args.quick:
        others = {}
        s2, w2 = max(100, side_steps // 2), max(3, side_warmup // 2)
        for name, fn in (("quant_2a", lambda: quant2a(s2, w2)), ("dequant_2b", lambda: dequant2b(s2, w2)),
                         ("antiquant_2c", lambda: antiquant2c(s2, w2))):
            r = strip(fn())
            r["hbm_frac"] = r["gbs"] / PEAK_HBM_GBS
            others[name] = r
            torch.cuda.empty_cache()
        for M in (1, 8, 16, 128, 512):
            r = strip(w8a8(M, s2, w2, sets=7))
            others[f"w8a8_m{M}"] = {"gemm_kernel_ms": r["gemm_kernel_ms"], "gemm_tops": r["gemm_tops"],
                                    "gemm_gbs": r["gemm_gbs"], "hbm_frac": r["gemm_gbs"] / PEAK_HBM_GBS,
                                    "mfma_frac": r["gemm_tops"] / PEAK_INT8_TOPS}
        for M in (1, 8, 16, 32, 64, 128):
            r = strip(w8a8(M, s2, w2, sets=7, packed=True))
            others[f"w8a8_packed_m{M}"] = {"gemm_kernel_ms": r["gemm_kernel_ms"], "gemm_gbs": r["gemm_gbs"],
                                           "hbm_frac": r["gemm_gbs"] / PEAK_HBM_GBS,
                                           "note": "weights pre-packed by ascq_pack_weight_w8 (outside the timed "
                                                   "region): one launch, no workspace"}
            torch.cuda.empty_cache()
        for M in (16, 64):
            r = strip(w8a8(M, s2, w2, sets=7, packed=True, shape=(11008, 4096)))
            others[f"w8a8_packed_down_m{M}"] = {"gemm_kernel_ms": r["gemm_kernel_ms"], "gemm_gbs": r["gemm_gbs"],
                                                "hbm_frac": r["gemm_gbs"] / PEAK_HBM_GBS,
                                                "note": "the down projection of the same layer (K=11008, N=4096) on "
                                                        "packed weights: one launch, weights held in registers"}
            torch.cuda.empty_cache()
        r = strip(w8a8(8192, 40, 5, settle=40))
        others["w8a8_m8192"] = {"gemm_kernel_ms": r["gemm_kernel_ms"], "gemm_tops": r["gemm_tops"],
                                "mfma_frac": r["gemm_tops"] / PEAK_INT8_TOPS,
                                "note": "the same linear with 8192 rows: 1376 tiles, 5.4 rounds of the chip"}
        torch.cuda.empty_cache()
        for M in (1, 16, 128):
            r = strip(w8a8(M, s2, w2, sets=7, b_nk=True))
            others[f"w8a8_nk_m{M}"] = {"gemm_kernel_ms": r["gemm_kernel_ms"], "gemm_gbs": r["gemm_gbs"],
                                       "hbm_frac": r["gemm_gbs"] / PEAK_HBM_GBS,
                                       "note": "weights kept as [n, k] (isTransposeB)" +
                                               (": one launch, no workspace" if M <= 224 else "")}
            torch.cuda.empty_cache()
        for M in (1, 4):
            r = strip(w8a8_linear(M, s2, w2))
            others[f"w8a8_linear_nk_m{M}"] = {"step_ms": r["ms_per_step"], "kernel_ms": r["kernel_ms"], "gbs": r["gbs"],
                                              "hbm_frac": r["gbs"] / PEAK_HBM_GBS,
                                              "note": "ascq_linear_w8a8_dynamic on [n, k] weights: bf16 x quantised "
                                                      "per token inside the weight-streaming kernel, one launch per "
                                                      "step (w8a8_nk_m1 is the matmul alone, after a quantiser launch)"}
            torch.cuda.empty_cache()
        for M in (1, 4):
            r = strip(w8a8_linear(M, s2, w2, packed=True))
            others[f"w8a8_linear_packed_m{M}"] = {"step_ms": r["ms_per_step"], "kernel_ms": r["kernel_ms"],
                                                  "gbs": r["gbs"], "hbm_frac": r["gbs"] / PEAK_HBM_GBS,
                                                  "note": "ascq_linear_w8a8_dynamic_packed: the same one-launch "
                                                          "linear on weights packed by ascq_pack_weight_w8"}
            torch.cuda.empty_cache()
        for M in (1, 4):
            r = strip(w8a8_decode_layer(M, s2, w2))
            others[f"w8a8_decode_layer_packed_m{M}"] = {
                "step_ms": r["ms_per_step"], "kernel_ms": r["kernel_ms"], "gbs": r["gbs"],
                "hbm_frac": r["gbs"] / PEAK_HBM_GBS,
                "note": "the four linears of a decoder layer (hidden 4096, feed-forward 11008: QKV, attention output, "
                        "gate / up with SwiGLU, down) on packed weights, four launches per step, 202 MB of weights"}
            torch.cuda.empty_cache()
        for M in (4, 16):
            r = strip(w4a16(M, s2, w2))
            others[f"w4a16_m{M}"] = {"kernel_ms": r["kernel_ms"], "gbs": r["gbs"], "hbm_frac": r["gbs"] / PEAK_HBM_GBS}
            torch.cuda.empty_cache()
            r = strip(w4a16(M, s2, w2, packed=True, mode=abi.W4A16_GROUP_SUM))
            others[f"w4a16_packed_m{M}"] = {"kernel_ms": r["kernel_ms"], "gbs": r["gbs"],
                                            "hbm_frac": r["gbs"] / PEAK_HBM_GBS, "mode": "ASCQ_W4A16_GROUP_SUM"}
            torch.cuda.empty_cache()
            r = strip(w4a16(M, s2, w2, packed=True))
            others[f"w4a16_packed_per_weight_m{M}"] = {"kernel_ms": r["kernel_ms"], "gbs": r["gbs"],
                                                       "hbm_frac": r["gbs"] / PEAK_HBM_GBS,
                                                       "mode": "ASCQ_W4A16_PER_WEIGHT"}
            torch.cuda.empty_cache()
        for M in (1, 16):
            r = w8a16(M, s2, w2)
            others[f"w8a16_m{M}_k8192_n28672"] = {"kernel_ms": r["kernel_ms"], "gbs": r["gbs"], "bytes": r["bytes"],
                                                  "hbm_frac": r["gbs"] / PEAK_HBM_GBS}
            torch.cuda.empty_cache()
            r = w8a16(M, s2, w2, b_nk=True)
            others[f"w8a16_nk_m{M}_k8192_n28672"] = {"kernel_ms": r["kernel_ms"], "gbs": r["gbs"], "bytes": r["bytes"],
                                                     "hbm_frac": r["gbs"] / PEAK_HBM_GBS,
                                                     "note": "weights kept as [n, k]: one launch, no workspace"}
            torch.cuda.empty_cache()
            if M == 1:
                r = w8a16(M, s2, w2, b_nk=True, mode=abi.W8A16_CHANNEL_SUM)
                others["w8a16_nk_channel_sum_m1_k8192_n28672"] = {
                    "kernel_ms": r["kernel_ms"], "gbs": r["gbs"], "bytes": r["bytes"], "hbm_frac": r["gbs"] / PEAK_HBM_GBS,
                    "mode": "ASCQ_W8A16_CHANNEL_SUM", "note": "weights kept as [n, k]: one launch, no workspace"}
                torch.cuda.empty_cache()
        for nk in (True, False):
            r = w8a16(2048, 30, 5, sets=1, b_nk=nk)
            others["w8a16_nk_m2048_k8192_n28672" if nk else "w8a16_m2048_k8192_n28672"] = {
                "kernel_ms": r["kernel_ms"], "tflops": r["tflops"], "f16_mfma_frac": r["tflops"] / PEAK_F16_TFLOPS,
                "note": "half GEMM whose B-tile loader de-quantises (w8a16_nk_gemm_kernel)" +
                        ("" if nk else ", after one transposed copy of the [k, n] weights into the workspace")}
            torch.cuda.empty_cache()
        r = group5(max(20, side_steps // 5), 5)
        r["mfma_frac"] = r["tops"] / PEAK_INT8_TOPS
        r["hbm_frac"] = r["gbs"] / PEAK_HBM_GBS
        others["group_matmul_config5"] = r
        torch.cuda.empty_cache()
        r = group_example(max(20, side_steps // 5), 5)
        r["mfma_frac"] = r["tops"] / PEAK_INT8_TOPS
        others["group_matmul_reference_example"] = r
        torch.cuda.empty_cache()
        for fmt in ("fp4", "fp8", "fp4_e1m2"):
            others[f"mx_{fmt}_8192"] = mx(fmt, 100, 20)
            torch.cuda.empty_cache()
        out["others"] = others

    # ------------------------------------------------------------------ CPU baseline (the oracle; a checker being timed)
    if not args.no_cpu:
        import orc
        cores = min(16, os.cpu_count() or 1)
        orc.set_threads(cores)
        x, w, cs = head["tensors"]
        xb = x.view(torch.int16).cpu().numpy().view(np.uint16)
        wn, csn = w.cpu().numpy(), cs.cpu().numpy()
        d = abi.MatmulDesc(m=2048, n=11008, k=4096, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                           scale_format=abi.MM_SCALE_F32, has_tok_scale=1)
        reps, t0 = 0, time.perf_counter()
        while True:                                   # bounded sample: whole steps until about 12 s have passed
            qn, tsn = orc.dynamic_quant_per_token(abi.BF16, xb)
            orc.matmul_w8a8(d, qn, wn, None, csn, tsn)
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= 12.0 or reps >= 64:
                break
        cpu_model = "unknown"
        try:
            with open("/proc/cpuinfo") as f:
                cpu_model = next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")), "unknown")
        except OSError:
            pass
        out["cpu_baseline"] = {"value": reps * 2.0 * 2048 * 4096 * 11008 / dt / 1e12, "unit": "TOPS", "cores": cores,
                               "kind": "port", "cpu_model": cpu_model,
                               "label": "CPU restatement of asc-devkit semantics (oracle/), not the reference's CPU-debug build",
                               "sample": f"{reps} whole steps of the same workload (per-token quant + int8 GEMM + "
                                         f"epilogue, all 2048 rows) in {dt:.2f} s, OpenMP over rows"}
        # the same on one thread, on a row sample: 256 of the 2048 rows (the work is independent per row)
        orc.set_threads(1)
        d1 = abi.MatmulDesc(m=256, n=11008, k=4096, out_dtype=abi.BF16, quant_mode=abi.MM_QUANT_VECTOR,
                            scale_format=abi.MM_SCALE_F32, has_tok_scale=1)
        t0 = time.perf_counter()
        q1, ts1 = orc.dynamic_quant_per_token(abi.BF16, xb[:256])
        orc.matmul_w8a8(d1, q1, wn, None, csn, ts1)
        dt1 = time.perf_counter() - t0
        out["cpu_baseline"]["single_thread"] = {"value": 2.0 * 256 * 4096 * 11008 / dt1 / 1e12, "unit": "TOPS", "cores": 1,
                                                "sample": f"rows 0..255 of the same step (an eighth of it) in {dt1:.2f} s"}
        orc.set_threads(cores)
        xs, w4, sc4, of4 = gemv["tensors"]
        d4 = abi.W4A16Desc(m=1, n=28672, k=8192, group_size=128, has_offset=1)
        a4 = (xs.cpu().numpy(), w4.cpu().numpy(), sc4.cpu().numpy(), of4.cpu().numpy())
        reps, t0 = 0, time.perf_counter()
        while True:
            orc.matmul_w4a16(d4, *a4)
            reps += 1
            dt = time.perf_counter() - t0
            if dt >= 6.0 or reps >= 64:
                break
        out["w4a16_gemv"]["cpu_baseline"] = {"value": reps * gemv["bytes"] / dt / 1e9, "unit": "GB/s",
                                             "cores": cores, "kind": "port", "cpu_model": cpu_model,
                                             "sample": f"{reps} whole GEMVs (all 28672 columns) in {dt:.2f} s"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
