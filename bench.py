#!/usr/bin/env python3
"""Benchmark of the MME compute path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: the fp8_143 (exponent bias 7) GEMM
M = N = K = 4096 with fp32 accumulation and bf16 output (the configuration the baseline metric is quoted on).  The
operands are N(0,1) tensors quantised once, before the timed region, with per-tensor power-of-two scales and RNE +
saturation; the descale 2^-(eA+eB) and the bf16 cast are fused behind the contraction.  Operands and output are
resident in HBM when the timed region starts.

Prints one JSON line.  `roofline` is measured live with events on the stream the kernel runs on; `cpu_baseline` is the
reference calculator (oracle/_ref, the reference's own sources) or, where that library is absent, the oracle
restatement, timed on a bounded M-slab of the same GEMM on this host's cores.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--extra]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"fp8": 5000.0, "bf16": 2500.0, "fp32": 157.3}  # dense MFMA peaks of MI355X (fp16 as bf16)
PEAK_HBM_GBS = 8000.0
METRIC = "TFLOP/s & % fp8/bf16 MFMA peak (GEMM, conv); cast GB/s vs HBM peak; 1 GPU"


# HBM bytes per launch of the fp8 GEMM kernel on this workload, from the FETCH_SIZE / WRITE_SIZE counter runs summarised in
# profiles/gemm_fp8_fast_kernel_4096x4096x4096_hbm_traffic.txt (96.3 MiB fetched + 32.1 MiB written; 64 MiB algorithmic)
GEMM_TRAFFIC_BYTES = 134.6e6


def pow2_scale_exp(absmax, fmax):
    import math
    return int(math.floor(math.log2(fmax / absmax)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=256, help="rows of A in the CPU baseline's M-slab")
    ap.add_argument("--extra", action="store_true", help="also time the other configurations (conv, casts, batched fp8)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also launch a plain elementwise copy of 2^26 floats (256 MiB read, 256 MiB written) a few times: a "
                         "counter run (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) scales the GEMM kernel's reading by this kernel's")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path has no multi-GPU part in this build (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from intel_gaudi3_software_amd import Epilogue, HipCalculator, MmeSimTensor, abi

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    calc = HipCalculator()
    # run on a torch-owned (non-default) stream so that torch.cuda.Event brackets exactly the kernels launched here
    stream = torch.cuda.Stream()
    assert stream.cuda_stream != 0
    calc.setStream(stream.cuda_stream)

    M = N = K = 4096
    rng = np.random.default_rng(2002)
    a32 = rng.standard_normal(M * K).astype(np.float32)
    b32 = rng.standard_normal(K * N).astype(np.float32)
    d_a32, d_b32 = torch.from_numpy(a32).cuda(), torch.from_numpy(b32).cuda()
    absmax = torch.zeros(2, dtype=torch.float32, device="cuda")
    calc.absmax(absmax[0:1], d_a32, M * K)
    calc.absmax(absmax[1:2], d_b32, K * N)
    torch.cuda.synchronize()
    eA, eB = (pow2_scale_exp(float(v), 240.0) for v in absmax.cpu())
    qa = torch.zeros(M * K, dtype=torch.uint8, device="cuda")
    qb = torch.zeros(K * N, dtype=torch.uint8, device="cuda")
    calc.castFromFp32(qa, abi.FP8_143, d_a32, M * K, fpBias=7, scale_exp=eA, clipFp=True)
    calc.castFromFp32(qb, abi.FP8_143, d_b32, K * N, fpBias=7, scale_exp=eB, clipFp=True)
    out = torch.zeros(M * N, dtype=torch.int16, device="cuda")
    X = MmeSimTensor([K, M], 2, abi.FP8_143, qa, 7)
    W = MmeSimTensor([N, K], 2, abi.FP8_143, qb, 7)
    Y = MmeSimTensor([N, M], 2, abi.BF16, out)
    epi = Epilogue(scale_exp=-(eA + eB), clipFp=True)
    del d_a32, d_b32

    def step():
        calc.doBatchGemm(Y, X, W, abi.OP_AB, epilogue=epi)

    if args.pmc_calibration:
        with torch.cuda.stream(stream):
            src = torch.ones(1 << 26, dtype=torch.float32, device="cuda")
            dst = torch.empty_like(src)
            for _ in range(5):
                torch.add(src, 0.0, out=dst)
        torch.cuda.synchronize()
        del src, dst

    # The operands come out of the saturating quantiser above, which never emits an exponent-all-ones code, so the
    # device-side scan for such codes (the default, MME_HIP_FP8_SPECIALS_CHECK) is told to stand down for the timed
    # region; its cost is measured separately below and reported as `fp8_specials_check`.
    calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_CHECK)
    for _ in range(max(3, args.warmup // 4)):
        step()
    torch.cuda.synchronize()
    c0, c1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    c0.record(stream)
    for _ in range(20):
        step()
    c1.record(stream)
    torch.cuda.synchronize()
    checked_ms = c0.elapsed_time(c1) / 20
    calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_ASSUME_NONE)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for _ in range(args.steps):
        step()
    ev1.record(stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = ev0.elapsed_time(ev1)
    flop = 2.0 * M * N * K
    ms_per_step = wall * 1e3 / args.steps
    value = flop * args.steps / wall / 1e12
    kernel_ms = dev_ms / args.steps            # average launch-to-launch duration on the stream
    achieved = flop / (kernel_ms * 1e-3) / 1e12

    result = {
        "metric": METRIC, "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8", "data": "synthetic",
        "config": {"workload": "fp8_143 (exp bias 7) GEMM M=N=K=4096, per-tensor pow2 scales, fp32 accumulate, fused descale + bf16 "
                               "output (BASELINE.json configs[1])", "op": "ab", "M": M, "N": N, "K": K, "scale_exp_a": eA, "scale_exp_b": eB},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["fp8"], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS["fp8"], 4), "traffic": GEMM_TRAFFIC_BYTES,
                     "kernel": "gemm_fp8_fast_kernel<0, false>", "kernel_ms": round(kernel_ms, 5)},
        "fp8_specials_check": {"policy_in_timed_region": "assume_none (operands produced by the saturating quantiser)",
                               "ms_per_step_with_device_side_scan": round(checked_ms, 5)},
    }

    # ---- parity of the timed output on an M-slab + CPU baseline -----------------------------------------------------
    if not args.no_cpu_baseline:
        import oracle
        rows = min(args.cpu_rows, M)
        a8 = qa.cpu().numpy()[:rows * K].copy()
        b8 = qb.cpu().numpy()
        acc = np.zeros(rows * N, np.float32)
        da = abi.make_tensor(a8.ctypes.data, [K, rows], abi.FP8_143, 7)
        db = abi.make_tensor(b8.ctypes.data, [N, K], abi.FP8_143, 7)
        do = abi.make_tensor(acc.ctypes.data, [N, rows], abi.FP32)
        R = oracle.ref()
        threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
        t1 = time.perf_counter()
        if R is not None:
            R.ref_set_num_threads(threads)
            rc = R.ref_batch_gemm(C.addressof(do), C.addressof(da), C.addressof(db), abi.OP_AB)
            kind = "reference"
        else:
            O = oracle.oracle()
            O.orc_set_num_threads(threads)
            rc = O.orc_batch_gemm(C.addressof(do), C.addressof(da), C.addressof(db), abi.OP_AB)
            kind = "port"
        cpu_s = time.perf_counter() - t1
        assert rc == 0
        want = np.zeros(rows * N, np.uint16)
        O = oracle.oracle()
        assert O.orc_cast_from_fp32(want.ctypes.data, abi.BF16, 0, 0, acc.ctypes.data, rows * N, -(eA + eB), None, 0, 0, 0, 1, 0, 0) == 0
        got = out.cpu().numpy().view(np.uint16)[:rows * N]
        wf = (want.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        gf = (got.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        result["parity"] = {"rows_checked": rows, "rel_frobenius_vs_reference_bf16": float(np.linalg.norm(gf - wf) / np.linalg.norm(wf)),
                            "bf16_codes_equal_frac": float(np.mean(got == want)), "tolerance": 1e-2}
        result["cpu_baseline"] = {"value": round(2.0 * rows * N * K / cpu_s / 1e12, 7), "unit": "TFLOP/s", "cores": threads, "kind": kind,
                                  "sample": "first %d rows of A against the full B (%.2f GFLOP of the 137.4 GFLOP GEMM, doBatchGemm only), "
                                            "%.1f s wall" % (rows, 2.0 * rows * N * K / 1e9, cpu_s)}

    if args.extra:
        result["extra"] = extra_measurements(calc, stream)

    print(json.dumps(result))
    calc.close()


def extra_measurements(calc, stream):
    """The other configurations of the baseline, each with its own roofline line (device-resident, events)."""
    import numpy as np
    import torch
    from intel_gaudi3_software_amd import ConvolutionParams, Epilogue, MmeSimTensor, abi

    def timed(fn, n=50, warm=5):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n):
            fn()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e-3

    res = {}
    # casts on 2^28 elements
    n = 1 << 28
    x = torch.randn(n, device="cuda")
    for dt, name, ob in ((abi.FP8_143, "cast_fp32_to_fp8_143", 1), (abi.BF16, "cast_fp32_to_bf16", 2)):
        o = torch.zeros(n * ob, dtype=torch.uint8, device="cuda")
        t = timed(lambda: calc.castFromFp32(o, dt, x, n, fpBias=7, clipFp=True), n=20)
        res[name] = {"seconds": t, "GB/s": n * (4 + ob) / t / 1e9, "frac_hbm_peak": n * (4 + ob) / t / 1e9 / PEAK_HBM_GBS}
    o8 = torch.zeros(n, dtype=torch.uint8, device="cuda")
    t = timed(lambda: calc.castToFp32(x, o8, abi.FP8_143, n, fpBias=7), n=20)
    res["dequant_fp8_143_to_fp32"] = {"seconds": t, "GB/s": n * 5 / t / 1e9, "frac_hbm_peak": n * 5 / t / 1e9 / PEAK_HBM_GBS}
    del x, o8
    # conv fwd bf16 N=64 H=W=56 C=K=64 3x3
    Cc = Kk = 64
    H = Wd = 56
    B = 64
    xs, ws, ys = [Cc, Wd, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, Wd, H, 1, B]
    tx = torch.relu(torch.randn(int(np.prod(xs)), device="cuda")).to(torch.bfloat16).view(torch.int16)
    tw = (torch.randn(int(np.prod(ws)), device="cuda") * (2.0 / (Cc * 9)) ** 0.5).to(torch.bfloat16).view(torch.int16)
    ty = torch.zeros(int(np.prod(ys)), dtype=torch.int16, device="cuda")
    cp = ConvolutionParams(2, [1, 1, 0, 0])
    XT, WT, YT = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw), MmeSimTensor(ys, 5, abi.BF16, ty)
    e = Epilogue(clipFp=True)
    t = timed(lambda: calc.doConvolution(YT, XT, WT, YT, cp, abi.OP_FWD, epilogue=e))
    fl = 2.0 * B * H * Wd * Kk * Cc * 9
    res["conv_fwd_bf16_n64_56x56_c64_k64_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_bf16_peak": fl / t / 1e12 / PEAK_TFLOPS["bf16"]}
    del tx, tw, ty

    def rand_bf16(n, scale=1.0):
        return (torch.randn(n, device="cuda") * scale).to(torch.bfloat16).view(torch.int16)

    # c1: bf16 512^3 -> fp32
    n1 = 512
    A1, B1 = MmeSimTensor([n1, n1], 2, abi.BF16, rand_bf16(n1 * n1)), MmeSimTensor([n1, n1], 2, abi.BF16, rand_bf16(n1 * n1))
    Y1 = MmeSimTensor([n1, n1], 2, abi.FP32, torch.zeros(n1 * n1, dtype=torch.float32, device="cuda"))
    t = timed(lambda: calc.doBatchGemm(Y1, A1, B1, abi.OP_AB))
    res["gemm_bf16_512x512x512_fp32_out"] = {"seconds": t, "TFLOP/s": 2.0 * n1 ** 3 / t / 1e12, "frac_bf16_peak": 2.0 * n1 ** 3 / t / 1e12 / PEAK_TFLOPS["bf16"]}
    # fp16 (IEEE half through the fp16 matrix instruction) and ufp16 (decoded to fp32 first) 4096^3 -> fp32; fp32 -> fp16 cast
    # c4: bf16 3x3 dedx / dedw, N=32 28x28 C=K=256
    Cc = Kk = 256
    H = Wd = 28
    B = 32
    xs, ws, ys = [Cc, Wd, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, Wd, H, 1, B]
    XT = MmeSimTensor(xs, 5, abi.BF16, rand_bf16(int(np.prod(xs))))
    WT = MmeSimTensor(ws, 5, abi.BF16, rand_bf16(int(np.prod(ws)), 0.02))
    YT = MmeSimTensor(ys, 5, abi.BF16, rand_bf16(int(np.prod(ys))))
    DX = MmeSimTensor(xs, 5, abi.FP32, torch.zeros(int(np.prod(xs)), dtype=torch.float32, device="cuda"))
    DW = MmeSimTensor(ws, 5, abi.FP32, torch.zeros(int(np.prod(ws)), dtype=torch.float32, device="cuda"))
    fl = 2.0 * B * H * Wd * Kk * Cc * 9
    t = timed(lambda: calc.doConvolution(DX, XT, WT, YT, cp, abi.OP_DEDX), n=20)
    res["conv_dedx_bf16_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_bf16_peak": fl / t / 1e12 / PEAK_TFLOPS["bf16"]}
    t = timed(lambda: calc.doConvolution(DW, XT, WT, YT, cp, abi.OP_DEDW), n=20)
    res["conv_dedw_bf16_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_bf16_peak": fl / t / 1e12 / PEAK_TFLOPS["bf16"]}
    # the same layer with Gaudi fp8 operands (fp8_143 activations, bias 7; fp8_152 gradients, bias 15): fwd and dedx
    q8 = lambda n, hi: torch.randint(0, hi, (n,), dtype=torch.uint8, device="cuda")
    X8 = MmeSimTensor(xs, 5, abi.FP8_143, q8(int(np.prod(xs)), 0x60), 7)
    W8 = MmeSimTensor(ws, 5, abi.FP8_143, q8(int(np.prod(ws)), 0x40), 7)
    Y8 = MmeSimTensor(ys, 5, abi.FP8_152, q8(int(np.prod(ys)), 0x70), 15)
    YO = MmeSimTensor(ys, 5, abi.FP32, torch.zeros(int(np.prod(ys)), dtype=torch.float32, device="cuda"))
    t = timed(lambda: calc.doConvolution(YO, X8, W8, YO, cp, abi.OP_FWD), n=20)
    res["conv_fwd_fp8_143_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_fp8_peak": fl / t / 1e12 / PEAK_TFLOPS["fp8"]}
    t = timed(lambda: calc.doConvolution(DX, X8, W8, Y8, cp, abi.OP_DEDX), n=20)
    res["conv_dedx_fp8_152x143_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_fp8_peak": fl / t / 1e12 / PEAK_TFLOPS["fp8"]}
    t = timed(lambda: calc.doConvolution(DW, X8, W8, Y8, cp, abi.OP_DEDW), n=20)
    res["conv_dedw_fp8_143x152_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_fp8_peak": fl / t / 1e12 / PEAK_TFLOPS["fp8"]}
    del XT, WT, YT, DX, DW, X8, W8, Y8, YO
    # c5: batched mixed fp8: A fp8_143 (bias 7) [4096, 2048, 4] x B fp8_152 (bias 15) [14336, 4096, 1] (broadcast) -> fp8_143
    M5, K5, N5, b5 = 2048, 4096, 14336, 4
    qa = torch.randint(0, 0x78, (b5 * M5 * K5,), dtype=torch.uint8, device="cuda")
    qb = torch.randint(0, 0x7C, (K5 * N5,), dtype=torch.uint8, device="cuda")
    o5 = torch.zeros(b5 * M5 * N5, dtype=torch.uint8, device="cuda")
    A5 = MmeSimTensor([K5, M5, b5], 3, abi.FP8_143, qa, 7)
    B5 = MmeSimTensor([N5, K5, 1], 3, abi.FP8_152, qb, 15)
    Y5 = MmeSimTensor([N5, M5, b5], 3, abi.FP8_143, o5, 7)
    e5 = Epilogue(scale_exp=-12, clipFp=True)
    fl = 2.0 * b5 * M5 * N5 * K5
    t = timed(lambda: calc.doBatchGemm(Y5, A5, B5, abi.OP_AB, epilogue=e5), n=10, warm=2)
    res["bgemm_fp8_143x152_4x2048x14336x4096_fp8_out"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_fp8_peak": fl / t / 1e12 / PEAK_TFLOPS["fp8"]}
    # fp8 GEMM with A stored K x M ("atb": A read through transposing LDS loads)
    nt = 4096
    qt = lambda: torch.randint(0, 0x60, (nt * nt,), dtype=torch.uint8, device="cuda")
    AT, BT = MmeSimTensor([nt, nt], 2, abi.FP8_143, qt(), 7), MmeSimTensor([nt, nt], 2, abi.FP8_143, qt(), 7)
    YT8 = MmeSimTensor([nt, nt], 2, abi.FP32, torch.zeros(nt * nt, dtype=torch.float32, device="cuda"))
    t = timed(lambda: calc.doBatchGemm(YT8, AT, BT, abi.OP_ATB), n=20)
    res["gemm_fp8_143_atb_4096x4096x4096_fp32_out"] = {"seconds": t, "TFLOP/s": 2.0 * nt ** 3 / t / 1e12, "frac_fp8_peak": 2.0 * nt ** 3 / t / 1e12 / PEAK_TFLOPS["fp8"]}
    del AT, BT, YT8
    # the fp16 flavours last: their work spaces (two bf16 copies of both operands) are the largest allocations of the run
    n4 = 4096
    h16 = lambda: torch.randn(n4 * n4, device="cuda").to(torch.float16).view(torch.int16)
    AH, BH = MmeSimTensor([n4, n4], 2, abi.FP16, h16(), 15), MmeSimTensor([n4, n4], 2, abi.FP16, h16(), 15)
    YH = MmeSimTensor([n4, n4], 2, abi.FP32, torch.zeros(n4 * n4, dtype=torch.float32, device="cuda"))
    t = timed(lambda: calc.doBatchGemm(YH, AH, BH, abi.OP_ABT), n=20)
    res["gemm_fp16_4096x4096x4096_fp32_out"] = {"seconds": t, "TFLOP/s": 2.0 * n4 ** 3 / t / 1e12, "frac_fp16_peak": 2.0 * n4 ** 3 / t / 1e12 / PEAK_TFLOPS["bf16"]}
    u16 = lambda: torch.randint(0x7000, 0x8800, (n4 * n4,), dtype=torch.int32, device="cuda").to(torch.int16)
    AU, BU = MmeSimTensor([n4, n4], 2, abi.UFP16, u16(), 31), MmeSimTensor([n4, n4], 2, abi.UFP16, u16(), 31)
    t = timed(lambda: calc.doBatchGemm(YH, AU, BU, abi.OP_ABT), n=10, warm=2)
    # unsigned fp16 runs as a bf16 contraction over 4 K (operands split into two bf16 parts): TFLOP/s counts the algorithm's
    # 2 M N K, the fraction prices the four bf16 products per multiply-add that the matrix cores execute
    res["gemm_ufp16_4096x4096x4096_fp32_out"] = {"seconds": t, "TFLOP/s": 2.0 * n4 ** 3 / t / 1e12,
                                                 "frac_bf16_peak_of_issued_products": 4 * 2.0 * n4 ** 3 / t / 1e12 / PEAK_TFLOPS["bf16"]}
    # fp32 operands: three bf16 parts per value, six cross products on the bf16 matrix cores
    f32 = lambda: torch.randn(n4 * n4, device="cuda")
    AF, BF = MmeSimTensor([n4, n4], 2, abi.FP32, f32()), MmeSimTensor([n4, n4], 2, abi.FP32, f32())
    t = timed(lambda: calc.doBatchGemm(YH, AF, BF, abi.OP_ABT), n=10, warm=2)
    res["gemm_fp32_4096x4096x4096_fp32_out"] = {"seconds": t, "TFLOP/s": 2.0 * n4 ** 3 / t / 1e12, "frac_fp32_peak": 2.0 * n4 ** 3 / t / 1e12 / PEAK_TFLOPS["fp32"],
                                                "frac_bf16_peak_of_issued_products": 6 * 2.0 * n4 ** 3 / t / 1e12 / PEAK_TFLOPS["bf16"]}
    del AH, BH, AU, BU, YH, AF, BF
    nc = 1 << 28
    xc = torch.randn(nc, device="cuda")
    oc = torch.zeros(nc, dtype=torch.int16, device="cuda")
    t = timed(lambda: calc.castFromFp32(oc, abi.FP16, xc, nc, fpBias=15, clipFp=True), n=20)
    res["cast_fp32_to_fp16"] = {"seconds": t, "GB/s": nc * 6 / t / 1e9, "frac_hbm_peak": nc * 6 / t / 1e9 / PEAK_HBM_GBS}
    del xc, oc
    return res


if __name__ == "__main__":
    main()
