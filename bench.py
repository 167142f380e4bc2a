#!/usr/bin/env python3
"""Benchmark of the MME compute path on one MI355X.

A "step" is one pass of the hot path over one batch of synthetic input: the fp8_143 (exponent bias 7) GEMM
M = N = K = 4096 with fp32 accumulation and bf16 output (the configuration the baseline metric is quoted on).  The
operands are N(0,1) tensors quantised once, before the timed region, with per-tensor power-of-two scales and RNE +
saturation; the descale 2^-(eA+eB) and the bf16 cast are fused behind the contraction.  Operands and output are
resident in HBM when the timed region starts.

Prints one JSON line.  `roofline` is measured live with events on the stream the kernel runs on; `cpu_baseline` is the
reference calculator (oracle/_ref, the reference's own sources) or, where that library is absent, the oracle
restatement, timed on this host's cores on a bounded sample of the same workload.  `secondary` holds the other
configurations of the baseline (bf16 512^3 GEMM, bf16 3x3 forward convolution, the backward convolutions, the batched
mixed-fp8 GEMM, the casts), each on the baseline's input distributions, with its own roofline, parity figure and CPU
baseline.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-secondary] [--only NAME] [--extra]
"""
import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"fp8": 5000.0, "bf16": 2500.0, "fp32": 157.3}  # dense MFMA peaks of MI355X (fp16 as bf16)
PEAK_HBM_GBS = 8000.0
METRIC = "TFLOP/s & % fp8/bf16 MFMA peak (GEMM, conv); cast GB/s vs HBM peak; 1 GPU"

# The rocprofv3 summary of each workload under profiles/ ends with a line "bench.py reads: kernel_us=... fetch_bytes=...
# write_bytes=..." (traced average duration of the workload's kernels per call; bytes that crossed the L2 <-> memory
# boundary per call, from the FETCH_SIZE / WRITE_SIZE counter runs).  roofline.traffic and roofline.profile come from that
# line, so they change when the profile is taken again and are null when there is none.
PROFILE_FILE = {"c2": "gemm_fp8_w4_kernel_fp8_gemm_4096x4096x4096.txt", "c1": "gemm_2byte_fast128_kernel_bf16_gemm_512x512x512.txt",
                "c3": "conv_fwd_resident_kernel_bf16_conv_fwd_n64_56x56_c64_k64_3x3.txt",
                "c4_dedx": "conv_2byte_fast128_kernel_bf16_conv_dedx_n32_28x28_c256_k256_3x3.txt",
                "c4_dedw": "conv_dedw_2byte_fast128_kernel_bf16_conv_dedw_n32_28x28_c256_k256_3x3.txt",
                "c5": "gemm_fp8_persistent_chk_kernel_fp8_batched_gemm_4x2048x4096x14336.txt",
                "cast_fp8_143": "cast_from_fp32_kernel_fp32_to_fp8_143_2pow28.txt", "cast_bf16": "cast_from_fp32_kernel_fp32_to_bf16_2pow28.txt",
                "dequant_fp8_143": "cast_to_fp32_kernel_fp8_143_to_fp32_2pow28.txt"}
SETTLE_MS = 60
ROTATE_BYTES = 320 << 20  # operand / output sets of the rotating variants cycle through at least this much memory (memory-side cache: 256 MiB)


def profile_figures(name, work, peak):
    """What the committed profile of workload `name` says: traced kernel time per call, the roofline fraction that follows
    from it (work / time / peak) and the bytes moved per call.  None when the file or its last line is missing."""
    import re
    path = os.path.join(ROOT, "profiles", PROFILE_FILE.get(name, ""))
    try:
        with open(path) as f:
            m = re.search(r"^bench\.py reads: (.*)$", f.read(), re.M)
    except OSError:
        return None
    if not m:
        return None
    kv = dict(t.split("=") for t in m.group(1).split())
    us = float(kv["kernel_us"])
    out = {"file": "profiles/" + PROFILE_FILE[name], "kernel_us": us, "frac": round(work / (us * 1e-6) / peak, 4)}
    if "fetch_bytes" in kv and "write_bytes" in kv:
        out["traffic"] = float(kv["fetch_bytes"]) + float(kv["write_bytes"])
    return out


def attach_profile(roof, name, work=None):
    """roofline.profile / roofline.traffic of a workload from its committed profile (work in flop or bytes, as the bound says)."""
    work = roof["work_per_launch"] if work is None else work
    peak = roof["peak"] * (1e12 if roof["bound"] == "mfma" else 1e9)
    prof = profile_figures(name, work, peak)
    roof["profile"] = prof
    roof["traffic"] = prof.get("traffic") if prof else None

SECONDARY = ("c1", "c3", "c4_dedx", "c4_dedw", "c5", "cast_fp8_143", "cast_bf16", "dequant_fp8_143")


def pow2_scale_exp(absmax, fmax):
    return int(math.floor(math.log2(fmax / absmax)))


def bf16_bits(x):
    import numpy as np
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_to_f64(b):
    import numpy as np
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


class Bench:
    """Device, calculator, stream and the timing / CPU-baseline helpers shared by the workloads."""

    def __init__(self, args):
        import torch
        from intel_gaudi3_software_amd import HipCalculator
        assert torch.cuda.is_available(), "bench.py needs a GPU"
        torch.cuda.set_device(0)
        self.args = args
        self.torch = torch
        self.calc = HipCalculator()
        # run on a torch-owned (non-default) stream so that torch.cuda.Event brackets exactly the kernels launched here
        self.stream = torch.cuda.Stream()
        assert self.stream.cuda_stream != 0
        self.calc.setStream(self.stream.cuda_stream)
        self.cpu = not args.no_cpu_baseline
        self.threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
        self._ref = self._orc = None

    def settle(self, fn, seconds=SETTLE_MS * 1e-3):
        """Calls fn back to back for some tens of milliseconds.  After an idle period (operand set-up on the host) the device
        needs about 50 ms of work to reach the rate it then sustains: the headline GEMM takes 63-74 us per call over the first
        25 ms, 61 us up to 45 ms, and 59.7-59.9 us from there on for as long as it was watched (2.5 s).  Every measurement here
        is of the sustained rate, so each one starts from a device that is already at work (0.06, 0.5 and 2 s of it give the
        same figures for the GEMMs and the convolutions)."""
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(10):
                fn()
            self.torch.cuda.synchronize()

    def timed(self, fn, n=50, warm=5):
        """Average launch-to-launch duration in seconds of n calls of fn on the calculator's stream."""
        torch = self.torch
        self.settle(fn)
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(self.stream)
        for _ in range(n):
            fn()
        e1.record(self.stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e-3

    def per_launch(self, fn, n=60, group=5):
        if self.args.plain:
            return None
        return self._per_launch(fn, n, group)

    def _per_launch(self, fn, n=60, group=5):
        """Distribution of the stream time per call over n x group consecutive calls of fn (n >= 50 intervals): an event after
        every `group` calls, each interval divided by `group`.  An event is a marker on the stream and costs about 3.5 us
        of stream time itself (one per interval, so 0.7 us per call at group = 5): the figures of this pass sit that much above
        the mean of the marker-free timed region, which stays the reported one; `marker_us_per_call` says how much."""
        torch = self.torch
        n = max(n, 50)
        self.settle(fn)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(self.stream)
        for _ in range(n * group):
            fn()
        e1.record(self.stream)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
        ev[0].record(self.stream)
        for i in range(n):
            for _ in range(group):
                fn()
            ev[i + 1].record(self.stream)
        torch.cuda.synchronize()
        free = e0.elapsed_time(e1) * 1e3 / (n * group)
        us = sorted(ev[i].elapsed_time(ev[i + 1]) * 1e3 / group for i in range(n))
        med = us[n // 2] if n % 2 else 0.5 * (us[n // 2 - 1] + us[n // 2])
        mean = sum(us) / n
        return {"launches": n * group, "intervals": n, "calls_per_interval": group, "mean": round(mean, 3), "median": round(med, 3), "min": round(us[0], 3),
                "max": round(us[-1], 3), "mean_without_markers": round(free, 3), "marker_us_per_call": round(mean - free, 3)}

    def rotating(self, fns, n=60):
        """The same call on len(fns) separate sets of operands and outputs taken in turn, which together hold more than the
        memory-side cache: no call finds its operands, or the lines of its output, where its predecessor on the same set left
        them.  Returns (mean seconds per call, per-launch distribution)."""
        k = [0]

        def step():
            fns[k[0] % len(fns)]()
            k[0] += 1

        return self.timed(step, n=max(n, 4 * len(fns))), self._per_launch(step, n=n)

    def clocked(self, fn, n=30):
        if self.args.plain:
            return None
        return self._clocked(fn, n)

    def _clocked(self, fn, n=30):
        """The shader clock the large-tile kernels ran at during n back-to-back calls of fn, and how long a workgroup took
        (stamps taken inside the kernels; the published peak rates are quoted at 2400 MHz).  call_us_with_probe is the wall
        time per call while the stamps are on, the read-out of the stamps at the end included (2 us per call at n = 50): the
        probe is not free for every kernel (the persistent walk of the batched GEMM ran 3 to 17 % slower with it on
        different boxes), so a clock read here belongs to that time, not to the timed region's."""
        self.calc.clockProbe(True)
        self.settle(fn)
        self.calc.readClockProbe()
        t0 = time.perf_counter()
        for _ in range(n):
            fn()
        r = self.calc.readClockProbe()   # (synchronises)
        wall = time.perf_counter() - t0
        self.calc.clockProbe(False)
        return {"shader_clock_mhz": round(r["shader_mhz"]), "workgroup_us_mean": round(r["workgroup_us_mean"], 2),
                "workgroup_us_max": round(r["workgroup_us_max"], 2), "workgroups_seen": r["workgroups"],
                "call_us_with_probe": round(wall / n * 1e6, 2)}

    def matrix_core_ceiling(self, dtype):
        """What back-to-back matrix instructions with operands in registers sustain on this device: with all-zero operands
        (the published rate) and with operands that change from instruction to instruction (power management lowers the clock)."""
        out = {}
        if self.args.plain:
            return None
        for name, rnd in (("zero_operands", 0), ("random_operands", 1)):
            tf, mhz = self.calc.matrixCoreRate(dtype, rnd, iters=4096, launches=10)
            out[name] = {"TFLOP/s": round(tf, 1), "shader_clock_mhz": round(mhz)}
        return out

    def pmc_calibration(self):
        """Five launches of a plain copy of 2^26 floats (256 MiB read, 256 MiB written): the unit of FETCH_SIZE / WRITE_SIZE."""
        torch = self.torch
        with torch.cuda.stream(self.stream):
            src = torch.ones(1 << 26, dtype=torch.float32, device="cuda")
            dst = torch.empty_like(src)
            for _ in range(5):
                torch.add(src, 0.0, out=dst)
        torch.cuda.synchronize()

    def checker(self):
        """(library, kind, prefix): the compiled reference where it has been built, else the oracle restatement."""
        import oracle
        if self._orc is None:
            self._orc = oracle.oracle()
            self._ref = oracle.ref()
            self._orc.orc_set_num_threads(self.threads)
            if self._ref is not None:
                self._ref.ref_set_num_threads(self.threads)
        if self._ref is not None:
            return self._ref, "reference", "ref_"
        return self._orc, "port", "orc_"

    def oracle_lib(self):
        """The oracle restatement (its casts define the expected output codes of a reference accumulator)."""
        self.checker()
        return self._orc

    def cpu_gemm(self, out_desc, a_desc, b_desc, op):
        lib, kind, pre = self.checker()
        t = time.perf_counter()
        rc = getattr(lib, pre + "batch_gemm")(C.addressof(out_desc), C.addressof(a_desc), C.addressof(b_desc), op)
        assert rc == 0
        return time.perf_counter() - t, kind

    def cpu_conv(self, out_desc, x_desc, w_desc, y_desc, params, op):
        lib, kind, pre = self.checker()
        t = time.perf_counter()
        rc = getattr(lib, pre + "convolution")(C.addressof(out_desc), C.addressof(x_desc), C.addressof(w_desc), C.addressof(y_desc),
                                               C.addressof(params), op, 0)
        assert rc == 0
        return time.perf_counter() - t, kind

    def cpu_activation(self, out_desc, acc_desc, clip=1):
        lib, kind, pre = self.checker()
        t = time.perf_counter()
        if pre == "ref_":
            rc = lib.ref_activation(C.addressof(out_desc), C.addressof(acc_desc), 0, 0, clip, 0, 0, 0, None, 0, 0)
        else:
            rc = lib.orc_activation(C.addressof(out_desc), C.addressof(acc_desc), 0, 0, clip, 0, 0, 0, None, 0)
        assert rc == 0
        return time.perf_counter() - t, kind


def mfma_roofline(flop, seconds, kind, kernel):
    achieved = flop / seconds / 1e12
    return {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS[kind], "unit": "TFLOP/s", "frac": round(achieved / PEAK_TFLOPS[kind], 4),
            "traffic": None, "kernel": kernel, "kernel_ms": round(seconds * 1e3, 5), "settle_ms": SETTLE_MS, "work_per_launch": flop}


def rotating_figures(b, fns, work, roof, set_bytes):
    """roofline.rotating: the workload's call cycling through len(fns) operand / output sets (b.rotating)."""
    if b.args.plain:
        return None
    t, dist = b.rotating(fns)
    scale = 1e12 if roof["bound"] == "mfma" else 1e9
    return {"sets": len(fns), "bytes_cycled": int(set_bytes * len(fns)), "kernel_ms": round(t * 1e3, 5), "achieved": round(work / t / scale, 2),
            "frac": round(work / t / scale / roof["peak"], 4), "per_launch_us": dist}


def n_sets(set_bytes):
    return max(2, -(-ROTATE_BYTES // int(set_bytes)))


def hbm_roofline(nbytes, seconds, kernel):
    achieved = nbytes / seconds / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBS, 4),
            "traffic": None, "kernel": kernel, "kernel_ms": round(seconds * 1e3, 5), "settle_ms": SETTLE_MS, "work_per_launch": nbytes}


# ---- the headline workload: configs[1] -------------------------------------------------------------------------------------------
def run_c2(b):
    import numpy as np
    torch, calc, args = b.torch, b.calc, b.args
    from intel_gaudi3_software_amd import Epilogue, MmeSimTensor, abi
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

    # The library's default policy (MME_HIP_FP8_SPECIALS_CHECK) looks for exponent-all-ones codes, which mean inf / NaN to
    # Gaudi and numbers to the matrix cores, while the kernel multiplies, and enqueues the exact fall-back behind it; a
    # caller whose operands come out of a saturating quantiser, as here, may promise that there are none
    # (MME_HIP_FP8_SPECIALS_ASSUME_NONE).  Both are timed; the headline is the promise-free default.
    calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_ASSUME_NONE)
    assumed_s = b.timed(step, n=max(20, args.steps // 4), warm=max(3, args.warmup // 4))
    calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_CHECK)

    b.settle(step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(b.stream)
    for _ in range(args.steps):
        step()
    ev1.record(b.stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    dev_ms = ev0.elapsed_time(ev1)
    flop = 2.0 * M * N * K
    ms_per_step = wall * 1e3 / args.steps
    value = flop * args.steps / wall / 1e12
    kernel_ms = dev_ms / args.steps            # average launch-to-launch duration on the stream
    achieved = flop / (kernel_ms * 1e-3) / 1e12
    assumed = flop / assumed_s / 1e12

    result = {
        "metric": METRIC, "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8", "data": "synthetic",
        "config": {"workload": "fp8_143 (exp bias 7) GEMM M=N=K=4096, per-tensor pow2 scales, fp32 accumulate, fused descale + bf16 "
                               "output (BASELINE.json configs[1]); library default policy for fp8 special codes", "op": "ab", "M": M, "N": N, "K": K,
                   "scale_exp_a": eA, "scale_exp_b": eB},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_TFLOPS["fp8"], "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_TFLOPS["fp8"], 4), "traffic": None,
                     "kernel": "gemm_fp8_w4_kernel<0, false, true>", "kernel_ms": round(kernel_ms, 5), "settle_ms": SETTLE_MS, "work_per_launch": flop,
                     "policy": "check (default): the workgroups inspect the operand bytes they multiply and share what they find per operand panel; a tile whose panels hold a special code is computed again, exactly, inside the same launch",
                     "assume_none": {"achieved": round(assumed, 2), "frac": round(assumed / PEAK_TFLOPS["fp8"], 4), "kernel_ms": round(assumed_s * 1e3, 5),
                                     "kernel": "gemm_fp8_w4_kernel<0, false, false>",
                                     "policy": "the caller promises operands without exponent-all-ones codes (they come out of the saturating quantiser)"}},
    }

    attach_profile(result["roofline"], "c2", flop)
    # every launch on its own (events between the calls), and the same call cycling through operand / output sets that
    # together exceed the memory-side cache
    result["roofline"]["per_launch_us"] = b.per_launch(step, n=60)
    set_bytes = 2 * M * K + 2 * M * N
    sets = [(qa, qb, out)] + [(qa.clone(), qb.clone(), torch.zeros_like(out)) for _ in range(0 if args.plain else n_sets(set_bytes) - 1)]
    descs = [(MmeSimTensor([N, M], 2, abi.BF16, o), MmeSimTensor([K, M], 2, abi.FP8_143, a, 7), MmeSimTensor([N, K], 2, abi.FP8_143, w, 7)) for a, w, o in sets]
    fns = [(lambda y=y, x=x, w=w: calc.doBatchGemm(y, x, w, abi.OP_AB, epilogue=epi)) for y, x, w in descs]
    result["roofline"]["rotating"] = rotating_figures(b, fns, flop, result["roofline"], set_bytes)
    del sets, descs, fns
    torch.cuda.empty_cache()
    # the clock the kernel ran at (all-zero operands would let the device hold 2400 MHz; these operands do not), and what
    # bare matrix instructions sustain on zero and on random operands
    result["roofline"]["clock"] = b.clocked(step, n=50)
    calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_ASSUME_NONE)
    result["roofline"]["assume_none"]["clock"] = b.clocked(step, n=50)
    calc.setFp8SpecialsPolicy(abi.FP8_SPECIALS_CHECK)
    result["roofline"]["matrix_core_ceiling"] = b.matrix_core_ceiling(abi.FP8_143)
    step()  # (the parity check below reads the output of a default-policy call)
    torch.cuda.synchronize()

    # ---- parity of the timed output on M-slabs + CPU baseline --------------------------------------------------------
    if b.cpu:
        orc = b.oracle_lib()
        first = min(args.cpu_rows, M)
        rows = np.concatenate([np.arange(first), np.sort(np.random.default_rng(7).choice(np.arange(first, M), 64, replace=False))])
        a8_all = qa.cpu().numpy().reshape(M, K)
        b8 = qb.cpu().numpy()
        got_all = out.cpu().numpy().view(np.uint16).reshape(M, N)
        a8 = np.ascontiguousarray(a8_all[:first]).ravel()
        acc = np.zeros(first * N, np.float32)
        da = abi.make_tensor(a8.ctypes.data, [K, first], abi.FP8_143, 7)
        db = abi.make_tensor(b8.ctypes.data, [N, K], abi.FP8_143, 7)
        do = abi.make_tensor(acc.ctypes.data, [N, first], abi.FP32)
        cpu_s, kind = b.cpu_gemm(do, da, db, abi.OP_AB)
        # 64 further rows drawn at random (not part of the timed sample)
        a8x = np.ascontiguousarray(a8_all[rows[first:]]).ravel()
        accx = np.zeros(64 * N, np.float32)
        dax = abi.make_tensor(a8x.ctypes.data, [K, 64], abi.FP8_143, 7)
        dox = abi.make_tensor(accx.ctypes.data, [N, 64], abi.FP32)
        b.cpu_gemm(dox, dax, db, abi.OP_AB)
        acc_all = np.concatenate([acc, accx])
        want = np.zeros(acc_all.size, np.uint16)
        assert orc.orc_cast_from_fp32(want.ctypes.data, abi.BF16, 0, 0, acc_all.ctypes.data, acc_all.size, -(eA + eB), None, 0, 0, 0, 1, 0, 0) == 0
        got = got_all[rows].ravel()
        wf, gf = bf16_to_f64(want), bf16_to_f64(got)
        result["parity"] = {"rows_checked": int(rows.size), "rows": "the first %d and 64 drawn at random" % first,
                            "rel_frobenius_vs_reference_bf16": float(np.linalg.norm(gf - wf) / np.linalg.norm(wf)),
                            "bf16_codes_equal_frac": float(np.mean(got == want)), "tolerance": 1e-2}
        result["cpu_baseline"] = {"value": round(2.0 * first * N * K / cpu_s / 1e12, 7), "unit": "TFLOP/s", "cores": b.threads, "kind": kind,
                                  "sample": "first %d rows of A against the full B (%.2f GFLOP of the 137.4 GFLOP GEMM, doBatchGemm only), "
                                            "%.1f s wall" % (first, 2.0 * first * N * K / 1e9, cpu_s)}
    return result


# ---- secondary workloads -----------------------------------------------------------------------------------------------------
def run_c1(b):
    """configs[0]: bf16 512^3 -> fp32, A, B ~ N(0,1), seed 1001."""
    import numpy as np
    torch, calc = b.torch, b.calc
    from intel_gaudi3_software_amd import MmeSimTensor, abi
    n = 512
    rng = np.random.default_rng(1001)
    a, w = bf16_bits(rng.standard_normal(n * n)), bf16_bits(rng.standard_normal(n * n))
    ta, tw = torch.from_numpy(a.view(np.int16)).cuda(), torch.from_numpy(w.view(np.int16)).cuda()
    out = torch.zeros(n * n, dtype=torch.float32, device="cuda")
    A1, B1, Y1 = MmeSimTensor([n, n], 2, abi.BF16, ta), MmeSimTensor([n, n], 2, abi.BF16, tw), MmeSimTensor([n, n], 2, abi.FP32, out)
    t = b.timed(lambda: calc.doBatchGemm(Y1, A1, B1, abi.OP_AB))
    flop = 2.0 * n ** 3
    res = {"workload": "bf16 GEMM 512^3 -> fp32 (configs[0])", "value": round(flop / t / 1e12, 2), "unit": "TFLOP/s",
           "roofline": mfma_roofline(flop, t, "bf16", "gemm_2byte_fast128_kernel")}
    res["roofline"]["per_launch_us"] = b.per_launch(lambda: calc.doBatchGemm(Y1, A1, B1, abi.OP_AB))
    res["roofline"]["clock"] = b.clocked(lambda: calc.doBatchGemm(Y1, A1, B1, abi.OP_AB))
    if b.cpu:
        want = np.zeros(n * n, np.float32)
        da, dw, do = abi.make_tensor(a.ctypes.data, [n, n], abi.BF16), abi.make_tensor(w.ctypes.data, [n, n], abi.BF16), abi.make_tensor(want.ctypes.data, [n, n], abi.FP32)
        cpu_s, kind = b.cpu_gemm(do, da, dw, abi.OP_AB)
        got = out.cpu().numpy().astype(np.float64)
        res["parity"] = {"rel_frobenius_vs_reference_fp32": float(np.linalg.norm(got - want) / np.linalg.norm(want)), "tolerance": 2e-3, "checked": "whole output"}
        res["cpu_baseline"] = {"value": round(flop / cpu_s / 1e12, 7), "unit": "TFLOP/s", "cores": b.threads, "kind": kind,
                               "sample": "the whole GEMM, %.2f s wall" % cpu_s}
    return res


def run_c3(b):
    """configs[2]: bf16 3x3 forward convolution N=64, 56x56, 64 -> 64 channels, x = ReLU(N(0,1)), He-init weights, bf16 output."""
    import numpy as np
    torch, calc = b.torch, b.calc
    from intel_gaudi3_software_amd import ConvolutionParams, Epilogue, MmeSimTensor, abi
    Cc = Kk = 64
    H = Wd = 56
    B = 64
    xs, ws, ys = [Cc, Wd, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, Wd, H, 1, B]
    rng = np.random.default_rng(3003)
    x = bf16_bits(np.maximum(rng.standard_normal(int(np.prod(xs))), 0))
    w = bf16_bits(rng.standard_normal(int(np.prod(ws))) * (2.0 / (Cc * 9)) ** 0.5)
    tx, tw = torch.from_numpy(x.view(np.int16)).cuda(), torch.from_numpy(w.view(np.int16)).cuda()
    ty = torch.zeros(int(np.prod(ys)), dtype=torch.int16, device="cuda")
    cp = ConvolutionParams(2, [1, 1, 0, 0])
    XT, WT, YT = MmeSimTensor(xs, 5, abi.BF16, tx), MmeSimTensor(ws, 5, abi.BF16, tw), MmeSimTensor(ys, 5, abi.BF16, ty)
    e = Epilogue(clipFp=True)
    t = b.timed(lambda: calc.doConvolution(YT, XT, WT, YT, cp, abi.OP_FWD, epilogue=e))
    flop = 2.0 * B * H * Wd * Kk * Cc * 9
    nbytes = 2.0 * (np.prod(xs) + np.prod(ws) + np.prod(ys))
    roof = mfma_roofline(flop, t, "bf16", "conv_fwd_resident_kernel<56>")
    roof["hbm_GB/s_algorithmic"] = round(nbytes / t / 1e9, 1)  # (288 flop per byte: within 10 % of the ridge)
    roof["per_launch_us"] = b.per_launch(lambda: calc.doConvolution(YT, XT, WT, YT, cp, abi.OP_FWD, epilogue=e))
    set_bytes = 2 * (tx.numel() + tw.numel() + ty.numel())
    sets = [(MmeSimTensor(xs, 5, abi.BF16, tx.clone()), MmeSimTensor(ws, 5, abi.BF16, tw.clone()), MmeSimTensor(ys, 5, abi.BF16, torch.zeros_like(ty)))
            for _ in range(0 if b.args.plain else n_sets(set_bytes) - 1)] + [(XT, WT, YT)]
    roof["rotating"] = rotating_figures(b, [(lambda x_=x_, w_=w_, y_=y_: calc.doConvolution(y_, x_, w_, y_, cp, abi.OP_FWD, epilogue=e)) for x_, w_, y_ in sets],
                                        flop, roof, set_bytes)
    del sets
    res = {"workload": "bf16 conv2d fwd N=64 56x56 C=K=64 3x3 s1 p1, fused bf16 output (configs[2])", "value": round(flop / t / 1e12, 2),
           "unit": "TFLOP/s", "roofline": roof}
    if b.cpu:
        orc = b.oracle_lib()
        acc = np.zeros(int(np.prod(ys)), np.float32)
        p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
        dx, dw, do = abi.make_tensor(x.ctypes.data, xs, abi.BF16), abi.make_tensor(w.ctypes.data, ws, abi.BF16), abi.make_tensor(acc.ctypes.data, ys, abi.FP32)
        cpu_s, kind = b.cpu_conv(do, dx, dw, do, p, abi.OP_FWD)
        want = np.zeros(acc.size, np.uint16)
        assert orc.orc_cast_from_fp32(want.ctypes.data, abi.BF16, 0, 0, acc.ctypes.data, acc.size, 0, None, 0, 0, 0, 1, 0, 0) == 0
        got = ty.cpu().numpy().view(np.uint16)
        wf, gf = bf16_to_f64(want), bf16_to_f64(got)
        res["parity"] = {"rel_frobenius_vs_reference_bf16": float(np.linalg.norm(gf - wf) / np.linalg.norm(wf)),
                         "bf16_codes_equal_frac": float(np.mean(got == want)), "tolerance": 2e-3, "checked": "whole output"}
        res["cpu_baseline"] = {"value": round(flop / cpu_s / 1e12, 7), "unit": "TFLOP/s", "cores": b.threads, "kind": kind,
                               "sample": "the whole convolution (doConvolution incl. its im2col), %.1f s wall" % cpu_s}
    return res


def _c4_tensors(b):
    import numpy as np
    Cc = Kk = 256
    H = Wd = 28
    B = 32
    xs, ws, ys = [Cc, Wd, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, Wd, H, 1, B]
    rng = np.random.default_rng(4004)
    x = bf16_bits(np.maximum(rng.standard_normal(int(np.prod(xs))), 0))
    w = bf16_bits(rng.standard_normal(int(np.prod(ws))) * (2.0 / (Cc * 9)) ** 0.5)
    dy = bf16_bits(rng.standard_normal(int(np.prod(ys))) * 1e-2)
    return xs, ws, ys, x, w, dy


def _run_c4(b, op):
    """configs[3]: bf16 3x3 backward convolutions N=32, 28x28, C=K=256: x = ReLU(N(0,1)), dY ~ N(0, 1e-2), He-init weights, fp32 outputs."""
    import numpy as np
    torch, calc = b.torch, b.calc
    from intel_gaudi3_software_amd import ConvolutionParams, MmeSimTensor, abi
    xs, ws, ys, x, w, dy = _c4_tensors(b)
    dev = lambda a: torch.from_numpy(a.view(np.int16)).cuda()
    XT, WT, YT = MmeSimTensor(xs, 5, abi.BF16, dev(x)), MmeSimTensor(ws, 5, abi.BF16, dev(w)), MmeSimTensor(ys, 5, abi.BF16, dev(dy))
    osz = xs if op == abi.OP_DEDX else ws
    to = torch.zeros(int(np.prod(osz)), dtype=torch.float32, device="cuda")
    OT = MmeSimTensor(osz, 5, abi.FP32, to)
    cp = ConvolutionParams(2, [1, 1, 0, 0])
    t = b.timed(lambda: calc.doConvolution(OT, XT, WT, YT, cp, op), n=30)
    flop = 2.0 * 32 * 28 * 28 * 256 * 256 * 9
    name = "dedx" if op == abi.OP_DEDX else "dedw"
    kernel = "conv_2byte_fast128_kernel" if op == abi.OP_DEDX else "conv_dedw_2byte_fast128_kernel + splitk_reduce_kernel"
    res = {"workload": "bf16 conv2d %s N=32 28x28 C=K=256 3x3 s1 p1, fp32 output (configs[3])" % name, "value": round(flop / t / 1e12, 2),
           "unit": "TFLOP/s", "roofline": mfma_roofline(flop, t, "bf16", kernel)}
    res["roofline"]["per_launch_us"] = b.per_launch(lambda: calc.doConvolution(OT, XT, WT, YT, cp, op))
    set_bytes = 2 * (XT.data().numel() + WT.data().numel() + YT.data().numel()) + 4 * to.numel()
    sets = [(MmeSimTensor(xs, 5, abi.BF16, XT.data().clone()), MmeSimTensor(ws, 5, abi.BF16, WT.data().clone()), MmeSimTensor(ys, 5, abi.BF16, YT.data().clone()),
             MmeSimTensor(osz, 5, abi.FP32, torch.zeros_like(to))) for _ in range(0 if b.args.plain else n_sets(set_bytes) - 1)] + [(XT, WT, YT, OT)]
    res["roofline"]["rotating"] = rotating_figures(b, [(lambda x_=x_, w_=w_, y_=y_, o_=o_: calc.doConvolution(o_, x_, w_, y_, cp, op)) for x_, w_, y_, o_ in sets],
                                                   flop, res["roofline"], set_bytes)
    del sets
    res["roofline"]["clock"] = b.clocked(lambda: calc.doConvolution(OT, XT, WT, YT, cp, op))
    if op == abi.OP_DEDX:
        res["roofline"]["matrix_core_ceiling"] = b.matrix_core_ceiling(abi.BF16)
    if b.cpu:
        want = np.zeros(int(np.prod(osz)), np.float32)
        p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
        dx, dw, ddy = abi.make_tensor(x.ctypes.data, xs, abi.BF16), abi.make_tensor(w.ctypes.data, ws, abi.BF16), abi.make_tensor(dy.ctypes.data, ys, abi.BF16)
        do = abi.make_tensor(want.ctypes.data, osz, abi.FP32)
        cpu_s, kind = b.cpu_conv(do, do if op == abi.OP_DEDX else dx, do if op == abi.OP_DEDW else dw, ddy, p, op)
        got = to.cpu().numpy().astype(np.float64)
        res["parity"] = {"rel_frobenius_vs_reference_fp32": float(np.linalg.norm(got - want) / np.linalg.norm(want)), "tolerance": 2e-3, "checked": "whole output"}
        res["cpu_baseline"] = {"value": round(flop / cpu_s / 1e12, 7), "unit": "TFLOP/s", "cores": b.threads, "kind": kind,
                               "sample": "the whole %s (doConvolution incl. its im2col / col2im), %.1f s wall" % (name, cpu_s)}
    return res


def run_c4_dedx(b):
    from intel_gaudi3_software_amd import abi
    return _run_c4(b, abi.OP_DEDX)


def run_c4_dedw(b):
    from intel_gaudi3_software_amd import abi
    return _run_c4(b, abi.OP_DEDW)


def run_c5(b):
    """configs[4]: batch 4, M=2048, K=4096, N=14336: A fp8_143 (bias 7), N(0,1) with 0.1 % of the entries x20, per-tensor scale;
    B fp8_152 (bias 15), N(0, 0.02), per-output-channel scales; per-column descale, output scale calibrated on a slab, fp8_143
    output with saturation."""
    import numpy as np
    torch, calc = b.torch, b.calc
    from intel_gaudi3_software_amd import Epilogue, MmeSimTensor, abi
    M5, K5, N5, b5 = 2048, 4096, 14336, 4
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5005)
    a32 = torch.randn(b5 * M5 * K5, device="cuda", generator=gen)
    a32 = torch.where(torch.rand(a32.numel(), device="cuda", generator=gen) < 1e-3, a32 * 20.0, a32)
    w32 = torch.randn(K5 * N5, device="cuda", generator=gen) * 0.02
    sa = pow2_scale_exp(float(a32.abs().max()), 240.0)
    sb = torch.floor(torch.log2(57344.0 / w32.view(K5, N5).abs().amax(dim=0))).to(torch.int32).contiguous()
    qa = torch.zeros(a32.numel(), dtype=torch.uint8, device="cuda")
    qb = torch.zeros(w32.numel(), dtype=torch.uint8, device="cuda")
    calc.castFromFp32(qa, abi.FP8_143, a32, a32.numel(), fpBias=7, scale_exp=sa, clipFp=True)
    calc.castFromFp32(qb, abi.FP8_152, w32, w32.numel(), fpBias=15, col_scale_exp=sb, n_cols=N5, clipFp=True)
    torch.cuda.synchronize()
    del a32, w32
    col = (-sb).contiguous()
    A5 = MmeSimTensor([K5, M5, b5], 3, abi.FP8_143, qa, 7)
    B5 = MmeSimTensor([N5, K5, 1], 3, abi.FP8_152, qb, 15)
    # the output scale: bring the descaled results of a 256-row slab to the top of the fp8_143 range
    rows = 256
    slab = torch.zeros(rows * N5, dtype=torch.float32, device="cuda")
    calc.doBatchGemm(MmeSimTensor([N5, rows, 1], 3, abi.FP32, slab), MmeSimTensor([K5, rows, 1], 3, abi.FP8_143, qa, 7), B5, abi.OP_AB,
                     epilogue=Epilogue(scale_exp=-sa, col_scale_exp=col))
    calc.synchronize()
    so = pow2_scale_exp(float(slab.abs().max()) * 2.0, 240.0)  # (a factor of two of head room for the rows outside the slab)
    del slab
    o5 = torch.zeros(b5 * M5 * N5, dtype=torch.uint8, device="cuda")
    Y5 = MmeSimTensor([N5, M5, b5], 3, abi.FP8_143, o5, 7)
    e5 = Epilogue(scale_exp=so - sa, col_scale_exp=col, clipFp=True)
    t = b.timed(lambda: calc.doBatchGemm(Y5, A5, B5, abi.OP_AB, epilogue=e5), n=20, warm=3)
    flop = 2.0 * b5 * M5 * N5 * K5
    res = {"workload": "batched fp8 GEMM 4 x (2048 x 4096 . 4096 x 14336), A fp8_143 b7 per-tensor scale with 0.1 % outliers x20, B fp8_152 b15 per-channel "
                       "scales, fp8_143 output (configs[4]); library default policy for fp8 special codes", "value": round(flop / t / 1e12, 2),
           "unit": "TFLOP/s", "roofline": mfma_roofline(flop, t, "fp8", "gemm_fp8_persistent_chk_kernel<2, false>"),
           "scale_exp": {"a": sa, "out": so, "b_per_channel_min_max": [int(sb.min()), int(sb.max())]}}
    res["roofline"]["per_launch_us"] = b.per_launch(lambda: calc.doBatchGemm(Y5, A5, B5, abi.OP_AB, epilogue=e5), n=50, group=2)
    res["roofline"]["clock"] = b.clocked(lambda: calc.doBatchGemm(Y5, A5, B5, abi.OP_AB, epilogue=e5), n=10)
    if b.cpu:
        orc = b.oracle_lib()
        # 64 rows drawn at random over all four batch elements (16 of each): rows in the middle of the walk over the tiles
        r = 64
        prng = np.random.default_rng(55)
        rows = np.sort(np.concatenate([bz * M5 + prng.choice(M5, r // b5, replace=False) for bz in range(b5)]))
        ridx = torch.from_numpy(rows).cuda()
        a8 = qa.view(b5 * M5, K5)[ridx].cpu().numpy().ravel()
        b8 = qb.cpu().numpy()
        colh = col.cpu().numpy().astype(np.int32)
        acc = np.zeros(r * N5, np.float32)
        da, db, do = abi.make_tensor(a8.ctypes.data, [K5, r], abi.FP8_143, 7), abi.make_tensor(b8.ctypes.data, [N5, K5], abi.FP8_152, 15), \
            abi.make_tensor(acc.ctypes.data, [N5, r], abi.FP32)
        cpu_s, kind = b.cpu_gemm(do, da, db, abi.OP_AB)
        want = np.zeros(r * N5, np.uint8)
        assert orc.orc_cast_from_fp32(want.ctypes.data, abi.FP8_143, 7, 0, acc.ctypes.data, r * N5, so - sa, colh.ctypes.data, N5, 0, 0, 1, 0, 0) == 0
        got = o5.view(b5 * M5, N5)[ridx].cpu().numpy().ravel()
        dec = lambda c: _decode_fp8_143_b7(c)
        wf, gf = dec(want), dec(got)
        res["parity"] = {"rows_checked": r, "rows": "16 rows drawn at random from each of the 4 batch elements",
                         "rel_frobenius_vs_reference_fp8": float(np.linalg.norm(gf - wf) / np.linalg.norm(wf)),
                         "fp8_codes_equal_frac": float(np.mean(got == want)), "nonzero_codes_frac": float(np.mean((want & 0x7F) != 0)), "tolerance": 1e-2}
        res["cpu_baseline"] = {"value": round(2.0 * r * N5 * K5 / cpu_s / 1e12, 7), "unit": "TFLOP/s", "cores": b.threads, "kind": kind,
                               "sample": "%d rows drawn from all four batch elements against the full B (%.2f GFLOP of the 962 GFLOP job, doBatchGemm only), %.1f s wall"
                                         % (r, 2.0 * r * N5 * K5 / 1e9, cpu_s)}
    return res


def _decode_fp8_143_b7(codes):
    import numpy as np
    from intel_gaudi3_software_amd import abi
    from intel_gaudi3_software_amd.comparator import decode
    return decode(np.asarray(codes, np.uint8), abi.FP8_143, 7, 0).astype(np.float64)


def _cast_input(b, n):
    """N(0,1) * 2^U[-12, 12] with a 2^-10 share of special values (inf, NaN, zeros, huge, tiny)."""
    torch = b.torch
    gen = torch.Generator(device="cuda")
    gen.manual_seed(6006)
    x = torch.randn(n, device="cuda", generator=gen) * torch.exp2(torch.randint(-12, 13, (n,), device="cuda", generator=gen).float())
    pick = torch.rand(n, device="cuda", generator=gen) < 2.0 ** -10
    specials = torch.tensor([float("inf"), float("-inf"), float("nan"), 0.0, -0.0, 3.0e38, 1.0e-40, -2.0e-39], device="cuda")
    x = torch.where(pick, specials[torch.randint(0, 8, (n,), device="cuda", generator=gen)], x)
    return x.contiguous()


def _run_cast(b, which):
    import numpy as np
    torch, calc = b.torch, b.calc
    from intel_gaudi3_software_amd import abi
    n = 1 << 28
    x = _cast_input(b, n)
    ncpu = 1 << 24
    if which == "dequant":
        codes = torch.zeros(n, dtype=torch.uint8, device="cuda")
        calc.castFromFp32(codes, abi.FP8_143, x, n, fpBias=7, clipFp=True)
        calc.synchronize()
        t = b.timed(lambda: calc.castToFp32(x, codes, abi.FP8_143, n, fpBias=7), n=20)
        res = {"workload": "fp8_143 (bias 7) -> fp32 dequantise, 2^28 elements", "value": round(n * 5 / t / 1e9, 1), "unit": "GB/s",
               "roofline": hbm_roofline(n * 5.0, t, "cast_to_fp32_kernel")}
        res["roofline"]["per_launch_us"] = b.per_launch(lambda: calc.castToFp32(x, codes, abi.FP8_143, n, fpBias=7), n=50, group=2)
        if b.cpu:
            orc = b.oracle_lib()
            ch = codes[:ncpu].cpu().numpy()
            want = np.zeros(ncpu, np.float32)
            t0 = time.perf_counter()
            assert orc.orc_cast_to_fp32(want.ctypes.data, ch.ctypes.data, abi.FP8_143, 7, 0, ncpu, 0, None, 0) == 0
            cpu_s = time.perf_counter() - t0
            got = x[:ncpu].cpu().numpy()
            res["parity"] = {"bit_exact": bool(np.array_equal(got.view(np.uint32), want.view(np.uint32))), "elements_checked": ncpu}
            res["cpu_baseline"] = {"value": round(ncpu * 5 / cpu_s / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                                   "sample": "2^24 elements through the oracle's restatement of fp8_to_fp32 (the reference has no bulk dequantise entry point), %.2f s wall" % cpu_s}
        return res
    dt, ob, name, kern = (abi.FP8_143, 1, "fp32 -> fp8_143 (bias 7, RNE, saturation)", "cast_from_fp32_kernel<9>") if which == "fp8" else \
        (abi.BF16, 2, "fp32 -> bf16 (RNE, saturation)", "cast_from_fp32_kernel<12>")
    o = torch.zeros(n * ob, dtype=torch.uint8, device="cuda")
    t = b.timed(lambda: calc.castFromFp32(o, dt, x, n, fpBias=7 if ob == 1 else 0, clipFp=True), n=20)
    res = {"workload": "%s cast, 2^28 elements of N(0,1) * 2^U[-12,12] with 2^-10 specials" % name, "value": round(n * (4 + ob) / t / 1e9, 1), "unit": "GB/s",
           "roofline": hbm_roofline(n * (4.0 + ob), t, kern)}
    res["roofline"]["per_launch_us"] = b.per_launch(lambda: calc.castFromFp32(o, dt, x, n, fpBias=7 if ob == 1 else 0, clipFp=True), n=50, group=2)
    if b.cpu:
        xh = x[:ncpu].cpu().numpy()
        want = np.zeros(ncpu * ob, np.uint8)
        do = abi.make_tensor(want.ctypes.data, [ncpu], dt, 7 if ob == 1 else 0)
        da = abi.make_tensor(xh.ctypes.data, [ncpu], abi.FP32)
        cpu_s, kind = b.cpu_activation(do, da)
        got = o[:ncpu * ob].cpu().numpy()
        res["parity"] = {"bit_exact": bool(np.array_equal(got, want)), "elements_checked": ncpu}
        res["cpu_baseline"] = {"value": round(ncpu * (4 + ob) / cpu_s / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": kind,
                               "sample": "2^24 elements through doActivation (single-threaded by construction), %.2f s wall" % cpu_s}
    return res


WORKLOADS = {"c1": run_c1, "c3": run_c3, "c4_dedx": run_c4_dedx, "c4_dedw": run_c4_dedw, "c5": run_c5,
             "cast_fp8_143": lambda b: _run_cast(b, "fp8"), "cast_bf16": lambda b: _run_cast(b, "bf16"),
             "dequant_fp8_143": lambda b: _run_cast(b, "dequant")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="time the headline workload only")
    ap.add_argument("--only", default=None, help="run one workload only (c2 or one of: %s), e.g. under a profiler" % ", ".join(SECONDARY))
    ap.add_argument("--cpu-rows", type=int, default=256, help="rows of A in the CPU baseline's M-slab")
    ap.add_argument("--plain", action="store_true", help="the timed regions only: no per-call distribution, no rotating operand sets, no clock probe, no "
                    "matrix-core ceiling (what the profiles under profiles/ are taken with, so that a traced average is the average of the timed calls)")
    ap.add_argument("--extra", action="store_true", help="also time further shapes and operand types (fp16 / ufp16 / fp32 GEMMs, fp8 convolutions, host-pointer calls)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also launch a plain elementwise copy of 2^26 floats (256 MiB read, 256 MiB written) a few times: a "
                         "counter run (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) scales the GEMM kernel's reading by this kernel's")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path has no multi-GPU part in this build (--gpus %d refused)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    b = Bench(args)
    if args.pmc_calibration:
        b.pmc_calibration()
    if args.only and args.only != "c2":
        if args.only not in WORKLOADS:
            print("unknown workload %r" % args.only, file=sys.stderr)
            sys.exit(2)
        res = WORKLOADS[args.only](b)
        attach_profile(res["roofline"], args.only)
        print(json.dumps({args.only: res}))
        b.calc.close()
        return
    result = run_c2(b)
    if not args.no_secondary and not args.only:
        result["secondary"] = {}
        for name in SECONDARY:
            result["secondary"][name] = WORKLOADS[name](b)
            attach_profile(result["secondary"][name]["roofline"], name)
            b.torch.cuda.empty_cache()
    if args.extra:
        result["extra"] = extra_measurements(b.calc, b.stream)
    print(json.dumps(result))
    b.calc.close()


def extra_measurements(calc, stream):
    """Further shapes and operand types, each with its own roofline line (device-resident, events); not baseline configurations."""
    import numpy as np
    import torch
    from intel_gaudi3_software_amd import ConvolutionParams, MmeSimTensor, abi

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
    cp = ConvolutionParams(2, [1, 1, 0, 0])
    # the c4 layer with Gaudi fp8 operands (fp8_143 activations, bias 7; fp8_152 gradients, bias 15): fwd, dedx, dedw
    Cc = Kk = 256
    H = Wd = 28
    B = 32
    xs, ws, ys = [Cc, Wd, H, 1, B], [Kk, Cc, 3, 3, 1], [Kk, Wd, H, 1, B]
    fl = 2.0 * B * H * Wd * Kk * Cc * 9
    q8 = lambda n, hi: torch.randint(0, hi, (n,), dtype=torch.uint8, device="cuda")
    X8 = MmeSimTensor(xs, 5, abi.FP8_143, q8(int(np.prod(xs)), 0x60), 7)
    W8 = MmeSimTensor(ws, 5, abi.FP8_143, q8(int(np.prod(ws)), 0x40), 7)
    Y8 = MmeSimTensor(ys, 5, abi.FP8_152, q8(int(np.prod(ys)), 0x70), 15)
    YO = MmeSimTensor(ys, 5, abi.FP32, torch.zeros(int(np.prod(ys)), dtype=torch.float32, device="cuda"))
    DX = MmeSimTensor(xs, 5, abi.FP32, torch.zeros(int(np.prod(xs)), dtype=torch.float32, device="cuda"))
    DW = MmeSimTensor(ws, 5, abi.FP32, torch.zeros(int(np.prod(ws)), dtype=torch.float32, device="cuda"))
    t = timed(lambda: calc.doConvolution(YO, X8, W8, YO, cp, abi.OP_FWD), n=20)
    res["conv_fwd_fp8_143_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_fp8_peak": fl / t / 1e12 / PEAK_TFLOPS["fp8"]}
    t = timed(lambda: calc.doConvolution(DX, X8, W8, Y8, cp, abi.OP_DEDX), n=20)
    res["conv_dedx_fp8_152x143_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_fp8_peak": fl / t / 1e12 / PEAK_TFLOPS["fp8"]}
    t = timed(lambda: calc.doConvolution(DW, X8, W8, Y8, cp, abi.OP_DEDW), n=20)
    res["conv_dedw_fp8_143x152_n32_28x28_c256_k256_3x3"] = {"seconds": t, "TFLOP/s": fl / t / 1e12, "frac_fp8_peak": fl / t / 1e12 / PEAK_TFLOPS["fp8"]}
    del DX, DW, X8, W8, Y8, YO
    # fp8 GEMM with A stored K x M ("atb": A read through transposing LDS loads)
    nt = 4096
    qt = lambda: torch.randint(0, 0x60, (nt * nt,), dtype=torch.uint8, device="cuda")
    AT, BT = MmeSimTensor([nt, nt], 2, abi.FP8_143, qt(), 7), MmeSimTensor([nt, nt], 2, abi.FP8_143, qt(), 7)
    YT8 = MmeSimTensor([nt, nt], 2, abi.FP32, torch.zeros(nt * nt, dtype=torch.float32, device="cuda"))
    t = timed(lambda: calc.doBatchGemm(YT8, AT, BT, abi.OP_ATB), n=20)
    res["gemm_fp8_143_atb_4096x4096x4096_fp32_out"] = {"seconds": t, "TFLOP/s": 2.0 * nt ** 3 / t / 1e12, "frac_fp8_peak": 2.0 * nt ** 3 / t / 1e12 / PEAK_TFLOPS["fp8"]}
    # the host-pointer (reference-compatible) entry point on the same shape: operands and the fp32 result cross the host link
    ah, bh = AT.data().cpu().numpy(), BT.data().cpu().numpy()
    oh = np.zeros(nt * nt, np.float32)
    HA, HB, HO = MmeSimTensor([nt, nt], 2, abi.FP8_143, ah, 7), MmeSimTensor([nt, nt], 2, abi.FP8_143, bh, 7), MmeSimTensor([nt, nt], 2, abi.FP32, oh)
    calc.doBatchGemm(HO, HA, HB, abi.OP_AB)
    t0 = time.perf_counter()
    for _ in range(5):
        calc.doBatchGemm(HO, HA, HB, abi.OP_AB)
    th = (time.perf_counter() - t0) / 5
    moved = 2.0 * nt * nt + 4.0 * nt * nt
    res["host_pointer_gemm_fp8_143_4096x4096x4096_fp32_out"] = {"seconds": th, "TFLOP/s": 2.0 * nt ** 3 / th / 1e12, "bytes_over_the_host_link": moved,
                                                                 "GB/s_over_the_host_link": moved / th / 1e9}
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
