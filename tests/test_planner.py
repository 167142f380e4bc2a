"""The planner (mme_hip_plan_batch_gemm / mme_hip_plan_convolution): which kernel form a call would launch, answered by the
library's own checking and planning code on a handle without a device.  No GPU needed.  Held to (a) the forms an MI355X
reported after really launching every distinct contraction of the reference's Gaudi3 test configurations
(tests/golden/contraction_forms.json, written by tests/golden/gen_contraction_forms.py) and (b) what the benchmark
configurations are documented to take."""
import json
import os

import pytest

from intel_gaudi3_software_amd import abi, harness

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "contraction_forms.json")
P = 4096  # stands in for a 16-byte aligned device address: the planner never dereferences it


def T(sizes, dtype, bias=0, mode=0, strides=None):
    return abi.make_tensor(P, sizes, dtype, bias, mode, strides, dim=5)


def _plan_record(r):
    a_l, b_l, o_l = {"dedx": ("y", "w", "x"), "transposed_dedx": ("y", "w", "x"), "dedw": ("x", "y", "w")}.get(r["op"], ("x", "w", "y"))
    t = {"in_type": r["in_type"], "in2_type": r["in2_type"], "out_type": abi.FP32, "fp8_bias_in": 7 if r["in_type"] == abi.FP8_143 else 15,
         "fp8_bias_in2": 7 if r["in2_type"] == abi.FP8_143 else 15, "fp8_bias_out": 0, "inf_nan_a": 0, "inf_nan_b": 0, "inf_nan_out": 0}
    bias = {abi.FP8_143: 7, abi.FP8_152: 15, abi.FP16: 15, abi.UFP16: 31}
    d = {a_l: T(r[a_l], r["in_type"], bias.get(r["in_type"], 0), 0, r[a_l + "_strides"]),
         b_l: T(r[b_l], r["in2_type"], bias.get(r["in2_type"], 0), 0, r[b_l + "_strides"])}
    acc = T(r[o_l], abi.FP32, 0, 0, r[o_l + "_strides"])
    op = harness._OPS[r["op"]]
    if op in harness._CONV_OPS:
        cp = abi.make_conv_params(3, tuple(r["padding"]) + (0,), tuple(r["conv_strides"]) + (1,), tuple(r["dilation"]) + (1,))
        return abi.plan_convolution(acc, d.get("x", acc), d.get("w", acc), d.get("y", acc), cp, op)
    return abi.plan_batch_gemm(acc, d[a_l], d[b_l], op)


def test_planner_reproduces_the_forms_the_gpu_reported():
    rows = json.load(open(GOLDEN))
    assert len(rows) == 197
    large = 0
    for r in rows:
        got = _plan_record(r)
        # (the 3 x 3 forward kernel reports its own form since the records were written; none of these cases takes it)
        assert got["large_tile"] in (0, 1)
        assert got == r["form"], (r["file"], r["op"], r["x"], r["w"], got, r["form"])
        large += got["large_tile"] == 1
    # what the record says about shapes that miss the large-tile kernels: 26 of 197 take one, 22 of the 81 with >= 0.2 GFLOP
    assert large == 26
    big = [r for r in rows if r["flops"] >= 2e8]
    assert len(big) == 81 and sum(1 for r in big if r["form"]["large_tile"] == 1) == 22


def test_planner_on_the_benchmark_configurations():
    e = abi.Epilogue()
    e.scale_exp, e.clip_fp = -10, 1
    # fp8 4096^3 -> bf16: one round of 256 x 256 tiles, four wavefronts of 128 x 128
    assert abi.plan_batch_gemm(T([4096, 4096], abi.BF16), T([4096, 4096], abi.FP8_143, 7), T([4096, 4096], abi.FP8_143, 7), abi.OP_AB, e) == \
        {"large_tile": 1, "tile_rows": 256, "split_k": 1, "wavefronts": 4}
    # ... a short reduction keeps eight wavefronts, and so does a shape with several rounds of tiles
    assert abi.plan_batch_gemm(T([4096, 4096], abi.BF16), T([1024, 4096], abi.FP8_143, 7), T([4096, 1024], abi.FP8_143, 7), abi.OP_AB, e)["wavefronts"] == 8
    assert abi.plan_batch_gemm(T([8192, 8192], abi.BF16), T([4096, 8192], abi.FP8_143, 7), T([8192, 4096], abi.FP8_143, 7), abi.OP_AB, e)["wavefronts"] == 8
    # bf16 512^3: 128-row tiles (four 256-row tiles would use four compute units)
    assert abi.plan_batch_gemm(T([512, 512], abi.FP32), T([512, 512], abi.BF16), T([512, 512], abi.BF16), abi.OP_AB) == \
        {"large_tile": 1, "tile_rows": 128, "split_k": 1, "wavefronts": 8}
    # the batched mixed-fp8 GEMM: 256-row tiles, no split (the persistent walk)
    e5 = abi.Epilogue()
    e5.scale_exp, e5.clip_fp, e5.col_scale_exp = 2, 1, P
    assert abi.plan_batch_gemm(T([14336, 2048, 4], abi.FP8_143, 7), T([4096, 2048, 4], abi.FP8_143, 7), T([14336, 4096, 1], abi.FP8_152, 15), abi.OP_AB, e5) == \
        {"large_tile": 1, "tile_rows": 256, "split_k": 1, "wavefronts": 8}
    cp = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
    xs, ws, ys = [256, 28, 28, 1, 32], [256, 256, 3, 3, 1], [256, 28, 28, 1, 32]
    X, W, Y = T(xs, abi.BF16), T(ws, abi.BF16), T(ys, abi.BF16)
    assert abi.plan_convolution(T(xs, abi.FP32), T(xs, abi.FP32), W, Y, cp, abi.OP_DEDX) == {"large_tile": 1, "tile_rows": 128, "split_k": 1, "wavefronts": 8}
    assert abi.plan_convolution(T(ws, abi.FP32), X, T(ws, abi.FP32), Y, cp, abi.OP_DEDW) == {"large_tile": 1, "tile_rows": 128, "split_k": 14, "wavefronts": 8}
    xs, ws, ys = [64, 56, 56, 1, 64], [64, 64, 3, 3, 1], [64, 56, 56, 1, 64]
    ec = abi.Epilogue()
    ec.clip_fp = 1
    assert abi.plan_convolution(T(ys, abi.BF16), T(xs, abi.BF16), T(ws, abi.BF16), T(ys, abi.BF16), cp, abi.OP_FWD, ec)["large_tile"] == 2


def test_planner_shows_the_cliff_of_one_odd_dimension():
    """A reduction length that is not a multiple of 128 bytes, or rows that are not 16-byte aligned, leave the large-tile
    kernels: the planner makes that visible without a GPU."""
    ok = abi.plan_batch_gemm(T([4096, 4096], abi.FP32), T([4096, 4096], abi.BF16), T([4096, 4096], abi.BF16), abi.OP_AB)
    assert ok["large_tile"] == 1
    for k in (4100, 4104, 4128):
        odd = abi.plan_batch_gemm(T([4096, 4096], abi.FP32), T([k, 4096], abi.BF16), T([4096, k], abi.BF16), abi.OP_AB)
        assert odd["large_tile"] == 0, k
    assert abi.plan_batch_gemm(T([4096, 4096], abi.FP32), T([4160, 4096], abi.BF16), T([4096, 4160], abi.BF16), abi.OP_AB)["large_tile"] == 1
    # partial tiles are taken (N a multiple of 16 from 128 columns, any M from 64 rows)
    assert abi.plan_batch_gemm(T([4000, 3000], abi.FP32), T([4096, 3000], abi.BF16), T([4000, 4096], abi.BF16), abi.OP_AB)["large_tile"] == 1
    assert abi.plan_batch_gemm(T([4001, 3000], abi.FP32), T([4096, 3000], abi.BF16), T([4001, 4096], abi.BF16), abi.OP_AB)["large_tile"] == 0


def test_planner_refuses_what_the_calculator_refuses():
    with pytest.raises(ValueError, match="Common dim"):
        abi.plan_batch_gemm(T([512, 512], abi.FP32), T([512, 512], abi.BF16), T([512, 500], abi.BF16), abi.OP_AB)
    with pytest.raises(ValueError, match="mixed input type"):
        abi.plan_batch_gemm(T([512, 512], abi.FP32), T([512, 512], abi.BF16), T([512, 512], abi.FP32), abi.OP_AB)
    # a zero-size common dimension launches no contraction kernel
    assert abi.plan_batch_gemm(T([8, 8], abi.FP32), T([0, 8], abi.BF16), T([8, 0], abi.BF16), abi.OP_AB)["large_tile"] == -1
    # the fp8 policy is part of the plan's input (it does not change the form, only what rides along)
    a = abi.plan_batch_gemm(T([4096, 4096], abi.FP32), T([4096, 4096], abi.FP8_143, 7), T([4096, 4096], abi.FP8_143, 7), abi.OP_AB,
                            fp8_specials_policy=abi.FP8_SPECIALS_ASSUME_NONE)
    assert a["large_tile"] == 1 and a["wavefronts"] == 4
    # a stochastic epilogue plans through the fp32 intermediate
    e = abi.Epilogue()
    e.rounding_mode = 4
    assert abi.plan_batch_gemm(T([512, 512], abi.BF16), T([512, 512], abi.BF16), T([512, 512], abi.BF16), abi.OP_AB, e)["large_tile"] == 1


def test_planner_through_the_cpp_header():
    """MmeHip::Calculator::planBatchGemm / planConvolution (include/mme_hip_calculator.h) in tests/cpp/plan_calculator.cpp, built
    by intel_gaudi3_software_amd.build.build_cpp_tests() and run as a child process; no GPU."""
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = os.path.join(root, "tests", "cpp", "plan_calculator")
    if not os.path.exists(exe):  # (host code only: g++ over the header, two seconds)
        from intel_gaudi3_software_amd import build
        build.build_cpp_tests()
    r = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=60)
    text = r.stdout.decode(errors="replace")
    print(text)
    assert r.returncode == 0, text
    assert text.count("ok    ") == 4 and "all ok" in text and "FAILED" not in text


def test_planned_forms_respect_what_the_kernels_assume():
    """The large-tile kernels count on whole 64-byte stages in even numbers, at least six per k-slice, operand rows that are
    multiples of 16 bytes and outputs in groups of 16 columns; the four-wavefront form on fp8 operands, whole 256-row tiles in
    one round and a long reduction.  Whatever the planner picks for a few thousand shapes around the boundaries must stay
    inside those assumptions (a plan outside them would be a launch that reads or writes out of bounds)."""
    import numpy as np
    rng = np.random.default_rng(2024)
    es_of = {abi.BF16: 2, abi.FP16: 2, abi.FP8_143: 1, abi.FP8_152: 1}
    seen_split = seen_w4 = seen_128 = seen_large = 0
    for trial in range(4000):
        dt = [abi.BF16, abi.FP16, abi.FP8_143, abi.FP8_152][int(rng.integers(4))]
        es = es_of[dt]
        bias = {abi.FP8_143: 7, abi.FP8_152: 15, abi.FP16: 15}.get(dt, 0)
        pick = lambda unit, hi: int(rng.integers(1, hi)) * unit + (int(rng.integers(0, unit)) if rng.random() < 0.2 else 0)
        M, N, K = pick(64, 80), pick(64, 80), pick(64, 160)
        nb = int(rng.choice([1, 1, 1, 2, 5]))
        op = int(rng.choice([abi.OP_AB, abi.OP_ABT, abi.OP_ATB, abi.OP_ATBT]))
        if trial % 10 == 0:
            # the neighbourhood of the four-wavefront form: fp8, whole 256-row tiles around one round, long reductions
            dt, es, bias = abi.FP8_143, 1, 7
            M, N, K, nb = 256 * int(rng.integers(4, 20)), 256 * int(rng.integers(4, 20)), 128 * int(rng.integers(16, 40)), int(rng.choice([1, 1, 2]))
            op = int(rng.choice([abi.OP_AB, abi.OP_ABT]))
        ta, tb = op in (abi.OP_ATB, abi.OP_ATBT), op in (abi.OP_ABT, abi.OP_ATBT)
        x = T([M, K, nb] if ta else [K, M, nb], dt, bias)
        w = T([K, N, nb] if tb else [N, K, nb], dt, bias)
        f = abi.plan_batch_gemm(T([N, M, nb], abi.FP32), x, w, op, num_cus=256, fp8_specials_policy=int(rng.integers(2)))
        if f["large_tile"] != 1:
            continue
        seen_large += 1
        kb = K * es
        assert kb % 128 == 0 and kb >= 384, (M, N, K, dt, f)
        assert N % 16 == 0 and N >= 128 and M >= 64, (M, N, K, dt, f)
        # operand rows in multiples of 16 bytes
        assert ((M if ta else K) * es) % 16 == 0 and ((K if tb else N) * es) % 16 == 0, (M, N, K, op, dt, f)
        assert f["tile_rows"] in (128, 256) and f["wavefronts"] in (4, 8) and f["split_k"] >= 1
        nk = kb // 64
        if f["split_k"] > 1:
            seen_split += 1
            assert nk % (2 * f["split_k"]) == 0 and nk // f["split_k"] >= 6, (M, N, K, dt, f)
        if f["tile_rows"] == 128:
            seen_128 += 1
        if f["wavefronts"] == 4:
            seen_w4 += 1
            tiles = (M // 256) * (N // 256) * nb
            assert es == 1 and not ta and M % 256 == 0 and N % 256 == 0 and f["tile_rows"] == 256 and f["split_k"] == 1 and tiles <= 256 and nk >= 48, (M, N, K, f)
        if ta and (M % 256 or N % 256):
            # A contiguous along the tile's rows has no partial-tile kernels (the 2-byte types: whole 128- or 256-row tiles)
            assert es == 2 and M % 128 == 0 and N % 256 == 0, (M, N, K, op, f)
    assert seen_large > 500 and seen_split > 20 and seen_128 > 20 and seen_w4 > 5, (seen_large, seen_split, seen_128, seen_w4)


def test_planned_convolution_forms_respect_what_the_gather_kernels_assume():
    """The same for convolutions: the gather of fwd / dedx stages whole 64-byte runs of channels inside one filter tap (at most 32
    taps), dedw 16-byte runs; dedx in gather form exists for unit convolution strides only; the weights' channel extents are
    16-byte multiples; k-slices hold an even number of stages, at least six."""
    import numpy as np
    rng = np.random.default_rng(77)
    large = {abi.OP_FWD: 0, abi.OP_DEDX: 0, abi.OP_DEDW: 0}
    split = 0
    for trial in range(3000):
        dt = [abi.BF16, abi.FP16, abi.FP8_143][int(rng.integers(3))]
        es = 1 if dt == abi.FP8_143 else 2
        bias = {abi.FP8_143: 7, abi.FP16: 15}.get(dt, 0)
        C = int(rng.choice([8, 16, 24, 32, 48, 64, 96, 128, 200, 256, 320]))
        Kc = int(rng.choice([16, 64, 100, 128, 192, 256, 320, 512]))
        S, R, Q = int(rng.integers(1, 4)), int(rng.integers(1, 4)), int(rng.choice([1, 1, 1, 2, 4]))
        W, H, D, B = int(rng.integers(6, 40)), int(rng.integers(6, 40)), int(rng.choice([1, 1, 3])), int(rng.integers(1, 9))
        st = [int(rng.choice([1, 1, 1, 2])) for _ in range(3)]
        di = [int(rng.choice([1, 1, 1, 2])) for _ in range(3)]
        pad = [int(rng.integers(0, 2)) for _ in range(3)]
        if D == 1:
            Q, st[2], di[2], pad[2] = 1, 1, 1, 0
        out = [(n + 2 * p - d * (k - 1) - 1) // s + 1 for n, p, d, k, s in zip((W, H, D), pad, di, (S, R, Q), st)]
        if min(out) < 1:
            continue
        xs, ws, ys = [C, W, H, D, B], [Kc, C, S, R, Q], [Kc, out[0], out[1], out[2], B]
        cp = abi.make_conv_params(3, tuple(pad) + (0,), tuple(st) + (1,), tuple(di) + (1,))
        op = [abi.OP_FWD, abi.OP_DEDX, abi.OP_DEDW][int(rng.integers(3))]
        X, Wt, Y = T(xs, dt, bias), T(ws, dt, bias), T(ys, dt, bias)
        if op == abi.OP_FWD:
            f = abi.plan_convolution(T(ys, abi.FP32), X, Wt, T(ys, abi.FP32), cp, op)
        elif op == abi.OP_DEDX:
            f = abi.plan_convolution(T(xs, abi.FP32), T(xs, abi.FP32), Wt, Y, cp, op)
        else:
            f = abi.plan_convolution(T(ws, abi.FP32), X, T(ws, abi.FP32), Y, cp, op)
        if f["large_tile"] != 1:
            continue
        large[op] += 1
        taps = S * R * Q
        assert taps <= 32, (xs, ws, f)
        nch, n_out = (C, Kc) if op == abi.OP_FWD else ((Kc, C) if op == abi.OP_DEDX else (C, Kc))
        assert n_out % 16 == 0 and n_out >= 128, (op, xs, ws, f)
        if op == abi.OP_DEDW:
            assert (nch * es) % 16 == 0, (xs, ws, f)
            kb = B * out[0] * out[1] * out[2] * es   # the reduction runs over the output pixels
        else:
            assert (nch * es) % 64 == 0, (op, xs, ws, f)
            kb = taps * nch * es
        if op == abi.OP_DEDX:
            assert st == [1, 1, 1], (xs, ws, st, f)
        assert kb % 128 == 0 and kb >= 384, (op, xs, ws, ys, f)
        if f["split_k"] > 1:
            split += 1
            nk = kb // 64
            assert nk % (2 * f["split_k"]) == 0 and nk // f["split_k"] >= 6, (op, xs, ws, f)
    assert min(large.values()) > 20 and split > 10, (large, split)
