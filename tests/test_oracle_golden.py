"""Pins the oracle (oracle/mme_oracle.c) without the reference tree:
 - the known answers of the reference's own unit tests (tests/golden/kat_vectors.json),
 - vectors written by the compiled reference (tests/golden/ref_vectors.npz, see gen_golden.py),
 - what the mathematics fixes (identities, monotonicity, IEEE conversions of torch, exact fp64 sums, direct convolution).
"""
import ctypes as C
import json
import os

import numpy as np
import pytest

from intel_gaudi3_software_amd import abi
from helpers import A, bf16_bits_to_f32, decode_fp8, decode_operand, desc, quantize_fp8, random_operand, to_bf16_bits

HERE = os.path.dirname(os.path.abspath(__file__))
DT = {"fp8_143": abi.FP8_143, "fp8_152": abi.FP8_152, "bf16": abi.BF16, "fp32": abi.FP32}


@pytest.fixture(scope="module")
def kat():
    with open(os.path.join(HERE, "golden", "kat_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(HERE, "golden", "ref_vectors.npz"))


def _fill(orc, dt, value, n, bias):
    if dt == abi.FP32:
        return np.full(n, value, np.float32)
    if dt == abi.BF16:
        return np.full(n, orc.orc_fp32_to_bf16(int(np.float32(value).view(np.uint32)), 0, 0, 0, 0, 0), np.uint16)
    E = 4 if dt == abi.FP8_143 else 5
    code = orc.orc_fp32_to_fp8(int(np.float32(value).view(np.uint32)), E, 7 - E, bias, 0, 0, 0, 0, 0, 0, 0)
    return np.full(n, code, np.uint8)


# ---- the reference's own known answers ---------------------------------------------------------------------------------
def test_kat_bf16(orc, kat):
    for v in kat["bf16"]:
        bits = int(v["bits"], 16)
        assert (bits << 16) == int(v["fp32_bits"], 16)
        assert (((bits >> 7) & 0xFF) == 0xFF and (bits & 0x7F) == 0) == v["is_inf"]
    # bf16_t::max() is what the saturating conversion of FLT_MAX gives
    assert orc.orc_fp32_to_bf16(0x7F7FFFFF, 0, 0, 1, 0, 0) == 0x7F7F


def test_kat_fp8_convert_and_mul(orc, kat):
    for v in kat["fp8_convert"]:
        E = 4 if v["dtype"] == "fp8_143" else 5
        code = orc.orc_fp32_to_fp8(int(np.float32(v["value"]).view(np.uint32)), E, 7 - E, v["bias"], 0, 0, 0, 0, 0, 0, 0)
        assert code == int(v["code"], 16)
        back = np.uint32(orc.orc_fp8_to_fp32(code, E, 7 - E, v["bias"], 0)).view(np.float32)
        assert back == np.float32(v["value"])
    for v in kat["fp8_mul"]:
        E = 4 if v["dtype"] == "fp8_143" else 5
        f = lambda x: np.uint32(orc.orc_fp8_to_fp32(orc.orc_fp32_to_fp8(int(np.float32(x).view(np.uint32)), E, 7 - E, v["bias"], 0,
                                                                          0, 0, 0, 0, 0, 0), E, 7 - E, v["bias"], 0)).view(np.float32)
        assert f(v["a"]) * f(v["b"]) == np.float32(v["product"])


def test_kat_gemm_fill(orc, kat):
    for v in kat["gemm_fill"]:
        dt = DT[v["dtype"]]
        a = _fill(orc, dt, v["a"], int(np.prod(v["a_sizes"])), v["bias"])
        b = _fill(orc, dt, v["b"], int(np.prod(v["b_sizes"])), v["bias"])
        y = np.zeros(int(np.prod(v["y_sizes"])), np.float32)
        da, db, dy = desc(a, v["a_sizes"], dt, v["bias"]), desc(b, v["b_sizes"], dt, v["bias"]), desc(y, v["y_sizes"], abi.FP32)
        assert orc.orc_batch_gemm(A(dy), A(da), A(db), abi.OP_AB) == 0, orc.orc_last_error()
        assert np.all(y == np.float32(v["expect"])), v["src"]
        if v.get("then_cast") == "bf16":
            o = np.zeros(y.size, np.uint16)
            do = desc(o, v["y_sizes"], abi.BF16)
            assert orc.orc_activation(A(do), A(dy), 0, 0, 0, 0, 0, 0, None, 0) == 0
            assert np.all(bf16_bits_to_f32(o) == np.float32(v["expect"]))


def test_kat_conv_smoke(orc, kat):
    """The reference only checks that these run; every tap sees 0.5 * -0.5 products, so the sums are closed forms."""
    for v in kat["conv_smoke"]:
        dt = DT[v["dtype"]]
        x = _fill(orc, dt, v["x"], 25, v["bias"])
        w = np.zeros(25, np.uint8)
        w[:v["w_filled"]] = _fill(orc, dt, v["w"], v["w_filled"], v["bias"])
        y = np.zeros(25, np.float32)
        dx, dw, dy = desc(x, v["x_sizes"], dt, v["bias"]), desc(w, v["w_sizes"], dt, v["bias"]), desc(y, v["y_sizes"], abi.FP32)
        p = abi.make_conv_params(v["dim"])
        assert orc.orc_convolution(A(dy), A(dx), A(dw), A(dy), A(p), abi.OP_FWD, 0) == 0, orc.orc_last_error()
        # x = [C=5, W=5], w = [K=5, C=5]: Y[w][k] = sum_c x[w][c] * W[c][k]; only the first 4 weights (c=0, k=0..3) are set
        want = np.zeros((5, 5), np.float32)
        want[:, :4] = v["x"] * v["w"]
        assert np.array_equal(y.reshape(5, 5), want)


# ---- vectors from the compiled reference -------------------------------------------------------------------------------
def test_golden_decode_tables(orc, gold):
    codes = np.arange(256, dtype=np.uint8)
    for (E, M, bias, mode), tab in zip(gold["decode_cfg"], gold["decode_tab"]):
        t = np.zeros(256, np.uint32)
        orc.orc_fp8_to_fp32_n(t.ctypes.data, codes.ctypes.data, 256, int(E), int(M), int(bias), int(mode))
        assert np.array_equal(t, tab), (E, M, bias, mode)


def test_golden_casts(orc, gold):
    x, lf = np.ascontiguousarray(gold["cast_in"]), np.ascontiguousarray(gold["cast_lfsr"])
    for cfg, want in zip(gold["fp8_cfg"], gold["fp8_out"]):
        E, M, bias, mode, rm, clip, cinf, ftz, sftz = (int(v) for v in cfg)
        o = np.zeros(x.size, np.uint8)
        orc.orc_fp32_to_fp8_n(o.ctypes.data, x.ctypes.data, x.size, E, M, bias, rm, lf.ctypes.data, ftz, clip, cinf, sftz, mode)
        assert np.array_equal(o, want), tuple(cfg)
    for cfg, w16, w32 in zip(gold["bf16_cfg"], gold["bf16_out"], gold["fp32_out"]):
        rm, clip, cinf, ftz = (int(v) for v in cfg)
        o = np.zeros(x.size, np.uint16)
        orc.orc_fp32_to_bf16_n(o.ctypes.data, x.ctypes.data, x.size, rm, lf.ctypes.data, clip, ftz, cinf)
        assert np.array_equal(o, w16), tuple(cfg)
        o32 = np.zeros(x.size, np.uint32)
        orc.orc_fp32_to_fp32_n(o32.ctypes.data, x.ctypes.data, x.size, rm, clip, ftz, cinf)
        assert np.array_equal(o32, w32), tuple(cfg)


def test_golden_add_and_tree(orc, gold):
    a, b = np.ascontiguousarray(gold["add_a"]), np.ascontiguousarray(gold["add_b"])
    for rm in range(4):
        o = np.zeros(a.size, np.uint32)
        orc.orc_add_fp32_n(o.ctypes.data, a.ctypes.data, b.ctypes.data, a.size, rm)
        assert np.array_equal(o, gold["add_out"][rm]), rm
    for emul in (0, 1):
        Aa, Bb = np.ascontiguousarray(gold["tree%d_a" % emul]), np.ascontiguousarray(gold["tree%d_b" % emul])
        o = np.zeros(Aa.shape[0], np.uint32)
        orc.orc_tree9_n(o.ctypes.data, Aa.ctypes.data, Bb.ctypes.data, Aa.shape[0], emul)
        assert np.array_equal(o, gold["tree%d_out" % emul]), emul


def test_golden_gemm(orc, gold):
    for i in range(int(gold["gemm_count"][0])):
        dtA, dtB, bA, bB, mA, mB, op, M, N, K = (int(v) for v in gold["gemm%d_meta" % i])
        a = np.ascontiguousarray(gold["gemm%d_a" % i]).view(abi.DTYPE_NUMPY[dtA])
        b = np.ascontiguousarray(gold["gemm%d_b" % i]).view(abi.DTYPE_NUMPY[dtB])
        ta, tb = op in (abi.OP_ATB, abi.OP_ATBT), op in (abi.OP_ABT, abi.OP_ATBT)
        asz, bsz = ([M, K] if ta else [K, M]) + [2, 1, 1], ([K, N] if tb else [N, K]) + [1, 1, 1]
        o = np.zeros(M * N * 2, np.float32)
        da, db, do = desc(a, asz, dtA, bA, mA), desc(b, bsz, dtB, bB, mB), desc(o, [N, M, 2, 1, 1], abi.FP32)
        assert orc.orc_batch_gemm(A(do), A(da), A(db), op) == 0
        assert np.array_equal(o.view(np.uint32), gold["gemm%d_out" % i]), i


def test_golden_conv(orc, gold):
    for i in range(int(gold["conv_count"][0])):
        m = [int(v) for v in gold["conv%d_meta" % i]]
        dt, bias, op, rm = m[:4]
        xs, ws, ys, pad, st, dil = m[4:9], m[9:14], m[14:19], m[19:22], m[22:25], m[25:28]
        x = np.ascontiguousarray(gold["conv%d_x" % i]).view(abi.DTYPE_NUMPY[dt])
        w = np.ascontiguousarray(gold["conv%d_w" % i]).view(abi.DTYPE_NUMPY[dt])
        y = np.ascontiguousarray(gold["conv%d_y" % i]).view(abi.DTYPE_NUMPY[dt])
        os_ = {abi.OP_FWD: ys, abi.OP_DEDX: xs, abi.OP_DEDW: ws}[op]
        o = np.zeros(int(np.prod(os_)), np.float32)
        p = abi.make_conv_params(2, pad, st, dil)
        dx, dw, dy, do = desc(x, xs, dt, bias), desc(w, ws, dt, bias), desc(y, ys, dt, bias), desc(o, os_, abi.FP32)
        assert orc.orc_convolution(A(do), A(dx), A(dw), A(dy), A(p), op, rm) == 0
        assert np.array_equal(o.view(np.uint32), gold["conv%d_out" % i]), (i, op, rm)


def test_golden_activation_stochastic(orc, gold):
    acc0 = np.ascontiguousarray(gold["act_acc"]).view(np.float32)
    for i in range(int(gold["act_count"][0])):
        dt, bias, rm, sftz, ftz, poly = (int(v) for v in gold["act%d_meta" % i])
        a = acc0.copy()
        o = np.zeros(a.size * abi.DTYPE_SIZE[dt], np.uint8)
        l = np.ascontiguousarray(gold["act_lfsr"]).copy()
        do, da = desc(o, [64, 10], dt, bias), desc(a, [64, 10], abi.FP32)
        assert orc.orc_activation(A(do), A(da), 0, rm, 1, 0, ftz, sftz, l.ctypes.data, poly) == 0
        assert np.array_equal(o, gold["act%d_out" % i]), i


# ---- what the mathematics fixes ----------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt,biases", [(abi.FP8_143, [3, 7, 11, 15]), (abi.FP8_152, [1, 8, 15, 30])])
def test_fp8_roundtrip_monotone_symmetric(orc, dt, biases):
    E = 4 if dt == abi.FP8_143 else 5
    codes = np.arange(256, dtype=np.uint8)
    for bias in biases:
        for mode in (0, 1, 2):
            val = decode_fp8(orc, codes, dt, bias, mode)
            fin = np.isfinite(val)
            # encode(decode(c)) == c for every finite code, in every rounding mode (the value is exactly representable)
            for rm in (0, 1, 2, 3, 6):
                back = np.zeros(256, np.uint8)
                orc.orc_fp32_to_fp8_n(back.ctypes.data, val.view(np.uint32).ctypes.data, 256, E, 7 - E, bias, rm, None, 0, 0, 0, 0, mode)
                assert np.array_equal(back[fin], codes[fin]), (bias, mode, rm)
            # decode is odd: code ^ 0x80 negates
            assert np.array_equal(val[:128][fin[:128]], -val[128:][fin[:128]])
            # the positive finite codes decode to a strictly increasing sequence: value = (1 + m / 2^M) 2^(e - bias)
            pos = val[:128][fin[:128]]
            assert np.all(np.diff(pos) > 0)
            M = 7 - E
            e, m = (codes[:128] & 0x7F) >> M, codes[:128] & ((1 << M) - 1)
            closed = np.where(e == 0, m / 2.0 ** M * 2.0 ** (1 - bias), (1 + m / 2.0 ** M) * 2.0 ** (e.astype(np.int32) - bias))
            assert np.array_equal(val[:128][fin[:128]].astype(np.float64), closed[fin[:128]])
            # encode is monotone non-decreasing over sorted finite inputs (RNE, saturating)
            xs = np.sort(np.random.default_rng(bias).standard_normal(20000).astype(np.float32) * np.float32(2.0 ** (8 - bias)))
            enc = np.zeros(xs.size, np.uint8)
            orc.orc_fp32_to_fp8_n(enc.ctypes.data, xs.view(np.uint32).ctypes.data, xs.size, E, 7 - E, bias, 0, None, 0, 1, 0, 0, 0)
            dec = decode_fp8(orc, enc, dt, bias, 0)
            assert np.all(np.diff(dec) >= 0)
            # round to nearest: the decoded value is never further than half a step from the input (inside the range)
            inside = np.abs(xs) <= np.max(pos[np.isfinite(pos)]) if mode == 0 else np.zeros(xs.size, bool)
            if mode == 0 and inside.any():
                allv = np.sort(np.concatenate([-pos, pos]))
                nearest = allv[np.abs(allv[None, :] - xs[inside][:2000, None]).argmin(axis=1)]
                assert np.all(np.abs(dec[inside][:2000] - xs[inside][:2000]) <= np.abs(nearest - xs[inside][:2000]) + 0)


def test_casts_agree_with_ieee_conversions_of_torch(orc):
    """fp8_152 / bias 15 / full mode is IEEE e5m2, fp8_143 / bias 7 / minimal mode is OCP e4m3fn, bf16 RNE is bf16:
    torch's CPU conversions implement those independently."""
    import torch
    rng = np.random.default_rng(17)
    x = (rng.standard_normal(200000) * np.exp2(rng.integers(-20, 18, 200000))).astype(np.float32)
    x[:4] = [0.0, -0.0, np.inf, -np.inf]
    t = torch.from_numpy(x)
    o = np.zeros(x.size, np.uint16)
    orc.orc_fp32_to_bf16_n(o.ctypes.data, x.view(np.uint32).ctypes.data, x.size, 0, None, 0, 0, 0)
    assert np.array_equal(o, t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))
    o8 = np.zeros(x.size, np.uint8)
    orc.orc_fp32_to_fp8_n(o8.ctypes.data, x.view(np.uint32).ctypes.data, x.size, 5, 2, 15, 0, None, 0, 0, 0, 0, 0)
    assert np.array_equal(o8, t.to(torch.float8_e5m2).view(torch.uint8).numpy())
    orc.orc_fp32_to_fp8_n(o8.ctypes.data, x.view(np.uint32).ctypes.data, x.size, 4, 3, 7, 0, None, 0, 0, 0, 0, 2)
    ref8 = t.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    nan = (ref8 & 0x7F) == 0x7F   # overflow -> NaN in both; the sign of that NaN is not pinned by the format
    assert np.array_equal((o8 & 0x7F) == 0x7F, nan)
    assert np.array_equal(o8[~nan], ref8[~nan])
    # and the decoders agree with torch's
    codes = torch.arange(256, dtype=torch.uint8)
    for dt, bias, mode, tdt in [(abi.FP8_152, 15, 0, torch.float8_e5m2), (abi.FP8_143, 7, 2, torch.float8_e4m3fn)]:
        mine = decode_fp8(orc, codes.numpy(), dt, bias, mode)
        theirs = codes.view(tdt).to(torch.float32).numpy()
        assert np.array_equal(np.isnan(mine), np.isnan(theirs))
        assert np.array_equal(mine[~np.isnan(mine)], theirs[~np.isnan(theirs)])


def test_saturation_never_emits_inf_or_nan_for_finite_input(orc):
    x = np.array([1000.0, -1000.0, 3.4e38, -3.4e38, 240.0, 248.0, 1e9], np.float32)
    o = np.zeros(x.size, np.uint8)
    orc.orc_fp32_to_fp8_n(o.ctypes.data, x.view(np.uint32).ctypes.data, x.size, 4, 3, 7, 0, None, 0, 1, 0, 0, 0)
    assert list(o[:4]) == [0x77, 0xF7, 0x77, 0xF7] and o[4] == 0x77 and o[6] == 0x77
    orc.orc_fp32_to_fp8_n(o.ctypes.data, x.view(np.uint32).ctypes.data, x.size, 4, 3, 7, 0, None, 0, 0, 0, 0, 0)
    assert o[0] == 0x78 and o[1] == 0xF8   # without clipping: +-inf
    orc.orc_fp32_to_fp8_n(o.ctypes.data, x.view(np.uint32).ctypes.data, x.size, 5, 2, 15, 0, None, 0, 1, 0, 0, 0)
    assert o[6] == 0x7B                    # fp8_152 bias 15: 57344
    assert orc.orc_fp32_to_bf16(int(np.float32(3.4e38).view(np.uint32)), 0, 0, 1, 0, 0) == 0x7F7F


@pytest.mark.parametrize("dt,bias", [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP8_152, 15), (abi.FP32, 0)])
def test_tree_accumulation_close_to_exact_sum(orc, dt, bias):
    """The truncating 8-wide tree stays within (K / 8 + 1) * 2^-22 * sum|a_i b_i| of the exact dot product."""
    rng = np.random.default_rng(5)
    M, N, K = 6, 7, 1000
    a = random_operand(rng, dt, M * K, orc, bias)
    b = random_operand(rng, dt, N * K, orc, bias)
    o = np.zeros(M * N, np.float32)
    da, db, do = desc(a, [K, M], dt, bias), desc(b, [N, K], dt, bias), desc(o, [N, M], abi.FP32)
    assert orc.orc_batch_gemm(A(do), A(da), A(db), abi.OP_AB) == 0
    af, bf = decode_operand(orc, a, dt, bias).reshape(M, K), decode_operand(orc, b, dt, bias).reshape(K, N)
    exact = af @ bf
    bound = (K / 8 + 2) * 2.0 ** -22 * (np.abs(af) @ np.abs(bf))
    assert np.all(np.abs(o.reshape(M, N) - exact) <= bound)
    # the tree truncates toward zero at each step, so the error is systematically not above zero in magnitude
    assert np.linalg.norm(o.reshape(M, N) - exact) / np.linalg.norm(exact) < 1e-4


def test_transposed_ops_equal_explicit_transposes(orc):
    rng = np.random.default_rng(8)
    M, N, K = 9, 5, 19
    a = to_bf16_bits(rng.standard_normal((M, K)))
    b = to_bf16_bits(rng.standard_normal((K, N)))
    res = {}
    for op, am, bm in [(abi.OP_AB, a, b), (abi.OP_ABT, a, b.T.copy()), (abi.OP_ATB, a.T.copy(), b), (abi.OP_ATBT, a.T.copy(), b.T.copy())]:
        o = np.zeros(M * N, np.float32)
        da, db, do = desc(am, [am.shape[1], am.shape[0]], abi.BF16), desc(bm, [bm.shape[1], bm.shape[0]], abi.BF16), desc(o, [N, M], abi.FP32)
        assert orc.orc_batch_gemm(A(do), A(da), A(db), op) == 0
        res[op] = o.copy()
    for op in (abi.OP_ABT, abi.OP_ATB, abi.OP_ATBT):
        assert np.array_equal(res[op].view(np.uint32), res[abi.OP_AB].view(np.uint32))


def _direct_conv(x, w, pad, st, dil):
    """7-loop fp64 convolution: x [B,D,H,W,C], w [Q,R,S,C,K] -> y [B,Do,Ho,Wo,K]."""
    B, D, H, W, C = x.shape
    Q, R, S, _, K = w.shape
    osz = lambda i, k, p, s, d: (i + 2 * p - d * (k - 1) - 1) // s + 1
    Wo, Ho, Do = osz(W, S, pad[0], st[0], dil[0]), osz(H, R, pad[1], st[1], dil[1]), osz(D, Q, pad[2], st[2], dil[2])
    y = np.zeros((B, Do, Ho, Wo, K))
    for b in range(B):
        for do in range(Do):
            for ho in range(Ho):
                for wo in range(Wo):
                    for q in range(Q):
                        for r in range(R):
                            for s in range(S):
                                d_, h_, w_ = do * st[2] + q * dil[2] - pad[2], ho * st[1] + r * dil[1] - pad[1], wo * st[0] + s * dil[0] - pad[0]
                                if 0 <= d_ < D and 0 <= h_ < H and 0 <= w_ < W:
                                    y[b, do, ho, wo] += x[b, d_, h_, w_] @ w[q, r, s]
    return y


@pytest.mark.parametrize("case", [(3, 4, 6, 5, 1, 2, 3, 3, 1, (1, 1, 0), (2, 1, 1), (1, 2, 1), 2),
                                  (2, 3, 5, 4, 3, 1, 2, 2, 2, (1, 0, 1), (1, 2, 1), (1, 1, 2), 3)])
def test_conv_against_direct_convolution_and_adjoints(orc, case):
    (C_, K_, W, H, D, B, S, R, Q, pad, st, dil, dim) = case
    rng = np.random.default_rng(12)
    x = to_bf16_bits(rng.standard_normal((B, D, H, W, C_)))
    w = to_bf16_bits(rng.standard_normal((Q, R, S, C_, K_)))
    xf, wf = bf16_bits_to_f32(x).astype(np.float64), bf16_bits_to_f32(w).astype(np.float64)
    yw = _direct_conv(xf, wf, pad, st, dil)
    ys = [K_] + list(yw.shape[-2::-1])
    xs, ws = [C_, W, H, D, B], [K_, C_, S, R, Q]
    p = abi.make_conv_params(dim, pad, st, dil)
    y = np.zeros(yw.size, np.float32)
    dx, dw, dy = desc(x, xs, abi.BF16), desc(w, ws, abi.BF16), desc(y, ys, abi.FP32)
    assert orc.orc_convolution(A(dy), A(dx), A(dw), A(dy), A(p), abi.OP_FWD, 0) == 0
    assert np.allclose(y.reshape(yw.shape), yw, rtol=1e-5, atol=1e-5)
    # adjoints: <g, fwd(x, w)> = <dedx(g, w), x> = <dedw(x, g), w>
    g = to_bf16_bits(rng.standard_normal(yw.shape))
    gf = bf16_bits_to_f32(g).astype(np.float64)
    gx, gw = np.zeros(x.size, np.float32), np.zeros(w.size, np.float32)
    dg, dgx, dgw = desc(g, ys, abi.BF16), desc(gx, xs, abi.FP32), desc(gw, ws, abi.FP32)
    assert orc.orc_convolution(A(dgx), A(dx), A(dw), A(dg), A(p), abi.OP_DEDX, 0) == 0
    assert orc.orc_convolution(A(dgw), A(dx), A(dw), A(dg), A(p), abi.OP_DEDW, 0) == 0
    s_f = np.sum(gf * yw)
    assert abs(np.sum(gx.astype(np.float64) * xf.ravel()) - s_f) <= 1e-5 * abs(s_f) + 1e-4
    assert abs(np.sum(gw.astype(np.float64) * wf.ravel()) - s_f) <= 1e-5 * abs(s_f) + 1e-4


def test_oracle_error_conventions(orc):
    a = np.zeros(8, np.uint16)
    o = np.zeros(8, np.float32)
    ob = np.zeros(8, np.uint16)
    da, db = desc(a, [4, 2], abi.BF16), desc(a, [2, 4], abi.BF16)
    d_bad_out = desc(ob, [2, 2], abi.BF16)
    assert orc.orc_batch_gemm(A(d_bad_out), A(da), A(db), abi.OP_AB) != 0      # output must be fp32
    assert b"not registered" in orc.orc_last_error()
    df = desc(o, [2, 4], abi.FP32)
    do = desc(o, [2, 2], abi.FP32)
    assert orc.orc_batch_gemm(A(do), A(da), A(df), abi.OP_AB) != 0              # mixed non-fp8 types
    d3 = desc(a, [4, 2, 2], abi.BF16)
    do3 = desc(o, [2, 2, 1], abi.FP32)
    assert orc.orc_batch_gemm(A(do3), A(d3), A(db), abi.OP_AB) != 0             # batch dims
