"""The oracle restatement against the reference's own sources compiled into oracle/_ref (bit for bit).
Skipped where that library has not been built (the reference tree is not present everywhere)."""
import itertools

import numpy as np
import pytest

from intel_gaudi3_software_amd import abi
from helpers import rmw_operands, A, cast_sweep_inputs, desc


def test_fp8_encode_sweep(orc, ref):
    x = cast_sweep_inputs()
    rng = np.random.default_rng(0)
    lf = rng.integers(0, 2 ** 32, x.size, dtype=np.uint64).astype(np.uint32)
    lf[::7] = 0
    a, b = np.zeros(x.size, np.uint8), np.zeros(x.size, np.uint8)
    for (E, M, biases) in [(4, 3, [3, 7, 15]), (5, 2, [1, 15, 30])]:
        for bias, mode, rm in itertools.product(biases, (0, 1, 2), (0, 1, 2, 3, 4, 6, 7)):
            for clip, cinf, ftz, sftz in [(0, 0, 0, 0), (1, 0, 0, 0), (1, 1, 1, 0), (0, 0, 1, 1), (1, 0, 0, 1)]:
                ref.ref_fp32_to_fp8_n(a.ctypes.data, x.ctypes.data, x.size, E, M, bias, rm, lf.ctypes.data, ftz, clip, cinf, sftz, mode)
                orc.orc_fp32_to_fp8_n(b.ctypes.data, x.ctypes.data, x.size, E, M, bias, rm, lf.ctypes.data, ftz, clip, cinf, sftz, mode)
                assert np.array_equal(a, b), (E, bias, mode, rm, clip, cinf, ftz, sftz)


def test_decode_bf16_fp32_add(orc, ref):
    codes = np.arange(256, dtype=np.uint8)
    a, b = np.zeros(256, np.uint32), np.zeros(256, np.uint32)
    for E, M, biases in [(4, 3, [3, 7, 11, 15]), (5, 2, range(1, 31))]:
        for bias, mode in itertools.product(biases, (0, 1, 2)):
            ref.ref_fp8_to_fp32_n(a.ctypes.data, codes.ctypes.data, 256, E, M, bias, mode)
            orc.orc_fp8_to_fp32_n(b.ctypes.data, codes.ctypes.data, 256, E, M, bias, mode)
            assert np.array_equal(a, b)
    x = cast_sweep_inputs()
    rng = np.random.default_rng(1)
    lf = rng.integers(0, 2 ** 32, x.size, dtype=np.uint64).astype(np.uint32)
    h1, h2 = np.zeros(x.size, np.uint16), np.zeros(x.size, np.uint16)
    w1, w2 = np.zeros(x.size, np.uint32), np.zeros(x.size, np.uint32)
    for rm, (clip, cinf), ftz in itertools.product((0, 1, 2, 3, 4, 6, 7), [(0, 0), (1, 0), (1, 1)], (0, 1)):
        ref.ref_fp32_to_bf16_n(h1.ctypes.data, x.ctypes.data, x.size, rm, lf.ctypes.data, clip, ftz, cinf)
        orc.orc_fp32_to_bf16_n(h2.ctypes.data, x.ctypes.data, x.size, rm, lf.ctypes.data, clip, ftz, cinf)
        assert np.array_equal(h1, h2), (rm, clip, cinf, ftz)
        ref.ref_fp32_to_fp32_n(w1.ctypes.data, x.ctypes.data, x.size, rm, clip, ftz, cinf)
        orc.orc_fp32_to_fp32_n(w2.ctypes.data, x.ctypes.data, x.size, rm, clip, ftz, cinf)
        assert np.array_equal(w1, w2)
    p = rng.integers(0, 2 ** 32, 1 << 18, dtype=np.uint64).astype(np.uint32)
    q = p ^ rng.integers(0, 1 << 12, p.size, dtype=np.uint64).astype(np.uint32) ^ np.uint32(0x80000000)
    q[::2] = rng.integers(0, 2 ** 32, p.size // 2, dtype=np.uint64).astype(np.uint32)
    s1, s2 = np.zeros(p.size, np.uint32), np.zeros(p.size, np.uint32)
    for rm in range(4):
        ref.ref_add_fp32_n(s1.ctypes.data, p.ctypes.data, q.ctypes.data, p.size, rm)
        orc.orc_add_fp32_n(s2.ctypes.data, p.ctypes.data, q.ctypes.data, p.size, rm)
        assert np.array_equal(s1, s2)
    assert all(ref.ref_lfsr32(v, 0x37) == orc.orc_lfsr32(v, 0x37) for v in (0, 1, 2, 3, 0xFFFFFFFF, 0x12345678))


def _rand_bits(rng, n, kind):
    if kind == "any":
        return rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32)
    if kind == "normal":
        return rng.standard_normal(n).astype(np.float32).view(np.uint32)
    if kind == "small":
        return ((rng.integers(0, 2, n).astype(np.uint32) << 31) | (rng.integers(0, 40, n).astype(np.uint32) << 23) |
                rng.integers(0, 1 << 23, n).astype(np.uint32))
    ch = np.array([0, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 1, 0x807fffff, 0x3f800000, 0x00800000, 0x7f7fffff], np.uint32)
    return ch[rng.integers(0, ch.size, n)]


def test_tree(orc, ref):
    rng = np.random.default_rng(2)
    MA = np.array([0xff8000ff, 0xff8000ff, 0xff80ff00, 0xff80ff00, 0xff80ff00, 0xffff0000, 0xffff0000, 0xffff0000], np.uint32)
    MB = np.array([0xff80ff00, 0xffff0000, 0xff8000ff, 0xff80ff00, 0xffff0000, 0xff8000ff, 0xff80ff00, 0xffff0000], np.uint32)
    m = 20000
    for emul, ka, kb, kc in itertools.product((0, 1), ("any", "normal", "small", "special"), ("any", "normal", "small", "special"),
                                              ("normal", "small", "special")):
        Aa, Bb = _rand_bits(rng, m * 9, ka).reshape(m, 9).copy(), _rand_bits(rng, m * 9, kb).reshape(m, 9).copy()
        msk = rng.random((m, 9)) < 0.03
        Aa[msk] = _rand_bits(rng, int(msk.sum()), "special")
        Aa[:, 8], Bb[:, 8] = _rand_bits(rng, m, kc), 0x3f800000
        if emul:
            Aa[:, :8], Bb[:, :8] = Aa[:, :1] & MA[None, :], Bb[:, :1] & MB[None, :]
        x, y = np.zeros(m, np.uint32), np.zeros(m, np.uint32)
        ref.ref_tree9_n(x.ctypes.data, Aa.ctypes.data, Bb.ctypes.data, m, emul)
        orc.orc_tree9_n(y.ctypes.data, Aa.ctypes.data, Bb.ctypes.data, m, emul)
        assert np.array_equal(x, y), (emul, ka, kb, kc)


def _rand_op(rng, dt, n):
    if dt == abi.BF16:
        return (rng.standard_normal(n).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    if dt == abi.FP32:
        return rng.standard_normal(n).astype(np.float32)
    return rng.integers(0, 256, n).astype(np.uint8)


def test_batch_gemm(orc, ref):
    rng = np.random.default_rng(3)
    for (dtA, dtB, bA, bB, mA, mB), op in itertools.product(
            [(abi.BF16, abi.BF16, 0, 0, 0, 0), (abi.FP32, abi.FP32, 0, 0, 0, 0), (abi.FP8_143, abi.FP8_143, 7, 7, 0, 0),
             (abi.FP8_143, abi.FP8_152, 7, 15, 0, 0), (abi.FP8_152, abi.FP8_143, 20, 3, 2, 1)],
            (abi.OP_AB, abi.OP_ABT, abi.OP_ATB, abi.OP_ATBT)):
        M, N, K = 13, 11, 37
        ta, tb = op in (abi.OP_ATB, abi.OP_ATBT), op in (abi.OP_ABT, abi.OP_ATBT)
        asz, bsz = ([M, K] if ta else [K, M]) + [2, 3, 1], ([K, N] if tb else [N, K]) + [1, 3, 1]
        a, b = _rand_op(rng, dtA, M * K * 6), _rand_op(rng, dtB, N * K * 3)
        o1, o2 = np.zeros(M * N * 6, np.float32), np.zeros(M * N * 6, np.float32)
        da, db = desc(a, asz, dtA, bA, mA), desc(b, bsz, dtB, bB, mB)
        d1, d2 = desc(o1, [N, M, 2, 3, 1], abi.FP32), desc(o2, [N, M, 2, 3, 1], abi.FP32)
        assert ref.ref_batch_gemm(A(d1), A(da), A(db), op) == 0
        assert orc.orc_batch_gemm(A(d2), A(da), A(db), op) == 0
        assert np.array_equal(o1.view(np.uint32), o2.view(np.uint32)), (dtA, dtB, op)
    # row pitches larger than the rows
    M, N, K = 9, 10, 20
    a, b = _rand_op(rng, abi.BF16, M * (K + 5)), _rand_op(rng, abi.BF16, K * (N + 3))
    o1 = np.full(M * (N + 2), 7, np.float32)
    o2 = o1.copy()
    da, db = desc(a, [K, M], abi.BF16, strides=[1, K + 5]), desc(b, [N, K], abi.BF16, strides=[1, N + 3])
    d1, d2 = desc(o1, [N, M], abi.FP32, strides=[1, N + 2]), desc(o2, [N, M], abi.FP32, strides=[1, N + 2])
    assert ref.ref_batch_gemm(A(d1), A(da), A(db), abi.OP_AB) == 0 and orc.orc_batch_gemm(A(d2), A(da), A(db), abi.OP_AB) == 0
    assert np.array_equal(o1.view(np.uint32), o2.view(np.uint32))


def test_convolution(orc, ref):
    rng = np.random.default_rng(4)
    osz = lambda i, k, p, s, d: (i + 2 * p - d * (k - 1) - 1) // s + 1
    for (dt, bias), (C_, K_, W, H, D, B, S, R, Q, pad, st, dil, dim) in itertools.product(
            [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP32, 0)],
            [(3, 4, 5, 5, 1, 2, 3, 3, 1, (1, 1, 0), (2, 2, 1), (1, 1, 1), 2), (4, 3, 7, 6, 1, 2, 3, 2, 1, (2, 0, 0), (1, 2, 1), (2, 1, 1), 2),
             (2, 3, 5, 4, 3, 1, 2, 2, 2, (1, 0, 1), (1, 1, 1), (1, 2, 1), 3), (8, 8, 6, 6, 1, 1, 1, 1, 1, (0, 0, 0), (1, 1, 1), (1, 1, 1), 2)]):
        Wo, Ho, Do = osz(W, S, pad[0], st[0], dil[0]), osz(H, R, pad[1], st[1], dil[1]), osz(D, Q, pad[2], st[2], dil[2])
        xs, ws, ys = [C_, W, H, D, B], [K_, C_, S, R, Q], [K_, Wo, Ho, Do, B]
        x, w, y = _rand_op(rng, dt, int(np.prod(xs))), _rand_op(rng, dt, int(np.prod(ws))), _rand_op(rng, dt, int(np.prod(ys)))
        if dt == abi.FP8_143:
            x &= 0x77
            w &= 0xF7
            y &= 0xF7
        p = abi.make_conv_params(dim, pad, st, dil)
        for op, os_ in [(abi.OP_FWD, ys), (abi.OP_DEDX, xs), (abi.OP_DEDW, ws)]:
            for rm in ((0, 1, 2, 3) if op == abi.OP_DEDX else (0,)):
                n = int(np.prod(os_))
                o1, o2 = np.zeros(n, np.float32), np.zeros(n, np.float32)
                dx, dw, dy = desc(x, xs, dt, bias), desc(w, ws, dt, bias), desc(y, ys, dt, bias)
                d1, d2 = desc(o1, os_, abi.FP32), desc(o2, os_, abi.FP32)
                assert ref.ref_convolution(A(d1), A(dx), A(dw), A(dy), A(p), op, rm) == 0
                assert orc.orc_convolution(A(d2), A(dx), A(dw), A(dy), A(p), op, rm) == 0
                assert np.array_equal(o1.view(np.uint32), o2.view(np.uint32)), (dt, op, rm)


def test_transposed_dedx(orc, ref):
    """transposed_dedx (weights given with their first two dimensions exchanged, S axis read in reverse,
    mme_reference_impl.cpp:625-647): restatement against the compiled reference, bit for bit."""
    rng = np.random.default_rng(14)
    osz = lambda i, k, p, s, d: (i + 2 * p - d * (k - 1) - 1) // s + 1
    for (dt, bias), (C_, K_, W, H, D, B, S, R, Q, pad, st, dil, dim) in itertools.product(
            [(abi.BF16, 0), (abi.FP8_152, 15), (abi.FP32, 0)],
            [(3, 4, 5, 5, 1, 2, 3, 3, 1, (1, 1, 0), (2, 2, 1), (1, 1, 1), 2), (4, 3, 7, 6, 1, 2, 3, 2, 1, (2, 0, 0), (1, 2, 1), (2, 1, 1), 2),
             (2, 3, 5, 4, 3, 1, 2, 2, 2, (1, 0, 1), (1, 1, 1), (1, 2, 1), 3)]):
        Wo, Ho, Do = osz(W, S, pad[0], st[0], dil[0]), osz(H, R, pad[1], st[1], dil[1]), osz(D, Q, pad[2], st[2], dil[2])
        xs, wts, ys = [C_, W, H, D, B], [C_, K_, S, R, Q], [K_, Wo, Ho, Do, B]
        w, y = _rand_op(rng, dt, int(np.prod(wts))), _rand_op(rng, dt, int(np.prod(ys)))
        if dt == abi.FP8_152:
            w &= 0xF3
            y &= 0xF3
        p = abi.make_conv_params(dim, pad, st, dil)
        n = int(np.prod(xs))
        o1, o2 = np.zeros(n, np.float32), np.zeros(n, np.float32)
        dw, dy = desc(w, wts, dt, bias), desc(y, ys, dt, bias)
        d1, d2 = desc(o1, xs, abi.FP32), desc(o2, xs, abi.FP32)
        assert ref.ref_convolution(A(d1), A(d1), A(dw), A(dy), A(p), abi.OP_TRANSPOSED_DEDX, 0) == 0
        assert orc.orc_convolution(A(d2), A(d2), A(dw), A(dy), A(p), abi.OP_TRANSPOSED_DEDX, 0) == 0
        assert np.array_equal(o1.view(np.uint32), o2.view(np.uint32)), (dt, C_, K_)
        assert np.any(o1 != 0)


def test_activation(orc, ref):
    rng = np.random.default_rng(5)
    n = 4096 * 3
    acc = (rng.standard_normal(n) * np.exp2(rng.integers(-20, 20, n))).astype(np.float32)
    acc[::97], acc[::101], acc[::103], acc[::89] = np.inf, -np.inf, np.nan, -0.0
    for (dt, bias, mode), rm, relu in itertools.product(
            [(abi.BF16, 0, 0), (abi.FP32, 0, 0), (abi.FP8_143, 7, 0), (abi.FP8_143, 3, 2), (abi.FP8_152, 15, 0), (abi.FP8_152, 24, 1)],
            (0, 1, 2, 3, 4, 6, 7), (0, 1)):
        for clip, cinf, ftz, sftz in [(0, 0, 0, 0), (1, 0, 0, 0), (1, 1, 1, 0), (0, 0, 1, 1), (1, 0, 0, 1)]:
            a1, a2 = acc.copy(), acc.copy()
            o1, o2 = np.zeros(n * abi.DTYPE_SIZE[dt], np.uint8), np.zeros(n * abi.DTYPE_SIZE[dt], np.uint8)
            l1 = ((np.arange(256, dtype=np.uint64) + 2) * 2654435761 % 2 ** 32).astype(np.uint32)
            l2 = l1.copy()
            t1, t2 = desc(o1, [64, n // 64], dt, bias, mode), desc(o2, [64, n // 64], dt, bias, mode)
            ta1, ta2 = desc(a1, [64, n // 64], abi.FP32), desc(a2, [64, n // 64], abi.FP32)
            assert ref.ref_activation(A(t1), A(ta1), relu, rm, clip, cinf, ftz, sftz, l1.ctypes.data, 0x33, 256) == 0
            assert orc.orc_activation(A(t2), A(ta2), relu, rm, clip, cinf, ftz, sftz, l2.ctypes.data, 0x33) == 0
            assert np.array_equal(o1, o2) and np.array_equal(a1.view(np.uint32), a2.view(np.uint32)), (dt, bias, mode, rm, relu)


def test_memory_write_reductions(orc):
    """doMemoryWrite with add / sub / min / max / max_0 on fp32, bf16 and fp16 tensors, every reduction rounding mode, clipping on
    and off: the restatement (one correctly rounded adder with flush-to-zero) against the compiled reference's executeOp,
    bit for bit, on 2^18 operand pairs per setting (odd element count: the reference's 4-byte loop has a 2-byte tail).
    The reference side is oracle/_ref/libmme_ref_rmw.so: fs_fma.cpp compiled at -O0, where the flush-to-zero switches
    around fmaf take effect as written (at -O3 gcc moves the fmaf across them)."""
    import oracle
    rmw = oracle.ref_rmw()
    if rmw is None:
        pytest.skip("oracle/_ref/libmme_ref_rmw.so is not built (needs the reference tree)")
    rng = np.random.default_rng(21)
    n = (1 << 18) + 1
    from helpers import rmw_operands_fp16
    type_code = {abi.FP32: rmw.ref_rmw_type_fp32(), abi.BF16: rmw.ref_rmw_type_bf16(), abi.FP16: rmw.ref_rmw_type_fp16(),
                 abi.FP8_152: rmw.ref_rmw_type_fp8()}
    all_pairs = np.arange(65536, dtype=np.uint32)
    for dt in (abi.FP32, abi.BF16, abi.FP16, abi.FP8_152):
        if dt == abi.FP8_152:  # every pair of codes (plus one element: the 4-byte loop's tail)
            a, b = np.append(all_pairs >> 8, 0x3C).astype(np.uint8), np.append(all_pairs & 0xFF, 0xBC).astype(np.uint8)
        else:
            a, b = rmw_operands_fp16(rng, n) if dt == abi.FP16 else rmw_operands(rng, dt, n)
        for op, rm, clip in itertools.product(range(5), range(4), (0, 1)):
            if op in (abi.REDUCTION_MIN, abi.REDUCTION_MAX) and (rm or clip):
                continue
            m1, m2 = a.copy(), a.copy()
            sizes = [a.size, 1, 1, 1, 1]
            d2, do = desc(m2, sizes, dt, 15 if dt in (abi.FP16, abi.FP8_152) else 0), desc(b, sizes, dt, 15 if dt in (abi.FP16, abi.FP8_152) else 0)
            rmw.ref_memory_write_words(m1.ctypes.data, b.ctypes.data, m1.nbytes, op, type_code[dt], rm, clip)
            assert orc.orc_memory_write(A(d2), A(do), op, rm, clip) == 0
            bad = np.flatnonzero(m1 != m2)
            assert bad.size == 0, (dt, op, rm, clip, hex(int(a[bad[0]])), hex(int(b[bad[0]])), hex(int(m1[bad[0]])), hex(int(m2[bad[0]])))
    # reduction none: a byte copy
    a, b = rmw_operands(rng, abi.BF16, n)
    m1 = a.copy()
    d1, do = desc(m1, [n, 1, 1, 1, 1], abi.BF16), desc(b, [n, 1, 1, 1, 1], abi.BF16)
    assert orc.orc_memory_write(A(d1), A(do), abi.REDUCTION_NONE, 0, 0) == 0
    assert np.array_equal(m1, b)


def test_fp16_ufp16_tf32_converters(orc, ref):
    """cfp16_to_fp32 over all 65536 codes, fp32_to_cfp16 over the cast sweep with every rounding mode, fp32_to_tf32."""
    codes = np.arange(65536, dtype=np.uint16)
    a, b = np.zeros(65536, np.uint32), np.zeros(65536, np.uint32)
    for E, biases in [(5, (1, 7, 15, 20, 30)), (6, (1, 15, 31, 40, 62))]:
        for bias, nin in itertools.product(biases, (0, 1)):
            ref.ref_cfp16_to_fp32_n(a.ctypes.data, codes.ctypes.data, 65536, E, bias, nin)
            orc.orc_cfp16_to_fp32_n(b.ctypes.data, codes.ctypes.data, 65536, E, bias, nin)
            assert np.array_equal(a, b), (E, bias, nin)
    x = cast_sweep_inputs()
    rng = np.random.default_rng(21)
    lf = rng.integers(0, 2 ** 32, x.size, dtype=np.uint64).astype(np.uint32)
    lf[::7] = 0
    h1, h2 = np.zeros(x.size, np.uint16), np.zeros(x.size, np.uint16)
    for E, biases in [(5, (3, 15, 28)), (6, (5, 31, 60))]:
        for bias, nin, rm in itertools.product(biases, (0, 1), (0, 1, 2, 3, 4, 6, 7)):
            for clip, cinf, ftz in [(0, 0, 0), (1, 0, 0), (1, 1, 1), (0, 0, 1)]:
                ref.ref_fp32_to_cfp16_n(h1.ctypes.data, x.ctypes.data, x.size, E, bias, rm, lf.ctypes.data, ftz, clip, cinf, nin)
                orc.orc_fp32_to_cfp16_n(h2.ctypes.data, x.ctypes.data, x.size, E, bias, rm, lf.ctypes.data, ftz, clip, cinf, nin)
                assert np.array_equal(h1, h2), (E, bias, nin, rm, clip, cinf, ftz)
    # finer low halves around the 13 dropped bits of tf32
    lows = np.array([0, 1, 0xFFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x2FFF, 0x3000, 0x3001, 0x3FFF, 0xF000, 0xFFFF], np.uint32)
    y = ((np.arange(65536, dtype=np.uint32) << 16)[:, None] | lows[None, :]).ravel().copy()
    w1, w2 = np.zeros(y.size, np.uint32), np.zeros(y.size, np.uint32)
    for clip, cinf in [(0, 0), (1, 0), (1, 1)]:
        ref.ref_fp32_to_tf32_n(w1.ctypes.data, y.ctypes.data, y.size, clip, cinf)
        orc.orc_fp32_to_tf32_n(w2.ctypes.data, y.ctypes.data, y.size, clip, cinf)
        assert np.array_equal(w1, w2), (clip, cinf)


def test_tree_half_slices(orc, ref):
    """The tree in its fp16 / tf32 emulation mode: slices of one operand pair per quad, all special values."""
    rng = np.random.default_rng(22)
    LO, HI = np.uint32(0xff9fe000), np.uint32(0xffe00000)
    m = 20000
    for ka, kb, kc in itertools.product(("any", "normal", "small", "special"), ("any", "normal", "small", "special"),
                                        ("normal", "small", "special", "any")):
        Aa, Bb = np.zeros((m, 9), np.uint32), np.zeros((m, 9), np.uint32)
        for q in (0, 4):
            av, bv = _rand_bits(rng, m, ka), _rand_bits(rng, m, kb)
            msk = rng.random(m) < 0.05
            av[msk] = _rand_bits(rng, int(msk.sum()), "special")
            Aa[:, q + 0], Aa[:, q + 1], Aa[:, q + 2], Aa[:, q + 3] = av & LO, av & LO, av & HI, av & HI
            Bb[:, q + 0], Bb[:, q + 1], Bb[:, q + 2], Bb[:, q + 3] = bv & LO, bv & HI, bv & LO, bv & HI
        Aa[:, 8], Bb[:, 8] = _rand_bits(rng, m, kc), 0x3f800000
        x, y = np.zeros(m, np.uint32), np.zeros(m, np.uint32)
        ref.ref_tree9_n(x.ctypes.data, Aa.ctypes.data, Bb.ctypes.data, m, 2)
        orc.orc_tree9_n(y.ctypes.data, Aa.ctypes.data, Bb.ctypes.data, m, 2)
        assert np.array_equal(x, y), (ka, kb, kc)


def _rand_half(rng, n, kind):
    if kind == "any":
        return rng.integers(0, 65536, n).astype(np.uint16)
    if kind == "normal":
        return rng.standard_normal(n).astype(np.float16).view(np.uint16)
    return rng.integers(0, 0x0800, n).astype(np.uint16) | (rng.integers(0, 2, n).astype(np.uint16) << 15)  # denormals, tiny


def test_fma_vec_fp16_tf32(orc, ref):
    rng = np.random.default_rng(23)
    for (dtA, dtB, bA, bB, mA, mB), kind, cd in itertools.product(
            [(abi.FP16, abi.FP16, 15, 15, 0, 0), (abi.FP16, abi.UFP16, 15, 31, 0, 0), (abi.UFP16, abi.FP16, 20, 9, 1, 1),
             (abi.UFP16, abi.UFP16, 31, 31, 0, 1), (abi.FP16, abi.FP16, 3, 27, 1, 0)],
            ("any", "normal", "tiny"), (1, 2, 7, 64, 129)):
        for _ in range(40):
            a, b = _rand_half(rng, cd, kind), _rand_half(rng, cd, kind)
            r = ref.ref_fma_vec(a.ctypes.data, b.ctypes.data, cd, dtA, dtB, bA, bB, mA, mB)
            o = orc.orc_fma_vec_fp16(a.ctypes.data, 1, 6 if dtA == abi.UFP16 else 5, bA, int(mA != 0), b.ctypes.data, 1,
                                     6 if dtB == abi.UFP16 else 5, bB, int(mB != 0), cd)
            assert r == o, (dtA, dtB, bA, bB, mA, mB, kind, cd)
    for (clip, cinf), kind, cd in itertools.product([(0, 0), (1, 0), (1, 1)], ("any", "normal", "small", "special"), (1, 2, 9, 64, 131)):
        for _ in range(40):
            a, b = _rand_bits(rng, cd, kind), _rand_bits(rng, cd, kind)
            r = ref.ref_fma_vec_clip(a.ctypes.data, b.ctypes.data, cd, abi.TF32, abi.TF32, 0, 0, 0, 0, clip, cinf)
            o = orc.orc_fma_vec_tf32(a.ctypes.data, 1, b.ctypes.data, 1, cd, clip, cinf)
            assert r == o, (clip, cinf, kind, cd)


def test_batch_gemm_and_conv_fp16_tf32(orc, ref):
    rng = np.random.default_rng(24)
    for (dtA, dtB, bA, bB, mA, mB), op in itertools.product(
            [(abi.FP16, abi.FP16, 15, 15, 0, 0), (abi.FP16, abi.UFP16, 15, 31, 0, 0), (abi.UFP16, abi.UFP16, 29, 33, 1, 0),
             (abi.TF32, abi.TF32, 0, 0, 0, 0)],
            (abi.OP_AB, abi.OP_ABT, abi.OP_ATB, abi.OP_ATBT)):
        M, N, K = 13, 11, 37
        ta, tb = op in (abi.OP_ATB, abi.OP_ATBT), op in (abi.OP_ABT, abi.OP_ATBT)
        asz, bsz = ([M, K] if ta else [K, M]) + [2, 3, 1], ([K, N] if tb else [N, K]) + [1, 3, 1]
        gen = lambda dt, n: (rng.standard_normal(n).astype(np.float32).view(np.uint32) if dt == abi.TF32 else
                             rng.standard_normal(n).astype(np.float16).view(np.uint16) if dt == abi.FP16 else
                             rng.integers(0x7000, 0x8800, n).astype(np.uint16))
        a, b = gen(dtA, M * K * 6), gen(dtB, N * K * 3)
        o1, o2 = np.zeros(M * N * 6, np.float32), np.zeros(M * N * 6, np.float32)
        da, db = desc(a, asz, dtA, bA, mA), desc(b, bsz, dtB, bB, mB)
        d1, d2 = desc(o1, [N, M, 2, 3, 1], abi.FP32), desc(o2, [N, M, 2, 3, 1], abi.FP32)
        clip = int(dtA == abi.TF32)
        assert ref.ref_batch_gemm_clip(A(d1), A(da), A(db), op, clip, 0) == 0
        assert orc.orc_batch_gemm_clip(A(d2), A(da), A(db), op, clip, 0) == 0
        assert np.array_equal(o1.view(np.uint32), o2.view(np.uint32)), (dtA, dtB, op)
        assert np.any(o1 != 0)
    # one convolution of each operation with fp16 / ufp16 operands
    osz = lambda i, k, pd: i + 2 * pd - (k - 1)
    C_, K_, W, H, B, S, R = 5, 6, 6, 7, 2, 2, 3
    xs, ws, ys = [C_, W, H, 1, B], [K_, C_, S, R, 1], [K_, osz(W, S, 1), osz(H, R, 1), 1, B]
    p = abi.make_conv_params(2, (1, 1, 0), (1, 1, 1), (1, 1, 1))
    hgen = lambda n: rng.standard_normal(n).astype(np.float16).view(np.uint16)
    ugen = lambda n: rng.integers(0x7000, 0x8800, n).astype(np.uint16)
    for (dtx, bx, gx), (dtw, bw, gw) in [((abi.FP16, 15, hgen), (abi.FP16, 15, hgen)), ((abi.UFP16, 31, ugen), (abi.FP16, 12, hgen))]:
        x, w, y = gx(int(np.prod(xs))), gw(int(np.prod(ws))), gx(int(np.prod(ys)))
        for op, os_ in [(abi.OP_FWD, ys), (abi.OP_DEDX, xs), (abi.OP_DEDW, ws)]:
            n = int(np.prod(os_))
            o1, o2 = np.zeros(n, np.float32), np.zeros(n, np.float32)
            dx, dw, dy = desc(x, xs, dtx, bx), desc(w, ws, dtw, bw), desc(y, ys, dtx, bx)
            d1, d2 = desc(o1, os_, abi.FP32), desc(o2, os_, abi.FP32)
            assert ref.ref_convolution(A(d1), A(dx), A(dw), A(dy), A(p), op, 0) == 0, ref.ref_last_error()
            assert orc.orc_convolution(A(d2), A(dx), A(dw), A(dy), A(p), op, 0) == 0, orc.orc_last_error()
            assert np.array_equal(o1.view(np.uint32), o2.view(np.uint32)), (dtx, dtw, op)
            assert np.any(o1 != 0)


def test_activation_fp16(orc, ref):
    rng = np.random.default_rng(25)
    n = 5000
    src = (rng.standard_normal(n) * np.exp2(rng.integers(-30, 20, n))).astype(np.float32)
    src[::97] = np.inf
    src[5::89] = np.nan
    for dt, bias, mode, rm, clip, cinf, ftz in [(abi.FP16, 15, 0, 0, 0, 0, 0), (abi.FP16, 15, 0, 4, 1, 0, 1), (abi.FP16, 10, 1, 7, 0, 0, 0),
                                                 (abi.UFP16, 31, 0, 0, 1, 1, 0), (abi.UFP16, 31, 0, 4, 0, 0, 1), (abi.UFP16, 20, 1, 7, 1, 0, 0),
                                                 (abi.FP16, 15, 0, 2, 0, 0, 1), (abi.UFP16, 31, 0, 3, 0, 0, 1)]:
        o1, o2 = np.zeros(n, np.uint16), np.zeros(n, np.uint16)
        s1, s2 = src.copy(), src.copy()
        l1 = rng.integers(0, 2 ** 32, 256, dtype=np.uint64).astype(np.uint32)
        l2 = l1.copy()
        d1, d2 = desc(o1, [n], dt, bias, mode), desc(o2, [n], dt, bias, mode)
        a1, a2 = desc(s1, [n], abi.FP32), desc(s2, [n], abi.FP32)
        assert ref.ref_activation(A(d1), A(a1), 1, rm, clip, cinf, ftz, 0, l1.ctypes.data, 0x80200003, 256) == 0
        assert orc.orc_activation(A(d2), A(a2), 1, rm, clip, cinf, ftz, 0, l2.ctypes.data, 0x80200003) == 0
        assert np.array_equal(o1, o2), (dt, bias, mode, rm)


def test_activation_converts_the_whole_span_of_strided_tensors(orc, ref):
    """doActivation walks getSizeInElements() flat elements, which for a strided tensor is its span in memory: the gaps
    between rows are converted as well.  relu on a tensor with gaps is an error on both sides."""
    rng = np.random.default_rng(26)
    sizes, strides = [5, 4, 3, 1, 1], [1, 7, 30, 90, 90]
    acc = rng.standard_normal(90).astype(np.float32)
    for dt, bias in ((abi.BF16, 0), (abi.FP8_143, 7), (abi.FP16, 15), (abi.FP32, 0)):
        for relu, rm in ((0, 0), (0, 4), (1, 0)):
            o1 = np.full(90, 0x11, abi.DTYPE_NUMPY[dt]).view(abi.DTYPE_NUMPY[dt])
            o2 = o1.copy()
            a1, a2 = acc.copy(), acc.copy()
            l1 = (np.arange(256, dtype=np.uint32) * 2654435761 + 7).astype(np.uint32)
            l2 = l1.copy()
            d1, d2 = desc(o1, sizes, dt, bias, 0, strides), desc(o2, sizes, dt, bias, 0, strides)
            e1, e2 = desc(a1, sizes, abi.FP32, 0, 0, strides), desc(a2, sizes, abi.FP32, 0, 0, strides)
            r1 = ref.ref_activation(A(d1), A(e1), relu, rm, 1, 0, 0, 0, l1.ctypes.data, 0x33, 256)
            r2 = orc.orc_activation(A(d2), A(e2), relu, rm, 1, 0, 0, 0, l2.ctypes.data, 0x33)
            assert (r1 == 0) == (r2 == 0) == (relu == 0)
            if relu:
                assert b"should be flattened" in ref.ref_last_error() and b"should be flattened" in orc.orc_last_error()
            assert np.array_equal(o1.view(np.uint8), o2.view(np.uint8)) and np.array_equal(a1.view(np.uint32), a2.view(np.uint32)), (dt, relu, rm)
