"""fp16 / unsigned fp16 / tf32 on the GPU against the oracle: the converters bit for bit, the contractions within the
relative Frobenius bound of the 16-bit operand types (2e-3; exact where the arithmetic is exact)."""
import itertools

import numpy as np
import pytest

from intel_gaudi3_software_amd import ConvolutionParams, Epilogue, HipCalculator, MmeSimTensor, abi
from helpers import A, TOL, cast_sweep_inputs, desc, rel_frobenius

pytestmark = pytest.mark.gpu

OPS = [abi.OP_AB, abi.OP_ABT, abi.OP_ATB, abi.OP_ATBT]
# (type A, type B, bias A, bias B, inf/NaN mode A, mode B)
PAIRS = [(abi.FP16, abi.FP16, 15, 15, 0, 0),      # IEEE half on both sides: the fp16 matrix instruction
         (abi.FP16, abi.FP16, 9, 22, 0, 0),       # the same with the exponent biases folded into a power of two
         (abi.FP16, abi.FP16, 15, 15, 1, 0),      # exponent-all-ones codes are finite on one side: decoded operands
         (abi.FP16, abi.UFP16, 15, 31, 0, 0), (abi.UFP16, abi.FP16, 31, 12, 0, 1), (abi.UFP16, abi.UFP16, 31, 31, 0, 0),
         (abi.TF32, abi.TF32, 0, 0, 0, 0)]


def _torch_of(arr):
    import torch
    view = {2: np.int16, 4: np.int32, 1: np.uint8}[arr.dtype.itemsize]
    t = torch.from_numpy(arr.view(view).copy()).cuda()
    torch.cuda.synchronize()
    return t


def _zeros(n, dtype):
    """Device zeros, complete before returning: the library works on its own stream, torch fills on another."""
    import torch
    t = torch.zeros(n, dtype=dtype, device="cuda")
    torch.cuda.synchronize()
    return t


def _operand(rng, orc, dt, bias, mode, n, scale=1.0):
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    if dt == abi.TF32:
        return x.view(np.uint32).copy()  # fp32 words with all 23 mantissa bits: the contraction rounds them on entry
    if dt == abi.UFP16:
        x = np.abs(x)
    out = np.zeros(n, np.uint16)
    assert orc.orc_cast_from_fp32(out.ctypes.data, dt, bias, mode, x.ctypes.data, n, 0, None, 0, 0, 0, 1, 0, 0) == 0
    return out


def _shapes(op, M, N, K):
    ta, tb = op in (abi.OP_ATB, abi.OP_ATBT), op in (abi.OP_ABT, abi.OP_ATBT)
    return ([M, K] if ta else [K, M]), ([K, N] if tb else [N, K])


def _gemm_both(calc, orc, op, M, N, K, pair, a, b, batch=(1, 1, 1), clip=(0, 0), device=True):
    import torch
    dtA, dtB, bA, bB, mA, mB = pair
    asz, bsz = _shapes(op, M, N, K)
    nb = int(np.prod(batch))
    want = np.zeros(M * N * nb, np.float32)
    da, db = desc(a, asz + list(batch), dtA, bA, mA), desc(b, bsz + [1, 1, 1], dtB, bB, mB)
    do = desc(want, [N, M] + list(batch), abi.FP32)
    assert orc.orc_batch_gemm_clip(A(do), A(da), A(db), op, clip[0], clip[1]) == 0, orc.orc_last_error()
    if device:
        to = _zeros(want.size, torch.float32)
        calc.doBatchGemm(MmeSimTensor([N, M] + list(batch), 5, abi.FP32, to), MmeSimTensor(asz + list(batch), 5, dtA, _torch_of(a), bA, mA),
                         MmeSimTensor(bsz + [1, 1, 1], 5, dtB, _torch_of(b), bB, mB), op, 0, bool(clip[0]), bool(clip[1]))
        calc.synchronize()
        got = to.cpu().numpy()
    else:
        got = np.zeros(want.size, np.float32)
        calc.doBatchGemm(MmeSimTensor([N, M] + list(batch), 5, abi.FP32, got), MmeSimTensor(asz + list(batch), 5, dtA, a.copy(), bA, mA),
                         MmeSimTensor(bsz + [1, 1, 1], 5, dtB, b.copy(), bB, mB), op, 0, bool(clip[0]), bool(clip[1]))
    return got, want


@pytest.mark.parametrize("pair", PAIRS)
@pytest.mark.parametrize("op", OPS)
def test_gemm_ragged_and_aligned(calc, orc, op, pair):
    rng = np.random.default_rng(100 + op)
    for (M, N, K, batch, device) in [(13, 11, 37, (2, 3, 1), False), (160, 144, 208, (1, 1, 1), True)]:
        nb = int(np.prod(batch))
        a = _operand(rng, orc, pair[0], pair[2], pair[4], M * K * nb)
        b = _operand(rng, orc, pair[1], pair[3], pair[5], N * K)
        got, want = _gemm_both(calc, orc, op, M, N, K, pair, a, b, batch, device=device)
        assert np.any(want != 0)
        assert rel_frobenius(got, want) <= TOL[pair[0]], (M, N, K)


@pytest.mark.parametrize("pair", PAIRS[:6])
def test_gemm_exact_on_small_integers(calc, orc, pair):
    """Operands that are small integers (times the power of two the bias implies): every product and partial sum is exact
    in both the truncating tree and the IEEE accumulation, so the results agree bit for bit."""
    dtA, dtB, bA, bB, mA, mB = pair
    rng = np.random.default_rng(7)
    M, N, K = 96, 80, 192
    enc = lambda dt, bias, mode, v: _quant(orc, dt, bias, mode, v)
    ia = rng.integers(0 if dtA == abi.UFP16 else -8, 9, M * K).astype(np.float32) * np.float32(2.0 ** (15 - bA if dtA == abi.FP16 else 31 - bA))
    ib = rng.integers(0 if dtB == abi.UFP16 else -8, 9, N * K).astype(np.float32) * np.float32(2.0 ** (15 - bB if dtB == abi.FP16 else 31 - bB))
    a, b = enc(dtA, bA, mA, ia), enc(dtB, bB, mB, ib)
    got, want = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, pair, a, b)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.any(want != 0)


def _quant(orc, dt, bias, mode, values):
    out = np.zeros(values.size, np.uint16)
    assert orc.orc_cast_from_fp32(out.ctypes.data, dt, bias, mode, np.ascontiguousarray(values, np.float32).ctypes.data, values.size, 0, None, 0,
                                  0, 0, 0, 0, 0) == 0
    return out


def test_fp16_denormal_operands_are_not_flushed(calc, orc):
    """Both operands hold fp16 denormals only: the matrix instruction must multiply them as numbers (the reference does), not
    flush them to zero."""
    rng = np.random.default_rng(8)
    M, N, K = 64, 64, 256
    a = (rng.integers(1, 0x400, M * K) | (rng.integers(0, 2, M * K) << 15)).astype(np.uint16)
    b = (rng.integers(1, 0x400, N * K) | (rng.integers(0, 2, N * K) << 15)).astype(np.uint16)
    got, want = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, PAIRS[0], a, b)
    assert np.all(np.abs(want) > 0) or np.count_nonzero(want) > want.size * 0.99
    assert rel_frobenius(got, want) <= TOL[abi.FP16]


@pytest.mark.parametrize("pair", [PAIRS[0], PAIRS[2], PAIRS[3]])
def test_special_codes_propagate(calc, orc, pair):
    """inf, NaN (where the mode has them) and the largest codes in the operands: NaN and infinity land where the reference
    puts them; in the no-inf-NaN mode the exponent-all-ones codes count as numbers."""
    dtA, dtB, bA, bB, mA, mB = pair
    rng = np.random.default_rng(9)
    M, N, K = 48, 40, 64
    a = _operand(rng, orc, dtA, bA, mA, M * K)
    b = _operand(rng, orc, dtB, bB, mB, N * K)
    a.reshape(M, K)[3, 5] = 0x7C00   # +inf, or 2^16 in the no-inf-NaN mode
    a.reshape(M, K)[7, 9] = 0x7E01   # NaN, or a number
    a.reshape(M, K)[11, 0] = 0xFC00 if dtA == abi.FP16 else 0xFFFF
    b.reshape(N, K)[2, 5] = 0x7BFF if dtB == abi.FP16 else 0xFBFF  # largest finite code
    got, want = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, pair, a, b)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf])
    fin = np.isfinite(want)
    assert np.array_equal(fin, np.isfinite(got))
    assert rel_frobenius(got[fin], want[fin]) <= TOL[dtA]


@pytest.mark.parametrize("clip", [(0, 0), (1, 0), (1, 1)])
def test_tf32_operands_round_and_clip_on_entry(calc, orc, clip):
    """tf32 operands are fp32 words: values next to the largest fp32 round up to infinity unless clipping is on, infinite
    inputs stay infinite unless clip-inf-in is on too."""
    rng = np.random.default_rng(10)
    M, N, K = 32, 48, 40
    a = rng.standard_normal(M * K).astype(np.float32)
    b = rng.standard_normal(N * K).astype(np.float32)
    a.reshape(M, K)[1, :] = 0
    a.reshape(M, K)[1, 3] = np.float32(3.4028234e38)   # rounds to infinity in tf32
    b.reshape(N, K)[:, 3] = np.float32(2.0 ** -120)
    a.reshape(M, K)[2, :] = 0
    a.reshape(M, K)[2, 4] = np.inf
    b.reshape(N, K)[:, 4] = np.float32(2.0 ** -100)
    got, want = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, PAIRS[6], a.view(np.uint32), b.view(np.uint32), clip=clip)
    assert np.array_equal(np.isinf(got), np.isinf(want))
    assert np.isinf(want.reshape(M, N)[1, 0]) == (clip[0] == 0)
    assert np.isinf(want.reshape(M, N)[2, 0]) == (clip != (1, 1))
    fin = np.isfinite(want)
    assert rel_frobenius(got[fin], want[fin]) <= TOL[abi.TF32]


@pytest.mark.parametrize("types", [(abi.FP16, 15, abi.FP16, 15), (abi.UFP16, 31, abi.FP16, 12), (abi.TF32, 0, abi.TF32, 0)])
def test_convolution_three_operations(calc, orc, types):
    import torch
    dtx, bx, dtw, bw = types
    rng = np.random.default_rng(11)
    C, K_, W, H, B, S, R = 24, 40, 9, 7, 3, 3, 3
    xs, ws, ys = [C, W, H, 1, B], [K_, C, S, R, 1], [K_, W, H, 1, B]
    params = ConvolutionParams(2, [1, 1, 0, 0], [1, 1, 1, 1], [1, 1, 1, 1])
    x = _operand(rng, orc, dtx, bx, 0, int(np.prod(xs)))
    w = _operand(rng, orc, dtw, bw, 0, int(np.prod(ws)), 0.2)
    y = _operand(rng, orc, dtx, bx, 0, int(np.prod(ys)))
    pod = params.pod()
    for op, osz in [(abi.OP_FWD, ys), (abi.OP_DEDX, xs), (abi.OP_DEDW, ws)]:
        # operand B of dedw is dy, which carries the first operand's type in this set-up
        dty, by = (dtx, bx)
        if op == abi.OP_DEDW and dtw != dtx and not (dtx in (abi.FP16, abi.UFP16) and dtw in (abi.FP16, abi.UFP16)):
            continue
        n = int(np.prod(osz))
        want = np.zeros(n, np.float32)
        dx, dw, dy = desc(x, xs, dtx, bx), desc(w, ws, dtw, bw), desc(y, ys, dty, by)
        do = desc(want, osz, abi.FP32)
        args = {abi.OP_FWD: (A(do), A(dx), A(dw), A(do)), abi.OP_DEDX: (A(do), A(do), A(dw), A(dy)), abi.OP_DEDW: (A(do), A(dx), A(do), A(dy))}[op]
        assert orc.orc_convolution(*args, A(pod), op, 0) == 0, orc.orc_last_error()
        to = _zeros(n, torch.float32)
        tx, tw, ty = MmeSimTensor(xs, 5, dtx, _torch_of(x), bx), MmeSimTensor(ws, 5, dtw, _torch_of(w), bw), MmeSimTensor(ys, 5, dty, _torch_of(y), by)
        out_t = MmeSimTensor(osz, 5, abi.FP32, to)
        targs = {abi.OP_FWD: (out_t, tx, tw, out_t), abi.OP_DEDX: (out_t, out_t, tw, ty), abi.OP_DEDW: (out_t, tx, out_t, ty)}[op]
        calc.doConvolution(*targs, params, op)
        calc.synchronize()
        got = to.cpu().numpy()
        assert np.any(want != 0)
        assert rel_frobenius(got, want) <= TOL[dtx], op


@pytest.mark.parametrize("dt,E,biases", [(abi.FP16, 5, (15, 3, 28)), (abi.UFP16, 6, (31, 5, 60))])
def test_decode_every_code(calc, orc, dt, E, biases):
    import torch
    codes = np.arange(65536, dtype=np.uint16)
    src = _torch_of(codes)
    for bias, mode in itertools.product(biases, (0, 1)):
        want = np.zeros(65536, np.uint32)
        orc.orc_cfp16_to_fp32_n(want.ctypes.data, codes.ctypes.data, 65536, E, bias, int(mode != 0))
        out = _zeros(65536, torch.float32)
        calc.castToFp32(out, src, dt, 65536, fpBias=bias, infNanMode=mode)
        calc.synchronize()
        assert np.array_equal(out.cpu().numpy().view(np.uint32), want), (bias, mode)


@pytest.mark.parametrize("dt,E,biases", [(abi.FP16, 5, (15, 3, 28)), (abi.UFP16, 6, (31, 5, 60))])
def test_encode_sweep_every_deterministic_mode(calc, orc, dt, E, biases):
    """fp32 -> fp16 / ufp16 over every high half of an fp32 crossed with low halves that hit ties, sticky bits and carries."""
    import torch
    x = cast_sweep_inputs()
    src = _torch_of(x).view(torch.float32)
    want = np.zeros(x.size, np.uint16)
    for bias, mode, rm in itertools.product(biases, (0, 1), (0, 1, 2, 3, 6)):
        for clip, cinf, ftz in [(0, 0, 0), (1, 0, 0), (1, 1, 1), (0, 0, 1)]:
            orc.orc_fp32_to_cfp16_n(want.ctypes.data, x.ctypes.data, x.size, E, bias, rm, None, ftz, clip, cinf, int(mode != 0))
            out = _zeros(x.size, torch.int16)
            calc.castFromFp32(out, dt, src, x.size, fpBias=bias, infNanMode=mode, rm=rm, clipFp=bool(clip), clipInfIn=bool(cinf),
                              flushDenorms=bool(ftz))
            calc.synchronize()
            got = out.cpu().numpy().view(np.uint16)
            bad = np.flatnonzero(got != want)
            assert bad.size == 0, (bias, mode, rm, clip, cinf, ftz, hex(int(x[bad[0]])), hex(int(got[bad[0]])), hex(int(want[bad[0]])))


@pytest.mark.parametrize("dt,bias,mode", [(abi.FP16, 15, 0), (abi.FP16, 9, 1), (abi.UFP16, 31, 0), (abi.UFP16, 20, 1)])
@pytest.mark.parametrize("rm,sftz,ftz", [(4, 0, 0), (7, 0, 0), (4, 1, 1), (0, 1, 1), (7, 0, 1)])
def test_activation_stochastic_modes(orc, dt, bias, mode, rm, sftz, ftz):
    """Stochastic modes draw from LFSR register i % 64 for the 16-bit types; two calls in a row against the oracle with the
    same registers and polynomial, bit for bit (the second call pins the state the first leaves behind)."""
    import torch
    rng = np.random.default_rng(78)
    lfsr0 = rng.integers(1, 2**32, 256, dtype=np.uint64).astype(np.uint32)
    poly = 0xB400
    calc = HipCalculator(lfsrNumRegs=256, lfsr=lfsr0, polynomial=poly)
    lfsr_ref = lfsr0.copy()
    E = 5 if dt == abi.FP16 else 6
    for n in [64 * 500 + 33, 4001]:
        with np.errstate(over="ignore"):
            x = (rng.standard_normal(n) * np.exp2(rng.integers(1 - bias - 14, (1 << E) - bias + 1, n))).astype(np.float32)
        x[::97] = 0.0
        x[5::211] = np.inf
        x[7::223] = np.nan
        sizes = [n, 1, 1, 1, 1]
        want = np.zeros(n, np.uint16)
        a_ref = x.copy()
        assert orc.orc_activation(A(desc(want, sizes, dt, bias, mode)), A(desc(a_ref, sizes, abi.FP32)), 0, rm, 1, 0, ftz, sftz,
                                  lfsr_ref.ctypes.data, poly) == 0
        o_d = _zeros(n, torch.int16)
        calc.doActivation(MmeSimTensor(sizes, 5, dt, o_d, bias, mode), MmeSimTensor(sizes, 5, abi.FP32, _torch_of(x).view(torch.float32)),
                          relu=False, rm=rm, clipFp=True, flushDenorms=bool(ftz), stochasticFTZfp8=bool(sftz))
        calc.synchronize()
        got = o_d.cpu().numpy().view(np.uint16)
        assert np.array_equal(got, want), (n, int(np.flatnonzero(got != want)[0]))
    calc.close()


@pytest.mark.parametrize("out_dt,out_bias,out_mode", [(abi.FP16, 15, 0), (abi.UFP16, 31, 0), (abi.FP16, 11, 1)])
@pytest.mark.parametrize("in_pair", [PAIRS[0], PAIRS[3]])
def test_fused_epilogue_to_half_outputs(calc, orc, in_pair, out_dt, out_bias, out_mode):
    """GEMM with the fused descale + relu + cast to fp16 / ufp16 against the oracle's contraction followed by its cast: the
    accumulators differ in their last bits, so a few codes may land on the neighbour; the decoded values agree closely."""
    import torch
    rng = np.random.default_rng(12)
    M, N, K = 128, 96, 160
    a = _operand(rng, orc, in_pair[0], in_pair[2], in_pair[4], M * K)
    b = _operand(rng, orc, in_pair[1], in_pair[3], in_pair[5], N * K)
    _, acc = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, in_pair, a, b)
    want = np.zeros(M * N, np.uint16)
    assert orc.orc_cast_from_fp32(want.ctypes.data, out_dt, out_bias, out_mode, acc.ctypes.data, acc.size, -2, None, 0, 1, 0, 1, 0, 0) == 0
    to = _zeros(M * N, torch.int16)
    epi = Epilogue(scale_exp=-2, relu=True, clipFp=True)
    calc.doBatchGemm(MmeSimTensor([N, M, 1, 1, 1], 5, out_dt, to, out_bias, out_mode),
                     MmeSimTensor([K, M, 1, 1, 1], 5, in_pair[0], _torch_of(a), in_pair[2], in_pair[4]),
                     MmeSimTensor([K, N, 1, 1, 1], 5, in_pair[1], _torch_of(b), in_pair[3], in_pair[5]), abi.OP_ABT, epilogue=epi)
    calc.synchronize()
    got = to.cpu().numpy().view(np.uint16)
    assert np.mean(got == want) >= 0.97
    E = 5 if out_dt == abi.FP16 else 6
    dg, dw = np.zeros(M * N, np.uint32), np.zeros(M * N, np.uint32)
    orc.orc_cfp16_to_fp32_n(dg.ctypes.data, got.ctypes.data, got.size, E, out_bias, int(out_mode != 0))
    orc.orc_cfp16_to_fp32_n(dw.ctypes.data, want.ctypes.data, want.size, E, out_bias, int(out_mode != 0))
    assert rel_frobenius(dg.view(np.float32), dw.view(np.float32)) <= 1e-3
    assert np.count_nonzero(want) > want.size // 4


def test_tf32_rounding_is_applied_before_the_products(calc, orc):
    """Operands that turn into small integers only after the rounding to 10 mantissa bits (k + 2^-12 rounds down; 4 + 2^-9 lies
    half-way between two tf32 values and goes to the even one, 4): with the rounding every product and sum is exact and the
    result matches the oracle bit for bit; without it the fractions would show up in the sums."""
    rng = np.random.default_rng(13)
    M, N, K = 32, 32, 64
    k = rng.integers(1, 9, M * K).astype(np.float32)
    a = (k + np.float32(2.0 ** -12)).astype(np.float32)
    half = (np.float32(4.0) + np.float32(2.0 ** -9)).astype(np.float32)  # exactly between two tf32 values around 4: goes to 4.0
    a[::17] = half
    b = rng.integers(-8, 9, N * K).astype(np.float32)
    got, want = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, PAIRS[6], a.view(np.uint32), b.view(np.uint32))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.all(want == np.round(want)) and np.any(want != 0)


@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("pair", PAIRS[:2])
def test_fp16_large_tile_kernel(calc, orc, op, pair):
    """fp16 shapes that take the large-tile kernel (M, N multiples of 256, K a multiple of 64 and at least 192), all four
    layouts, a batch of two with B broadcast; and a long reduction over few tiles, which is split over k."""
    rng = np.random.default_rng(200 + op)
    for (M, N, K, batch) in [(256, 512, 320, (2, 1, 1)), (256, 256, 4096, (1, 1, 1))]:
        nb = int(np.prod(batch))
        a = _operand(rng, orc, pair[0], pair[2], pair[4], M * K * nb)
        b = _operand(rng, orc, pair[1], pair[3], pair[5], N * K)
        got, want = _gemm_both(calc, orc, op, M, N, K, pair, a, b, batch)
        assert rel_frobenius(got, want) <= 1e-4, (M, N, K)


def test_fp16_large_tile_every_k_position(calc, orc):
    """One-hot fp16 operands walk a single product through every k position and tile coordinate of the large-tile kernel."""
    M, N, K = 256, 256, 384
    a = np.zeros((M, K), np.float32)
    b = np.zeros((K, N), np.float32)
    rng = np.random.default_rng(5)
    perm_m = rng.permutation(M)
    for k in range(K):
        a[perm_m[k % M], k] = 1.0 + (k % 5)
        b[k, (k * 11 + 2) % N] = 2.0 if k % 2 else 1.0
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    for b_kc in (False, True):
        bmat = b.T.copy() if b_kc else b
        ha, hb = a.astype(np.float16).view(np.uint16).ravel(), bmat.astype(np.float16).view(np.uint16).ravel()
        got, ref = _gemm_both(calc, orc, abi.OP_ABT if b_kc else abi.OP_AB, M, N, K, PAIRS[0], ha, hb)
        assert np.array_equal(got.reshape(M, N), want) and np.array_equal(ref.reshape(M, N), want)


# ---- the two-part bf16 path: plain GEMMs of at least 2^26 multiply-adds whose operands are not both IEEE half ------------
TWO_PART_PAIRS = PAIRS[2:]


@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("pair", TWO_PART_PAIRS)
def test_two_part_path_vs_oracle(calc, orc, op, pair):
    """Operands written as hi + lo bf16 parts and contracted over 4 K by the bf16 kernels: a shape for the large-tile kernel
    and a ragged, batched one (B broadcast) for the general kernel, all four layouts."""
    rng = np.random.default_rng(300 + op)
    for (M, N, K, batch) in [(256, 256, 1024, (1, 1, 1)), (200, 136, 1237, (2, 1, 1))]:
        nb = int(np.prod(batch))
        a = _operand(rng, orc, pair[0], pair[2], pair[4], M * K * nb)
        b = _operand(rng, orc, pair[1], pair[3], pair[5], N * K)
        got, want = _gemm_both(calc, orc, op, M, N, K, pair, a, b, batch)
        assert rel_frobenius(got, want) <= 1e-4, (M, N, K)


@pytest.mark.parametrize("pair", [PAIRS[5], PAIRS[6]])
def test_two_part_path_every_k_position(calc, orc, pair):
    """One-hot operands whose values need all 11 significant bits (so both parts are non-zero) walk a single product through
    every k position of the concatenated reduction; the products are exact."""
    M, N, K = 256, 256, 1024
    a = np.zeros((M, K), np.float32)
    b = np.zeros((K, N), np.float32)
    perm_m = np.random.default_rng(6).permutation(M)
    for k in range(K):
        a[perm_m[k % M], k] = 1025.0 + (k % 1000)          # 11 significant bits
        b[k, (k * 11 + 2 + 64 * (k // M)) % N] = 1027.0 if k % 2 else 1.0
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32)
    assert np.array_equal(want.astype(np.float64), a.astype(np.float64) @ b.astype(np.float64))  # exactly representable
    for b_kc in (False, True):
        bmat = b.T.copy() if b_kc else b
        if pair[0] == abi.TF32:
            ha, hb = a.view(np.uint32).ravel().copy(), bmat.view(np.uint32).ravel().copy()
        else:
            ha, hb = _quant(orc, pair[0], pair[2], pair[4], a.ravel()), _quant(orc, pair[1], pair[3], pair[5], bmat.ravel())
        got, ref = _gemm_both(calc, orc, abi.OP_ABT if b_kc else abi.OP_AB, M, N, K, pair, ha, hb)
        assert np.array_equal(got.reshape(M, N), want) and np.array_equal(ref.reshape(M, N), want)


@pytest.mark.parametrize("pair", [PAIRS[3], PAIRS[6]])
def test_two_part_path_steps_aside_for_inf_and_nan(calc, orc, pair):
    """inf * 0 would appear among the partial products of split operands: a call whose operands hold inf or NaN is contracted
    from fp32 copies instead (decided on the device), and the next call without them takes the two-part path again."""
    dtA, dtB, bA, bB, mA, mB = pair
    rng = np.random.default_rng(10)
    M, N, K = 256, 256, 1024
    a = _operand(rng, orc, dtA, bA, mA, M * K)
    b = _operand(rng, orc, dtB, bB, mB, N * K)
    clean, want_clean = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, pair, a, b)
    a2 = a.copy()
    if dtA == abi.TF32:
        a2.reshape(M, K)[3, 5], a2.reshape(M, K)[7, 9] = 0x7F800000, 0x7FC00001
        b.reshape(N, K)[2, 5] = 0  # inf * 0
    else:
        a2.reshape(M, K)[3, 5], a2.reshape(M, K)[7, 9] = 0x7C00, 0x7E01
        b.reshape(N, K)[2, 5] = 0
    got, want = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, pair, a2, b)
    assert np.isnan(want).any() and np.isinf(want).any()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf])
    fin = np.isfinite(want)
    assert rel_frobenius(got[fin], want[fin]) <= 1e-4
    assert rel_frobenius(clean, want_clean) <= 1e-4
    again, want_again = _gemm_both(calc, orc, abi.OP_ABT, M, N, K, pair, a, b)
    assert np.isfinite(again).all() and rel_frobenius(again, want_again) <= 1e-4
