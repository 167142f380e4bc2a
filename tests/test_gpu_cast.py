"""GPU casts against the oracle: bit-exact (integer comparison of the encoded outputs)."""
import itertools

import numpy as np
import pytest

from intel_gaudi3_software_amd import abi
from helpers import A, cast_sweep_inputs, desc

pytestmark = pytest.mark.gpu

FORMATS = [(abi.FP8_143, 3), (abi.FP8_143, 7), (abi.FP8_143, 11), (abi.FP8_143, 15), (abi.FP8_152, 1), (abi.FP8_152, 15),
           (abi.FP8_152, 30), (abi.BF16, 0), (abi.FP32, 0)]
TORCH_OUT = {abi.FP8_143: "uint8", abi.FP8_152: "uint8", abi.BF16: "int16", abi.FP32: "int32"}


def _oracle_cast(orc, dt, bias, mode, x, scale_exp=0, col=None, n_cols=0, relu=0, rm=0, clip=0, cinf=0, ftz=0):
    out = np.zeros(x.size, abi.DTYPE_NUMPY[dt] if dt != abi.FP32 else np.uint32)
    rc = orc.orc_cast_from_fp32(out.ctypes.data, dt, bias, mode, x.ctypes.data, x.size, scale_exp,
                                col.ctypes.data if col is not None else None, n_cols, relu, rm, clip, cinf, ftz)
    assert rc == 0, orc.orc_last_error()
    return out


def _gpu_cast(calc, dt, bias, mode, x, scale_exp=0, col=None, n_cols=0, relu=0, rm=0, clip=0, cinf=0, ftz=0, offset=0):
    import torch
    xin = torch.zeros(x.size + offset, dtype=torch.float32, device="cuda")
    xin[offset:] = torch.from_numpy(x.view(np.int32)).cuda().view(torch.float32)
    out = torch.zeros(x.size + 16, dtype=getattr(torch, TORCH_OUT[dt]), device="cuda")
    dcol = torch.from_numpy(col).cuda() if col is not None else None
    calc.castFromFp32(out, dt, xin[offset:], x.size, bias, mode, scale_exp, dcol, n_cols, relu, rm, clip, cinf, ftz)
    calc.synchronize()
    res = out.cpu().numpy()[:x.size]
    return res.view(np.uint16) if dt == abi.BF16 else (res.view(np.uint32) if dt == abi.FP32 else res)


@pytest.mark.parametrize("dt,bias", FORMATS)
def test_cast_sweep_all_modes(calc, orc, dt, bias):
    """Structured sweep (every high half x tie/sticky low halves) in every deterministic rounding mode."""
    x = cast_sweep_inputs().view(np.float32)
    modes = [0, 1, 2] if dt in (abi.FP8_143, abi.FP8_152) else [0]
    for mode, rm, (clip, cinf), ftz in itertools.product(modes, [0, 1, 2, 3, 6], [(0, 0), (1, 0), (1, 1)], [0, 1]):
        want = _oracle_cast(orc, dt, bias, mode, x, rm=rm, clip=clip, cinf=cinf, ftz=ftz)
        got = _gpu_cast(calc, dt, bias, mode, x, rm=rm, clip=clip, cinf=cinf, ftz=ftz)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "dt=%d bias=%d mode=%d rm=%d clip=%d/%d ftz=%d: %d mismatches, first x=%#x got=%#x want=%#x" % (
            dt, bias, mode, rm, clip, cinf, ftz, bad.size, x.view(np.uint32)[bad[0]], got[bad[0]], want[bad[0]])


@pytest.mark.parametrize("dt,bias", [(abi.FP8_143, 7), (abi.FP8_152, 15), (abi.BF16, 0), (abi.FP32, 0)])
def test_cast_scaled_relu_ragged(calc, orc, dt, bias):
    """Quantise-with-scale: per-tensor and per-column powers of two, relu, ragged length, unaligned start."""
    rng = np.random.default_rng(11)
    for n, n_cols, offset in [(4096 * 5 + 3, 64, 0), (1000, 24, 0), (777, 7, 1), (5, 5, 0), (1, 1, 0), (0, 0, 0)]:
        x = (rng.standard_normal(n) * np.exp2(rng.integers(-14, 14, n))).astype(np.float32)
        if n > 10:
            x[3] = np.inf
            x[5] = -np.inf
            x[7] = np.nan
            x[9] = -0.0
        col = rng.integers(-6, 7, n_cols).astype(np.int32) if n_cols else None
        for scale_exp, relu, clip in [(0, 0, 1), (-3, 1, 1), (5, 0, 0)]:
            want = _oracle_cast(orc, dt, bias, 0, x, scale_exp, col, n_cols, relu, 0, clip, 0, 0)
            got = _gpu_cast(calc, dt, bias, 0, x, scale_exp, col, n_cols, relu, 0, clip, 0, 0, offset=offset)
            if dt == abi.FP32:
                # NaN payloads after a multiplication are not pinned by the reference; compare NaN-ness there
                nan = np.isnan(want.view(np.float32))
                assert np.array_equal(np.isnan(got.view(np.float32)), nan)
                got, want = got[~nan], want[~nan]
            assert np.array_equal(got, want), (n, n_cols, offset, scale_exp, relu, clip)


@pytest.mark.parametrize("dt,bias,mode", [(abi.FP8_143, 3, 0), (abi.FP8_143, 7, 0), (abi.FP8_143, 7, 2), (abi.FP8_143, 15, 1),
                                          (abi.FP8_152, 15, 0), (abi.FP8_152, 1, 2), (abi.FP8_152, 30, 1), (abi.BF16, 0, 0)])
def test_dequantize(calc, orc, dt, bias, mode):
    import torch
    rng = np.random.default_rng(5)
    if dt == abi.BF16:
        codes = np.arange(65536, dtype=np.uint16)
        tin = torch.from_numpy(codes.view(np.int16)).cuda()
    else:
        codes = np.concatenate([np.arange(256, dtype=np.uint8), rng.integers(0, 256, 1003).astype(np.uint8)])
        tin = torch.from_numpy(codes).cuda()
    n = codes.size
    col = rng.integers(-4, 5, 12).astype(np.int32)
    for scale_exp, use_col in [(0, False), (-7, False), (3, True)]:
        want = np.zeros(n, np.float32)
        rc = orc.orc_cast_to_fp32(want.ctypes.data, codes.ctypes.data, dt, bias, mode, n, scale_exp,
                                  col.ctypes.data if use_col else None, 12 if use_col else 0)
        assert rc == 0
        out = torch.zeros(n, dtype=torch.float32, device="cuda")
        calc.castToFp32(out, tin, dt, n, bias, mode, scale_exp, torch.from_numpy(col).cuda() if use_col else None,
                        12 if use_col else 0)
        calc.synchronize()
        got = out.cpu().numpy()
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


def test_absmax(calc):
    import torch
    rng = np.random.default_rng(3)
    for n in [1, 63, 4097, 1 << 20]:
        x = rng.standard_normal(n).astype(np.float32)
        x[rng.integers(0, n)] = np.nan
        want = np.nanmax(np.abs(x)) if n > 1 else (0.0 if np.isnan(x[0]) else abs(x[0]))
        out = torch.zeros(1, dtype=torch.float32, device="cuda")
        calc.absmax(out, torch.from_numpy(x).cuda(), n)
        calc.synchronize()
        assert out.item() == np.float32(want)


def test_activation_matches_reference_sequence(calc, orc):
    """doActivation through tensor descriptors, host and device resident, relu rewriting acc in place."""
    import torch
    from intel_gaudi3_software_amd import MmeSimTensor
    rng = np.random.default_rng(9)
    sizes = [48, 5, 3, 2, 1]
    n = int(np.prod(sizes))
    acc0 = (rng.standard_normal(n) * 300).astype(np.float32)
    acc0[::17] = np.nan
    for dt, bias in [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP8_152, 15), (abi.FP32, 0)]:
        for relu, rm, clip in [(False, 0, True), (True, 0, True), (True, 1, False), (False, 6, True)]:
            a_ref = acc0.copy()
            o_ref = np.zeros(n * abi.DTYPE_SIZE[dt], np.uint8)
            d_o, d_a = desc(o_ref, sizes, dt, bias), desc(a_ref, sizes, abi.FP32)
            assert orc.orc_activation(A(d_o), A(d_a), int(relu), rm, int(clip), 0, 0, 0, None, 0) == 0
            # host tensors
            a_h = acc0.copy()
            o_h = np.zeros(n, abi.DTYPE_NUMPY[dt])
            calc.doActivation(MmeSimTensor(sizes, 5, dt, o_h, bias), MmeSimTensor(sizes, 5, abi.FP32, a_h), relu=relu, rm=rm,
                              clipFp=clip)
            assert np.array_equal(o_h.view(np.uint8), o_ref)
            assert np.array_equal(a_h.view(np.uint32), a_ref.view(np.uint32))
            # device tensors
            a_d = torch.from_numpy(acc0.copy()).cuda()
            o_d = torch.zeros(n * abi.DTYPE_SIZE[dt], dtype=torch.uint8, device="cuda")
            td = {abi.BF16: torch.int16, abi.FP32: torch.float32}.get(dt, torch.uint8)
            calc.doActivation(MmeSimTensor(sizes, 5, dt, o_d.view(td), bias), MmeSimTensor(sizes, 5, abi.FP32, a_d), relu=relu,
                              rm=rm, clipFp=clip)
            calc.synchronize()
            assert np.array_equal(o_d.cpu().numpy(), o_ref)
            assert np.array_equal(a_d.cpu().numpy().view(np.uint32), a_ref.view(np.uint32))


@pytest.mark.parametrize("dt,bias,mode", [(abi.FP8_143, 7, 0), (abi.FP8_143, 3, 2), (abi.FP8_152, 15, 0), (abi.FP8_152, 20, 1), (abi.BF16, 0, 0)])
@pytest.mark.parametrize("rm,sftz,ftz", [(4, 0, 0), (7, 0, 0), (4, 1, 1), (0, 1, 1), (7, 0, 1), (2, 1, 0)])
def test_activation_stochastic_modes_follow_the_reference_lfsr(orc, dt, bias, mode, rm, sftz, ftz):
    """Stochastic rounding (modes 4 and 7) and stochastic flush draw from the calculator's LFSR registers: element i uses
    register i % 128 (fp8) / i % 64 (bf16), stepped after every use, and the registers persist between calls.  Two
    calls in a row (the second shorter and ragged) against the oracle's doActivation with the same registers and
    polynomial: outputs bit for bit, which also pins the state the first call leaves behind."""
    import torch
    from intel_gaudi3_software_amd import HipCalculator, MmeSimTensor
    rng = np.random.default_rng(77)
    lfsr0 = rng.integers(1, 2**32, 256, dtype=np.uint64).astype(np.uint32)
    poly = 0xD0000001
    calc = HipCalculator(lfsrNumRegs=256, lfsr=lfsr0, polynomial=poly)
    lfsr_ref = lfsr0.copy()
    for n in [128 * 300 + 77, 5003]:
        man = 3 if dt == abi.FP8_143 else 2
        # magnitudes across the target's denormal, normal and overflow ranges
        lo = (1 - bias - man - 3) if dt != abi.BF16 else -140
        hi = ((1 << (7 - man)) - bias + 1) if dt != abi.BF16 else 128
        with np.errstate(over="ignore"):
            x = (rng.standard_normal(n) * np.exp2(rng.integers(lo, hi, n))).astype(np.float32)
        x[::97] = 0.0
        x[5::211] = np.inf
        x[7::223] = np.nan
        sizes = [n, 1, 1, 1, 1]
        o_ref = np.zeros(n * abi.DTYPE_SIZE[dt], np.uint8)
        a_ref = x.copy()
        d_o, d_a = desc(o_ref, sizes, dt, bias, mode), desc(a_ref, sizes, abi.FP32)
        assert orc.orc_activation(A(d_o), A(d_a), 0, rm, 1, 0, ftz, sftz, lfsr_ref.ctypes.data, poly) == 0
        a_d = torch.from_numpy(x.copy()).cuda()
        td = torch.int16 if dt == abi.BF16 else torch.uint8
        o_d = torch.zeros(n, dtype=td, device="cuda")
        calc.doActivation(MmeSimTensor(sizes, 5, dt, o_d, bias, mode), MmeSimTensor(sizes, 5, abi.FP32, a_d), relu=False, rm=rm, clipFp=True,
                          flushDenorms=bool(ftz), stochasticFTZfp8=bool(sftz))
        calc.synchronize()
        got = o_d.cpu().numpy().view(np.uint8)
        assert np.array_equal(got, o_ref), (n, int(np.flatnonzero(got != o_ref)[0]))
    calc.close()


@pytest.mark.parametrize("dt", [abi.FP32, abi.BF16, abi.FP16, abi.FP8_152])
def test_memory_write_reductions(calc, orc, dt):
    """doMemoryWrite with add / sub / min / max / max_0, every reduction rounding mode, clipping on and off, device and host
    tensors: bit for bit against the oracle (pinned against the reference's executeOp).  Operands cover cancellation,
    exponent gaps around the mantissa width, denormals, signed zeros, inf, NaN, overflow; ragged length."""
    import torch
    from intel_gaudi3_software_amd import MmeSimTensor
    from helpers import rmw_operands, rmw_operands_fp16
    rng = np.random.default_rng(33)
    n = (1 << 16) + 3
    if dt == abi.FP8_152:  # every pair of codes, and three more elements for a ragged length
        pairs = np.arange(65536 + 3, dtype=np.uint32)
        a, b = (pairs >> 8).astype(np.uint8), (pairs & 0xFF).astype(np.uint8)
    else:
        a, b = rmw_operands_fp16(rng, n) if dt == abi.FP16 else rmw_operands(rng, dt, n)
    sizes = [n, 1, 1, 1, 1]
    td = {abi.FP32: torch.int32, abi.FP8_152: torch.uint8}.get(dt, torch.int16)
    sview = {abi.FP32: np.int32, abi.FP8_152: np.uint8}.get(dt, np.int16)
    tb = torch.from_numpy(b.view(sview)).cuda()
    for op, rm, clip in itertools.product(range(5), range(4), (0, 1)):
        if op in (abi.REDUCTION_MIN, abi.REDUCTION_MAX) and (rm or clip):
            continue
        want = a.copy()
        d_m, d_o = desc(want, sizes, dt), desc(b, sizes, dt)
        assert orc.orc_memory_write(A(d_m), A(d_o), op, rm, clip) == 0
        tm = torch.from_numpy(a.copy().view(sview)).cuda()
        calc.doMemoryWrite(MmeSimTensor(sizes, 5, dt, tm), MmeSimTensor(sizes, 5, dt, tb), op, rm, bool(clip))
        calc.synchronize()
        got = tm.cpu().numpy().view(a.dtype)
        bad = np.flatnonzero(got != want)
        assert bad.size == 0, (op, rm, clip, hex(int(a[bad[0]])), hex(int(b[bad[0]])), hex(int(got[bad[0]])), hex(int(want[bad[0]])))
    # host tensors, one setting; and reduction none as a copy
    want = a.copy()
    d_m, d_o = desc(want, sizes, dt), desc(b, sizes, dt)
    assert orc.orc_memory_write(A(d_m), A(d_o), abi.REDUCTION_ADD, 0, 1) == 0
    hm = a.copy()
    calc.doMemoryWrite(MmeSimTensor(sizes, 5, dt, hm), MmeSimTensor(sizes, 5, dt, b.copy()), abi.REDUCTION_ADD, 0, True)
    assert np.array_equal(hm, want)
    tm = torch.zeros(n, dtype=td, device="cuda")
    calc.doMemoryWrite(MmeSimTensor(sizes, 5, dt, tm), MmeSimTensor(sizes, 5, dt, tb))
    calc.synchronize()
    assert np.array_equal(tm.cpu().numpy().view(a.dtype), b)


@pytest.mark.parametrize("dt,bias", [(abi.BF16, 0), (abi.FP8_143, 7), (abi.FP16, 15), (abi.FP32, 0)])
def test_activation_converts_the_whole_span_of_strided_tensors(calc, orc, dt, bias):
    """A strided output: the reference's doActivation converts every flat element of the tensor's span, the gaps between
    rows included; device and host tensors against the oracle, bit for bit.  relu on such a tensor is refused like the
    reference refuses it."""
    import torch
    from intel_gaudi3_software_amd import MMEStackException, MmeSimTensor
    rng = np.random.default_rng(26)
    sizes, strides = [5, 4, 3, 1, 1], [1, 7, 30, 90, 90]
    acc = rng.standard_normal(90).astype(np.float32)
    want = np.full(90, 0x11, abi.DTYPE_NUMPY[dt])
    a_ref = acc.copy()
    d_o, d_a = desc(want, sizes, dt, bias, 0, strides), desc(a_ref, sizes, abi.FP32, 0, 0, strides)
    assert orc.orc_activation(A(d_o), A(d_a), 0, 0, 1, 0, 0, 0, None, 0) == 0
    host_out, host_acc = np.full(90, 0x11, abi.DTYPE_NUMPY[dt]), acc.copy()
    calc.doActivation(MmeSimTensor(sizes, 5, dt, host_out, bias, 0, strides), MmeSimTensor(sizes, 5, abi.FP32, host_acc, strides=strides), clipFp=True)
    assert np.array_equal(host_out.view(np.uint8), want.view(np.uint8))
    view = {1: np.uint8, 2: np.int16, 4: np.float32}[abi.DTYPE_SIZE[dt]]
    o_d = torch.from_numpy(np.full(90, 0x11, abi.DTYPE_NUMPY[dt]).view(view).copy()).cuda()
    a_d = torch.from_numpy(acc.copy()).cuda()
    calc.doActivation(MmeSimTensor(sizes, 5, dt, o_d, bias, 0, strides), MmeSimTensor(sizes, 5, abi.FP32, a_d, strides=strides), clipFp=True)
    calc.synchronize()
    assert np.array_equal(o_d.cpu().numpy().view(np.uint8), want.view(np.uint8))
    with pytest.raises(MMEStackException, match="should be flattened"):
        calc.doActivation(MmeSimTensor(sizes, 5, dt, o_d, bias, 0, strides), MmeSimTensor(sizes, 5, abi.FP32, a_d, strides=strides), relu=True)
