"""Shared helpers of the test-suite: seeded inputs, descriptors for the oracle, error metrics."""
import ctypes as C

import numpy as np

from intel_gaudi3_software_amd import abi

A = C.addressof


def desc(arr, sizes, dtype, bias=0, mode=0, strides=None):
    """mme_hip_tensor over a numpy buffer (keep the returned struct alive while a C call uses its address)."""
    return abi.make_tensor(arr.ctypes.data, sizes, dtype, bias, mode, strides)


def to_bf16_bits(x):
    """fp32 -> bf16 bit patterns, round to nearest even (inputs are finite test data)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def quantize_fp8(orc, x, dtype, bias, mode=0, clip=True):
    """fp32 -> Gaudi fp8 codes through the oracle's converter (RNE)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.zeros(x.size, np.uint8)
    E = 4 if dtype == abi.FP8_143 else 5
    orc.orc_fp32_to_fp8_n(out.ctypes.data, x.ctypes.data, x.size, E, 7 - E, bias, 0, None, 0, int(clip), 0, 0, mode)
    return out.reshape(x.shape)


def decode_fp8(orc, codes, dtype, bias, mode=0):
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.zeros(codes.size, np.uint32)
    E = 4 if dtype == abi.FP8_143 else 5
    orc.orc_fp8_to_fp32_n(out.ctypes.data, codes.ctypes.data, codes.size, E, 7 - E, bias, mode)
    return out.view(np.float32).reshape(codes.shape)


def random_operand(rng, dtype, n, orc=None, bias=7, mode=0, scale=1.0):
    """Seeded N(0, scale) test data in the storage type of `dtype`."""
    x = (rng.standard_normal(n) * scale).astype(np.float32)
    if dtype == abi.BF16:
        return to_bf16_bits(x)
    if dtype == abi.FP32:
        return x
    if dtype in (abi.FP16, abi.UFP16):
        out = np.zeros(n, np.uint16)
        src = np.abs(x) if dtype == abi.UFP16 else x
        assert orc.orc_cast_from_fp32(out.ctypes.data, dtype, bias, mode, src.ctypes.data, n, 0, None, 0, 0, 0, 1, 0, 0) == 0
        return out
    return quantize_fp8(orc, x, dtype, bias, mode)


def decode_operand(orc, arr, dtype, bias=0, mode=0):
    if dtype == abi.BF16:
        return bf16_bits_to_f32(arr).astype(np.float64)
    if dtype == abi.FP32:
        return arr.astype(np.float64)
    return decode_fp8(orc, arr, dtype, bias, mode).astype(np.float64)


def rel_frobenius(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    den = np.linalg.norm(want.ravel())
    num = np.linalg.norm((got - want).ravel())
    return num / den if den > 0 else num


def cast_sweep_inputs():
    """Every high half of an fp32 crossed with low halves that exercise ties, sticky bits and carries."""
    hi = np.arange(65536, dtype=np.uint32) << 16
    lows = np.array([0, 1, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x4000, 0xC000, 0x1000, 0x2000, 0x3000, 0xF000, 0x0800, 0x1800],
                    dtype=np.uint32)
    return (hi[:, None] | lows[None, :]).ravel().copy()


# relative Frobenius tolerances of the contraction against the reference's fp32-accumulated result
TOL = {abi.BF16: 2e-3, abi.FP32: 2e-3, abi.FP8_143: 1e-2, abi.FP8_152: 1e-2, abi.FP16: 2e-3, abi.UFP16: 2e-3, abi.TF32: 2e-3}


def rmw_operands(rng, dt, n):
    """Pairs that exercise the adder: random magnitudes over the whole exponent range, near-cancellation, exponent gaps
    around the mantissa width (where the smaller operand turns into guard / sticky bits), denormals, zeros of both
    signs, inf, NaN, values next to overflow."""
    if dt == abi.FP32:
        bits, man = np.uint32, 23
        rand = lambda k: rng.integers(0, 2**32, k, dtype=np.uint64).astype(np.uint32)
    else:
        bits, man = np.uint16, 7
        rand = lambda k: rng.integers(0, 2**16, k, dtype=np.uint64).astype(np.uint16)
    a, b = rand(n), rand(n)
    q = n // 8
    # near-cancellation: same exponent, opposite sign, close mantissas
    b[:q] = (a[:q] ^ (1 << (man + 8))) ^ rng.integers(0, 4, q).astype(bits)
    # exponent gaps of man-2 .. man+4 with both signs
    ea = rng.integers(40, 200, q)
    gap = rng.integers(man - 2, man + 5, q)
    sgn = rng.integers(0, 2, (2, q))
    a[q:2 * q] = ((sgn[0] << (man + 8)) | (ea << man) | rng.integers(0, 1 << man, q)).astype(bits)
    b[q:2 * q] = ((sgn[1] << (man + 8)) | ((ea - gap) << man) | rng.integers(0, 1 << man, q)).astype(bits)
    # small exponents: results around the denormal range
    a[2 * q:3 * q] = ((sgn[0] << (man + 8)) | (rng.integers(0, 4, q) << man) | rng.integers(0, 1 << man, q)).astype(bits)
    b[2 * q:3 * q] = ((sgn[1] << (man + 8)) | (rng.integers(0, 4, q) << man) | rng.integers(0, 1 << man, q)).astype(bits)
    # large exponents: overflow
    a[3 * q:4 * q] = ((sgn[0] << (man + 8)) | (rng.integers(252, 256, q) << man) | rng.integers(0, 1 << man, q)).astype(bits)
    b[3 * q:4 * q] = ((sgn[1] << (man + 8)) | (rng.integers(252, 256, q) << man) | rng.integers(0, 1 << man, q)).astype(bits)
    specials = np.array([0, 1 << (man + 8), 0xFF << man, (0xFF << man) | (1 << (man + 8)), (0xFF << man) | 1, 1, (1 << man), (0xFE << man) | ((1 << man) - 1)],
                        dtype=np.uint64).astype(bits)
    k = len(specials)
    a[4 * q:4 * q + k * k] = np.repeat(specials, k)
    b[4 * q:4 * q + k * k] = np.tile(specials, k)
    return a, b


def rmw_operands_fp16(rng, n):
    """The same families for fp16 (5 exponent bits, 10 mantissa bits)."""
    rand = lambda k: rng.integers(0, 1 << 16, k, dtype=np.uint64).astype(np.uint16)
    a, b = rand(n), rand(n)
    q = n // 8
    b[:q] = (a[:q] ^ 0x8000) ^ rng.integers(0, 4, q).astype(np.uint16)
    ea = rng.integers(14, 31, q)
    gap = rng.integers(8, 15, q)
    sgn = rng.integers(0, 2, (2, q))
    a[q:2 * q] = ((sgn[0] << 15) | (ea << 10) | rng.integers(0, 1 << 10, q)).astype(np.uint16)
    b[q:2 * q] = ((sgn[1] << 15) | ((ea - gap) << 10) | rng.integers(0, 1 << 10, q)).astype(np.uint16)
    a[2 * q:3 * q] = ((sgn[0] << 15) | (rng.integers(0, 4, q) << 10) | rng.integers(0, 1 << 10, q)).astype(np.uint16)
    b[2 * q:3 * q] = ((sgn[1] << 15) | (rng.integers(0, 4, q) << 10) | rng.integers(0, 1 << 10, q)).astype(np.uint16)
    a[3 * q:4 * q] = ((sgn[0] << 15) | (rng.integers(28, 32, q) << 10) | rng.integers(0, 1 << 10, q)).astype(np.uint16)
    b[3 * q:4 * q] = ((sgn[1] << 15) | (rng.integers(28, 32, q) << 10) | rng.integers(0, 1 << 10, q)).astype(np.uint16)
    specials = np.array([0, 0x8000, 0x7C00, 0xFC00, 0x7C01, 1, 0x0400, 0x7BFF, 0x03FF, 0x8001, 0xFBFF, 0x3C00], np.uint16)
    k = len(specials)
    a[4 * q:4 * q + k * k] = np.repeat(specials, k)
    b[4 * q:4 * q + k * k] = np.tile(specials, k)
    return a, b


class OracleCalculator:
    """The oracle behind CPUCalculator's method names, on host MmeSimTensor objects: lets the harness sequence
    (intel_gaudi3_software_amd.harness.run_reference_sequence) run on the CPU checker for comparison."""

    def __init__(self, orc, lfsr=None, polynomial=0):
        self.orc = orc
        self.lfsr = np.ascontiguousarray(lfsr, dtype=np.uint32).copy() if lfsr is not None else (np.arange(256, dtype=np.uint32) + 2)
        self.polynomial = polynomial

    def _ok(self, rc):
        assert rc == 0, self.orc.orc_last_error()

    def doBatchGemm(self, out, x, w, op, rm=0, clipFp=False, clipFpInfIn=False, zeroPoints=None):
        self._ok(self.orc.orc_batch_gemm_clip(A(out.desc), A(x.desc), A(w.desc), op, int(clipFp), int(clipFpInfIn)))

    def doConvolution(self, out, x, w, y, params, op, rm=0, clipFp=False, clipFpInfIn=False, zeroPoints=None):
        p = params.pod()
        self._ok(self.orc.orc_convolution_clip(A(out.desc), A(x.desc), A(w.desc), A(y.desc), A(p), op, rm, int(clipFp), int(clipFpInfIn)))

    def doActivation(self, output, acc, res=None, bias=None, relu=False, rm=0, actParams=None, clipFp=False, clipInfIn=False,
                     flushDenorms=False, stochasticFTZfp8=False):
        self._ok(self.orc.orc_activation(A(output.desc), A(acc.desc), int(relu), rm, int(clipFp), int(clipInfIn), int(flushDenorms),
                                         int(stochasticFTZfp8), self.lfsr.ctypes.data, self.polynomial))

    def doMemoryWrite(self, memory, mmeOut, reductionOp=abi.REDUCTION_NONE, reductionRm=0, clipFp=False):
        self._ok(self.orc.orc_memory_write(A(memory.desc), A(mmeOut.desc), reductionOp, reductionRm, int(clipFp)))
