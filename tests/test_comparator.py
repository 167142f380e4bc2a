"""The TensorComparator mirror: its element rule against the reference's own class (compiled into oracle/_ref) on pairs of
codes that sit on both sides of every threshold, and known cases that need no reference build."""
import itertools

import numpy as np
import pytest

from intel_gaudi3_software_amd import MmeSimTensor, abi
from intel_gaudi3_software_amd.comparator import TensorComparator, decode
from helpers import A, desc

NP = {1: np.uint8, 2: np.uint16, 4: np.uint32}
CASES = [(abi.FP8_143, 7, 0), (abi.FP8_143, 3, 2), (abi.FP8_143, 15, 1), (abi.FP8_152, 15, 0), (abi.FP8_152, 1, 1), (abi.FP8_152, 24, 2),
         (abi.BF16, 0, 0), (abi.FP16, 15, 0), (abi.FP16, 9, 1), (abi.UFP16, 31, 0), (abi.UFP16, 31, 1), (abi.FP32, 0, 0)]


def _pairs(rng, dt, n):
    """Code pairs: random, equal, a few codes apart (both sides of the ULP limit), across zero, next to inf / NaN."""
    bits = 8 * abi.DTYPE_SIZE[dt]
    t = NP[abi.DTYPE_SIZE[dt]]
    a = rng.integers(0, 1 << bits, n, dtype=np.uint64)
    if bits == 32:  # keep most fp32 exponents moderate so that the absolute and relative bounds matter
        a[: n // 2] = (rng.standard_normal(n // 2) * np.exp2(rng.integers(-8, 8, n // 2))).astype(np.float32).view(np.uint32)
    delta = rng.integers(-40, 41, n)
    if bits == 32:
        delta = delta * rng.choice([1, 1 << 8, 1 << 16, 1 << 20], n)
    b = (a.astype(np.int64) + delta) % (1 << bits)
    q = n // 6
    b[:q] = rng.integers(0, 1 << bits, q, dtype=np.uint64)     # unrelated
    b[q:q + q // 2] = a[q:q + q // 2]                           # equal
    b[2 * q:2 * q + q // 2] = a[2 * q:2 * q + q // 2] ^ (1 << (bits - 1))  # sign flipped
    return a.astype(t), b.astype(t)


@pytest.mark.parametrize("dt,bias,mode", CASES)
def test_element_rule_matches_the_reference_class(ref, dt, bias, mode):
    rng = np.random.default_rng(dt * 100 + bias)
    n = 6000
    a, b = _pairs(rng, dt, n)
    for cd in (1, 64, 27000, 1 << 20, 3 << 24):
        want = np.zeros(n, np.uint8)
        ref.ref_compare_elements(want.ctypes.data, a.ctypes.data, b.ctypes.data, n, dt, bias, mode, cd)
        got = TensorComparator(cd, dt, bias, mode).compare_codes(a, b)
        bad = np.flatnonzero(got != want.astype(bool))
        assert bad.size == 0, (cd, hex(int(a[bad[0]])), hex(int(b[bad[0]])), bool(want[bad[0]]))
        assert 0 < want.sum() < n


def test_whole_tensors_first_mismatch_and_stride_holes(ref, capsys):
    rng = np.random.default_rng(3)
    sizes, strides = [5, 4, 3, 1, 1], [1, 7, 30, 90, 90]
    span = 90
    a = (rng.standard_normal(span) * 4).astype(np.float32)
    b = a.copy()
    b[6] = 1e9      # a stride hole (row pitch 7, row length 5): not an element
    ta, tb = MmeSimTensor(sizes, 3, abi.FP32, a, strides=strides), MmeSimTensor(sizes, 3, abi.FP32, b, strides=strides)
    cmp = TensorComparator(64, abi.FP32)
    assert cmp.doCompare(ta, "a", tb, "b") and cmp.getDiffElement() is None
    assert cmp.doCompareBitExact(ta, "a", tb, "b")
    diff = np.zeros(5, np.uint32)
    assert ref.ref_compare_tensors(A(ta.desc), A(tb.desc), 64, 0, diff.ctypes.data) == 1
    assert ref.ref_compare_tensors(A(ta.desc), A(tb.desc), 64, 1, diff.ctypes.data) == 1
    b[2 + 7 * 3 + 30 * 1] += 100.0   # element (2, 3, 1)
    b[4 + 7 * 1 + 30 * 2] += 1e-6    # element (4, 1, 2): within tolerance, but not bit-exact
    assert not cmp.doCompare(ta, "mine", tb, "theirs", 3, "details")
    assert cmp.getDiffElement() == [2, 3, 1, 0, 0]
    assert ref.ref_compare_tensors(A(ta.desc), A(tb.desc), 64, 0, diff.ctypes.data) == 0 and list(diff) == [2, 3, 1, 0, 0]
    out = capsys.readouterr().out
    assert "ERROR: Comparison mismatch. mine <-> theirs. (test #3)" in out and "Mismatch at element  [2, 3, 1, 0, 0]" in out
    b[2 + 7 * 3 + 30 * 1] = a[2 + 7 * 3 + 30 * 1]
    assert cmp.doCompare(ta, "a", tb, "b")
    # bit-exact: the reference walks raw buffer positions and names them as if the tensor were dense
    for raw_index in (71, 53, 6, 10, 59, 61, 89):
        b[:] = a
        b[raw_index] += 1.0
        want = ref.ref_compare_tensors(A(ta.desc), A(tb.desc), 64, 1, diff.ctypes.data)
        assert cmp.doCompareBitExact(ta, "a", tb, "b") == bool(want), raw_index
        if not want:
            assert cmp.getDiffElement() == [int(v) for v in diff], raw_index


@pytest.mark.parametrize("dt,bias,mode", [(abi.BF16, 0, 0), (abi.FP16, 15, 0), (abi.FP16, 9, 1), (abi.UFP16, 31, 0), (abi.FP32, 0, 0)])
@pytest.mark.parametrize("num_partials", [2, 3, 5])
def test_partial_sum_rule_matches_the_reference_class(ref, dt, bias, mode, num_partials):
    """numPartials > 1: the first tensor holds partial results, the second their sum (tensor_comparator_impl.cpp:373-413).
    Groups whose rounded fp32 sum equals, nearly equals or misses the second tensor's element, incl. sums that overflow
    the type, cancel to zero or involve inf / NaN, element by element against the reference's class; then whole tensors."""
    rng = np.random.default_rng(dt * 10 + num_partials)
    n = 4000
    t = NP[abi.DTYPE_SIZE[dt]]
    bits = 8 * abi.DTYPE_SIZE[dt]
    from intel_gaudi3_software_amd.comparator import encode_rne
    default_bias = {abi.FP16: 15, abi.UFP16: 31}.get(dt, 0)
    vals = (rng.standard_normal((n, num_partials)) * np.exp2(rng.integers(-6, 7, (n, 1)))).astype(np.float32)
    if dt == abi.UFP16:
        vals = np.abs(vals)
    vals[: n // 8] *= np.float32(2.0 ** 14)                      # sums near and beyond fp16's largest value
    vals[n // 8: n // 4, 1] = -vals[n // 8: n // 4, 0]            # cancellation
    a = encode_rne(vals.ravel(), dt, default_bias).astype(t)
    a[rng.integers(0, a.size, 40)] = rng.integers(0, 1 << bits, 40, dtype=np.uint64).astype(t)   # arbitrary codes, inf and NaN among them
    total = np.zeros(n, np.float32)
    dec = decode(a, dt, default_bias, 0).reshape(n, num_partials)
    with np.errstate(invalid="ignore", over="ignore"):
        for p in range(num_partials):
            total = (total + dec[:, p]).astype(np.float32)
    b = encode_rne(total, dt, default_bias).astype(np.int64)
    b += rng.choice([0, 0, 1, -1, 3, -6, 40, 3000], n)            # equal, a few codes apart, far apart
    b = (b % (1 << bits)).astype(t)
    for cd in (1, 27000, 1 << 20):
        want = np.zeros(n, np.uint8)
        ref.ref_compare_elements_partials(want.ctypes.data, a.ctypes.data, b.ctypes.data, n, num_partials, dt, bias, mode, cd)
        cmp = TensorComparator(cd, dt, bias, mode)
        got = cmp.compare_codes(cmp._sum_partials(np.ascontiguousarray(a.reshape(n, num_partials).T).ravel(), n, num_partials), b)
        bad = np.flatnonzero(got != want.astype(bool))
        assert bad.size == 0, (cd, [hex(int(v)) for v in a.reshape(n, num_partials)[bad[0]]], hex(int(b[bad[0]])), bool(want[bad[0]]))
        assert want.sum() > 0 and (cd > 1 or want.sum() < n)
    # whole tensors: partials stacked along the last dimension, first mismatch reported by its coordinates in the sum tensor
    sizes = [6, 5, 4, 1, 1]
    nb = 120
    pa = encode_rne((rng.standard_normal(nb * num_partials) * 8).astype(np.float32), dt, default_bias).astype(t)
    if dt == abi.UFP16:
        pa = encode_rne(np.abs(rng.standard_normal(nb * num_partials) * 8).astype(np.float32), dt, default_bias).astype(t)
    cmp = TensorComparator(64, dt, bias, mode)
    sb = cmp._sum_partials(pa, nb, num_partials).astype(t)
    ta = MmeSimTensor([6, 5, 4 * num_partials, 1, 1], 3, dt, pa, bias, mode)
    tb = MmeSimTensor(sizes, 3, dt, sb, bias, mode)
    diff = np.zeros(5, np.uint32)
    assert cmp.doCompare(ta, "partials", tb, "sum", numPartials=num_partials)
    assert ref.ref_compare_tensors_partials(A(ta.desc), A(tb.desc), 64, num_partials, diff.ctypes.data) == 1
    sb[2 + 6 * 3 + 30 * 1] ^= t(1 << (bits - 2))   # element (2, 3, 1): the exponent's top bit
    assert not cmp.doCompare(ta, "partials", tb, "sum", numPartials=num_partials, failOnMismatch=False)
    assert ref.ref_compare_tensors_partials(A(ta.desc), A(tb.desc), 64, num_partials, diff.ctypes.data) == 0
    assert cmp.getDiffElement() == [int(v) for v in diff] == [2, 3, 1, 0, 0]


def test_partial_sums_of_fp8_tensors_are_refused():
    t8 = MmeSimTensor([4, 1, 1, 1, 1], 1, abi.FP8_143, np.zeros(4, np.uint8), 7)
    t2 = MmeSimTensor([2, 1, 1, 1, 1], 1, abi.FP8_143, np.zeros(2, np.uint8), 7)
    with pytest.raises(ValueError):
        TensorComparator(8, abi.FP8_143, 7).doCompare(t8, "a", t2, "b", numPartials=2)


def test_known_cases():
    """Cases that follow from the rule's text: NaN never compares equal, equal infinities do, an infinity against a number
    does not, small values compare by absolute tolerance, large ones by code distance."""
    c = TensorComparator(64, abi.BF16)   # maxULP = max(4, 320 >> 16) = 4
    bf = lambda *v: (np.array(v, np.float32).view(np.uint32) >> 16).astype(np.uint16)
    assert c.max_ulp == 4 and abs(float(c.abs_tol) - 0.05) < 1e-9
    a = bf(np.nan, np.inf, np.inf, 0.01, 0.0, 100.0, 100.0, -1.0, 3.0)
    b = bf(np.nan, np.inf, 5.0, 0.05, 0.04, 102.0, 104.0, 1.0, 3.3)
    #        NaN   =inf    inf/5  |d|<.05+  0 vs .04  4 codes  8 codes  signs   |d|=.3 <= .05+.3
    assert list(c.compare_codes(a, b)) == [False, True, False, True, True, True, False, False, True]
    c8 = TensorComparator(1 << 22, abi.FP8_143, 7)   # maxULP = (5 << 22) >> 20 = 20
    assert c8.max_ulp == 20
    assert abs(float(TensorComparator(1, abi.FP8_152, 1, 0).abs_tol) - 1.0) < 1e-9   # the code 4 of fp8_152 with bias 1 is 2^0
    with pytest.raises(ValueError):
        TensorComparator(1, abi.TF32)


def test_decoders_agree_with_the_oracle(orc):
    for dt, bias, mode in CASES[:11]:
        bits = 8 * abi.DTYPE_SIZE[dt]
        codes = np.arange(1 << bits).astype(NP[abi.DTYPE_SIZE[dt]])
        want = np.zeros(codes.size, np.float32)
        assert orc.orc_cast_to_fp32(want.ctypes.data, codes.ctypes.data, dt, bias, mode, codes.size, 0, None, 0) == 0
        got = decode(codes, dt, bias, mode)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
