"""The reference's own Gaudi3 test configurations (mme/mme_verification/gaudi3/configs, kept as data under
tests/golden/configs/gaudi3) through the harness seam: every test whose operation and types the calculator path covers
and whose contraction the CPU checker can afford runs MmeTestManager::runReference's sequence (contraction -> doActivation
-> doMemoryWrite) once on the GPU library and once on the oracle, on the same operands."""
import glob
import os

import numpy as np
import pytest

from intel_gaudi3_software_amd import MmeSimTensor, abi, harness
from helpers import A, OracleCalculator, TOL, rel_frobenius

pytestmark = pytest.mark.gpu

CONFIG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "configs", "gaudi3")
MAX_FLOPS = 1.2e9  # per test, for the CPU checker
RANDOM_SIZE_SEEDS = (1, 2, 3, 4, 5, 6, 7, 8)
REPORT = []  # (test id, input type, output type, stochastic, relative Frobenius distance, share of equal codes)


def _like_for_like_tolerance(t, out_dtype):
    """Bound on the relative Frobenius distance between the GPU's and the reference's outputs of one test, both decoded
    from the output type: the bound the accumulators themselves are held to (1e-2 for fp8 operands, 2e-3 for the others).
    The two accumulators differ in their last bits, so a rounded output lands on the neighbouring code where they straddle
    a rounding boundary; with accumulators a relative distance d apart and codes a relative step s apart that happens to a
    share d / s of the elements and each such element is off by s, a distance of sqrt(d * s) in all."""
    return TOL[t["in_type"]]


@pytest.fixture(scope="module", autouse=True)
def _parity_report():
    yield
    out = os.environ.get("MME_PARITY_REPORT")
    if out and REPORT:
        import json
        with open(out, "w") as f:
            json.dump(REPORT, f)


def _key(t):
    return (t["operation"], t["in_type"], t["in2_type"], t["out_type"], tuple(t["x_sizes"]), tuple(t["w_sizes"]), tuple(t["y_sizes"]),
            tuple(t["x_strides"] or ()), tuple(t["w_strides"] or ()), tuple(t["y_strides"] or ()), tuple(t["padding"]),
            tuple(t["conv_strides"]), tuple(t["dilation"]), t["fp8_bias_in"], t["fp8_bias_in2"], t["fp8_bias_out"], t["inf_nan_a"],
            t["inf_nan_b"], t["inf_nan_out"], t["rounding"], t["reduction_op"], t["reduction_rm"], t["clip"], t["clip_inf_in"],
            t["flush_denormals"], t["stochastic_flush"], t["relu"])


def _collect(large=False):
    cases, seen = [], set()
    for path in sorted(glob.glob(os.path.join(CONFIG_DIR, "*", "*.json"))):
        # a configuration with "random" sizes is a different test for every seed: eight fixed seeds of those, one of the rest
        seeds = RANDOM_SIZE_SEEDS if os.path.basename(os.path.dirname(path)) == "random_tests" else (7,)
        loaded = [(i, sd, test) for sd in seeds for i, test in enumerate(harness.load_tests(path, seed=sd))]
        for i, sd, test in loaded:
            if harness.supported(test) is not None:
                continue
            if any(v <= 0 for v in test["x_sizes"] + test["w_sizes"] + test["y_sizes"]):
                continue  # (a random filter no larger than twice its padding can leave no input pixel)
            if len(seeds) > 1:
                i = "seed%d" % sd
            for g, t in enumerate(harness.gemms_of(test)):  # (a dual-GEMM test is two contractions)
                if (harness.contraction_flops(t) > MAX_FLOPS) != large:
                    continue
                k = _key(t)
                if k in seen:  # tests that differ only in descriptor-generation parameters are one case for the calculator
                    continue
                seen.add(k)
                cases.append(pytest.param(t, id="%s-%s%s-%s" % (os.path.basename(path)[:-5], i, ".%d" % g if test["dual_gemm"] else "", t["operation_name"])))
    return cases


def _quantise(orc, values, dtype, bias, mode):
    out = np.zeros(values.size, abi.DTYPE_NUMPY[dtype])
    if dtype == abi.FP32:
        out[:] = values
        return out
    if dtype == abi.TF32:  # fp32 words; the contraction rounds them on entry
        return values.view(np.uint32).copy()
    assert orc.orc_cast_from_fp32(out.ctypes.data, dtype, bias, mode, values.ctypes.data, values.size, 0, None, 0, 0, 0, 1, 0, 0) == 0
    return out


def _decode(orc, codes, dtype, bias, mode):
    if dtype == abi.FP32:
        return codes.view(np.float32).copy()
    out = np.zeros(codes.size, np.float32)
    assert orc.orc_cast_to_fp32(out.ctypes.data, codes.ctypes.data, dtype, bias, mode, codes.size, 0, None, 0) == 0
    return out


@pytest.mark.parametrize("t", _collect())
def test_reference_config(calc, orc, t):
    types = harness.tensor_types(t)
    a_l, b_l, o_l = harness.operand_roles(t)
    values = harness.make_operand_values(t, seed=11)
    host = {}
    for letter in (a_l, b_l):
        dtype, bias, mode = types[letter]
        # (the generator cuts the draws to the finite range of the element type, so no operand holds inf or NaN)
        host[letter] = _quantise(orc, values[letter], dtype, bias, mode)
    mk = lambda letter: MmeSimTensor(t[letter + "_sizes"], 5, types[letter][0], host[letter].copy(), types[letter][1], types[letter][2],
                                     t[letter + "_strides"])
    out_dtype, out_bias, out_mode = types[o_l]
    n_out = max(st * sz for st, sz in zip(MmeSimTensor(t[o_l + "_sizes"], 5, out_dtype, None, out_bias, out_mode, t[o_l + "_strides"]).strides,
                                          t[o_l + "_sizes"] + [1] * 5))
    prev = None
    if t["reduction_op"] != abi.REDUCTION_NONE:
        rng = np.random.default_rng(5)
        prev = _quantise(orc, rng.uniform(-4, 4, n_out).astype(np.float32), out_dtype, out_bias, out_mode)
    lfsr = (np.arange(256, dtype=np.uint32) * 2654435761 + 12345).astype(np.uint32)
    poly = 0xB4BCD35C
    from intel_gaudi3_software_amd import HipCalculator
    gpu = HipCalculator(lfsrNumRegs=256, lfsr=lfsr, polynomial=poly) if t["uses_lfsr"] else calc
    cpu = OracleCalculator(orc, lfsr, poly)
    results = []
    for c in (gpu, cpu):
        tensors = {a_l: mk(a_l), b_l: mk(b_l)}
        p = None if prev is None else MmeSimTensor(t[o_l + "_sizes"], 5, out_dtype, prev.copy(), out_bias, out_mode, t[o_l + "_strides"])
        results.append(harness.run_reference_sequence(c, t, tensors, p))
    if gpu is not calc:
        gpu.close()
    # the test manager's own acceptance rule (TensorComparator with the tolerances of this contraction length and output
    # type) must accept the GPU output against the reference-semantics output; NaN never passes that rule, so only where
    # the expected tensor has none
    expected = _decode(orc, np.ascontiguousarray(results[1].data()), out_dtype, out_bias, out_mode)
    if not np.any(np.isnan(expected)):
        assert harness.compare_with_reference(t, results[0], results[1])
    results = [r.data() for r in results]
    got, want = (_decode(orc, np.ascontiguousarray(r), out_dtype, out_bias, out_mode) for r in results)
    fin = np.isfinite(want)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
    # the accumulators differ in the last bits (IEEE FMA order on the GPU, the Gaudi3 truncating tree in the reference), so
    # a rounded output may land on the neighbouring code; stochastic modes amplify that to one code wherever the draw falls
    # between the two accumulators
    dist = rel_frobenius(got[fin], want[fin])
    same = float(np.mean(results[0] == results[1]))
    REPORT.append((t["name"], t["operation_name"], t["in_type"], out_dtype, bool(t["uses_lfsr"]), harness.cd_size(t), float(dist), same))
    assert dist <= _like_for_like_tolerance(t, out_dtype), dist
    if out_dtype != abi.FP32:  # (fp32 outputs are the accumulators themselves)
        # (0.8: the longest reductions of the set, 10^5 products, let the tree's truncation reach a quarter of a bf16 ulp)
        assert same >= (0.5 if t["uses_lfsr"] else 0.8), same


def test_external_reference_protocol(calc, orc, tmp_path):
    """inputA.bin / inputB.bin -> mme_output.bin (mme_test_data_gen.cpp:561-573, mme_test_manager.cpp:586-611) equals the
    sequence run on tensors directly, byte for byte."""
    t = harness.load_tests(os.path.join(CONFIG_DIR, "basic_tests", "basic_fwd.json"))[0]
    assert harness.supported(t) is None
    types = harness.tensor_types(t)
    a_l, b_l, o_l = harness.operand_roles(t)
    values = harness.make_operand_values(t, seed=3)
    host = {letter: _quantise(orc, values[letter], *types[letter]) for letter in (a_l, b_l)}
    host[a_l].tofile(str(tmp_path / "inputA.bin"))
    host[b_l].tofile(str(tmp_path / "inputB.bin"))
    got = harness.run_ext_ref(t, str(tmp_path), calc)
    dumped = np.fromfile(str(tmp_path / "mme_output.bin"), dtype=got.dtype)
    tensors = {letter: MmeSimTensor(t[letter + "_sizes"], 5, types[letter][0], host[letter].copy(), types[letter][1], types[letter][2],
                                    t[letter + "_strides"]) for letter in (a_l, b_l)}
    want = harness.run_reference_sequence(calc, t, tensors).data()
    assert np.array_equal(dumped, want) and np.array_equal(got, want)
    assert np.any(want != 0)


def _dense_strides(sizes):
    out, acc = [], 1
    for v in sizes:
        out.append(acc)
        acc *= v
    return out


def _logical(tensor):
    """The tensor's elements as an array of shape sizes[::-1] (first dimension fastest), read through its strides."""
    data = tensor.data()
    data = data if isinstance(data, np.ndarray) else data.cpu().numpy()
    sizes, strides = tensor.getSizes(), tensor.getStrides()
    idx = np.zeros(sizes[::-1], np.int64)
    for d, (n, st) in enumerate(zip(sizes, strides)):
        shape = [1] * 5
        shape[4 - d] = n
        idx = idx + (np.arange(n, dtype=np.int64) * int(st)).reshape(shape)
    return data.ravel()[idx]


@pytest.mark.parametrize("t", _collect(large=True))
def test_reference_config_large(calc, orc, t):
    """The configurations whose contraction is too long for the CPU checker (up to 43 GFLOP): the GPU runs the whole test, the
    oracle the same test restricted to the first columns of the output (the leading entries of the output's first
    dimension), which it gets by reading a slice of the second operand through strides.  Every output element depends on
    its own column of that operand only, so the restriction changes nothing else."""
    types = harness.tensor_types(t)
    a_l, b_l, o_l = harness.operand_roles(t)
    values = harness.make_operand_values(t, seed=11)
    host = {}
    for letter in (a_l, b_l):
        dtype, bias, mode = types[letter]
        host[letter] = _quantise(orc, values[letter], dtype, bias, mode)
    out_dtype, out_bias, out_mode = types[o_l]
    mk = lambda tt, letter: MmeSimTensor(tt[letter + "_sizes"], 5, types[letter][0], host[letter].copy(), types[letter][1], types[letter][2],
                                         tt[letter + "_strides"])
    # the dimension of the second operand that runs along the output's first dimension
    op = t["operation"]
    b_dim = {abi.OP_AB: 0, abi.OP_ATB: 0, abi.OP_ABT: 1, abi.OP_ATBT: 1, abi.OP_FWD: 0, abi.OP_DEDX: 1, abi.OP_TRANSPOSED_DEDX: 0,
             abi.OP_DEDW: 0}[op]
    n_full = t[o_l + "_sizes"][0]
    assert t[b_l + "_sizes"][b_dim] == n_full
    budget = 1.5e8 if t["in_type"] in (abi.FP32, abi.TF32) else 6e8
    n_sub = int(max(1, min(n_full, n_full * budget // harness.contraction_flops(t))))
    ts = dict(t)
    ts[b_l + "_strides"] = t[b_l + "_strides"] or _dense_strides(t[b_l + "_sizes"])
    ts[b_l + "_sizes"] = [n_sub if d == b_dim else v for d, v in enumerate(t[b_l + "_sizes"])]
    ts[o_l + "_sizes"] = [n_sub] + list(t[o_l + "_sizes"][1:])
    ts[o_l + "_strides"] = None
    prev_full = None
    if t["reduction_op"] != abi.REDUCTION_NONE:
        span = max(st * sz for st, sz in zip(MmeSimTensor(t[o_l + "_sizes"], 5, out_dtype, None, out_bias, out_mode, t[o_l + "_strides"]).strides,
                                             t[o_l + "_sizes"]))
        prev_full = _quantise(orc, np.random.default_rng(5).uniform(-4, 4, span).astype(np.float32), out_dtype, out_bias, out_mode)
    lfsr = (np.arange(256, dtype=np.uint32) * 2654435761 + 12345).astype(np.uint32)
    from intel_gaudi3_software_amd import HipCalculator
    gpu = HipCalculator(lfsrNumRegs=256, lfsr=lfsr, polynomial=0xD35C) if t["uses_lfsr"] else calc
    p_full = None if prev_full is None else MmeSimTensor(t[o_l + "_sizes"], 5, out_dtype, prev_full.copy(), out_bias, out_mode, t[o_l + "_strides"])
    got_t = harness.run_reference_sequence(gpu, t, {a_l: mk(t, a_l), b_l: mk(t, b_l)}, p_full)
    if gpu is not calc:
        gpu.close()
    p_sub = None
    if prev_full is not None:
        full_view = MmeSimTensor(t[o_l + "_sizes"], 5, out_dtype, prev_full.copy(), out_bias, out_mode, t[o_l + "_strides"])
        p_sub = MmeSimTensor(ts[o_l + "_sizes"], 5, out_dtype, np.ascontiguousarray(_logical(full_view)[..., :n_sub]).ravel(), out_bias, out_mode)
    want_t = harness.run_reference_sequence(OracleCalculator(orc, lfsr, 0xD35C), ts, {a_l: mk(ts, a_l), b_l: mk(ts, b_l)}, p_sub)
    got_codes = np.ascontiguousarray(_logical(got_t)[..., :n_sub]).ravel()
    want_codes = np.ascontiguousarray(_logical(want_t)).ravel()
    got, want = (_decode(orc, c, out_dtype, out_bias, out_mode) for c in (got_codes, want_codes))
    fin = np.isfinite(want)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[~fin & ~np.isnan(want)], want[~fin & ~np.isnan(want)])
    dist = rel_frobenius(got[fin], want[fin])
    REPORT.append((t["name"], t["operation_name"], t["in_type"], out_dtype, bool(t["uses_lfsr"]), harness.cd_size(t), float(dist),
                   float(np.mean(got_codes == want_codes))))
    assert dist <= _like_for_like_tolerance(t, out_dtype), dist
    assert np.any(want != 0)
    if not t["uses_lfsr"]:
        if out_dtype != abi.FP32:
            assert np.mean(got_codes == want_codes) >= 0.8
        if not np.any(np.isnan(want)):
            sub_got = MmeSimTensor(ts[o_l + "_sizes"], 5, out_dtype, got_codes, out_bias, out_mode)
            assert harness.compare_with_reference(t, sub_got, want_t)


@pytest.mark.parametrize("in_type,in2_type,out_type,bias", [(abi.BF16, abi.BF16, abi.BF16, 0), (abi.FP8_143, abi.FP8_152, abi.FP8_143, 7),
                                                            (abi.FP32, abi.FP32, abi.FP32, 0)])
@pytest.mark.parametrize("op", [abi.OP_AB, abi.OP_ATBT])
def test_masked_bgemm_sequence(calc, orc, op, in_type, in2_type, out_type, bias):
    """runReference's masked batched GEMM (mme_test_manager.cpp:861-903): a second GEMM on the mask operands, added to the
    first one's accumulators by doMemoryWrite (reduction add), then the activation.  The sequence on the GPU library
    against the same sequence on the oracle, on the same operands; the reference's own acceptance rule must accept it."""
    t = dict(harness.load_tests(os.path.join(CONFIG_DIR, "basic_tests", "basic_ab.json"))[0])
    M, N, K, K2, nb = 200, 144, 136, 72, 3
    t["masked_bgemm"], t["operation"], t["operation_name"] = True, op, {abi.OP_AB: "ab", abi.OP_ATBT: "atbt"}[op]
    ta, tb = op == abi.OP_ATBT, op == abi.OP_ATBT
    t["x_sizes"], t["x_sizes2"] = ([M, K, nb, 1, 1], [M, K2, nb, 1, 1]) if ta else ([K, M, nb, 1, 1], [K2, M, nb, 1, 1])
    t["w_sizes"], t["w_sizes2"] = ([K, N, nb, 1, 1], [K2, N, nb, 1, 1]) if tb else ([N, K, nb, 1, 1], [N, K2, nb, 1, 1])
    t["y_sizes"] = [N, M, nb, 1, 1]
    for k in ("x_strides", "w_strides", "y_strides", "x_strides2", "w_strides2"):
        t[k] = None
    t["in_type"], t["in2_type"], t["out_type"] = in_type, in2_type, out_type
    t["fp8_bias_in"], t["fp8_bias_in2"], t["fp8_bias_out"] = bias, 15 if in2_type == abi.FP8_152 else bias, bias
    t["x_range"] = t["w_range"] = (-2.0, 2.0, 0.0, 0.5)
    assert harness.supported(t) is None
    types = harness.tensor_types(t)
    values = harness.make_operand_values(t, seed=13)
    host = {"x": _quantise(orc, values["x"], *types["x"]), "w": _quantise(orc, values["w"], *types["w"]),
            "x_aux": _quantise(orc, values["x_aux"], *types["x"]), "w_aux": _quantise(orc, values["w_aux"], *types["w"])}
    sizes = {"x": t["x_sizes"], "w": t["w_sizes"], "x_aux": t["x_sizes2"], "w_aux": t["w_sizes2"]}
    results = []
    for c in (calc, OracleCalculator(orc)):
        tensors = {k: MmeSimTensor(sizes[k], 5, types[k[0]][0], host[k].copy(), types[k[0]][1], types[k[0]][2]) for k in host}
        results.append(harness.run_reference_sequence(c, t, tensors))
    assert harness.compare_with_reference(t, results[0], results[1])
    out_dtype, out_bias, out_mode = types["y"]
    got, want = (_decode(orc, np.ascontiguousarray(r.data()), out_dtype, out_bias, out_mode) for r in results)
    assert np.isfinite(want).all() and np.any(want != 0)
    assert rel_frobenius(got, want) <= TOL[in_type]
    # the mask GEMM is in the result: without it the output is a different one
    plain = dict(t)
    plain["masked_bgemm"] = False
    tensors = {k: MmeSimTensor(sizes[k], 5, types[k][0], host[k].copy(), types[k][1], types[k][2]) for k in ("x", "w")}
    alone = _decode(orc, np.ascontiguousarray(harness.run_reference_sequence(calc, plain, tensors).data()), out_dtype, out_bias, out_mode)
    assert rel_frobenius(alone, want) > 0.05
