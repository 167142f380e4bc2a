"""Host logic of the harness seam (no GPU): the configuration reader against the reference's own configuration files."""
import glob
import os

from intel_gaudi3_software_amd import abi, harness

CONFIG_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "configs", "gaudi3")


def test_every_reference_config_parses():
    files = sorted(glob.glob(os.path.join(CONFIG_DIR, "*", "*.json")))
    assert len(files) >= 30
    total = 0
    for f in files:
        tests = harness.load_tests(f)
        assert tests, f
        total += len(tests)
        for t in tests:
            assert t["operation_name"]
            reason = harness.supported(t)
            assert reason is None or isinstance(reason, str)
    assert total >= 500


def test_cartesian_product_and_defaults():
    # numerics_fp8.json multiplies its tests over the listed types and modes (config_parser.cpp:286-315)
    tests = harness.load_tests(os.path.join(CONFIG_DIR, "numerics", "numerics_fp8.json"))
    combos = {(t["in_type"], t["in2_type"], t["out_type"]) for t in tests}
    assert (abi.FP8_143, abi.FP8_152, abi.FP8_143) in combos and (abi.FP8_152, abi.FP8_143, abi.FP8_152) in combos
    assert {t["inf_nan_out"] for t in tests} == {0, 1, 2}
    # vectors are single values, not factors of the product
    t = harness.load_tests(os.path.join(CONFIG_DIR, "basic_tests", "basic_ab.json"))
    assert len(t) == 1 and t[0]["x_sizes"] == [127, 400, 1, 1, 1] and t[0]["operation"] == abi.OP_AB
    assert t[0]["reduction_op"] == abi.REDUCTION_NONE and t[0]["rounding"] == 0 and not t[0]["clip"]
    assert harness.operand_roles(t[0]) == ("x", "w", "y")
    assert harness.contraction_flops(t[0]) == 2.0 * 1020 * 400 * 127


def test_operand_roles_follow_the_operation():
    tests = harness.load_tests(os.path.join(CONFIG_DIR, "basic_tests", "basic_dedx.json"))
    assert harness.operand_roles(tests[0]) == ("y", "w", "x")
    tests = harness.load_tests(os.path.join(CONFIG_DIR, "basic_tests", "basic_dedw.json"))
    assert harness.operand_roles(tests[0]) == ("x", "y", "w")


def test_dual_gemm_tests_are_two_contractions():
    tests = harness.load_tests(os.path.join(CONFIG_DIR, "basic_tests", "basic_dual_gemm.json"))
    assert len(tests) == 7 and all(t["dual_gemm"] and harness.supported(t) is None for t in tests)
    first, second = harness.gemms_of(tests[0])
    assert (first["x_sizes"], first["w_sizes"], first["y_sizes"]) == ([120, 112], [80, 120], [80, 112])
    assert (second["x_sizes"], second["w_sizes"], second["y_sizes"]) == ([128, 88], [90, 128], [90, 88])
    assert harness.cd_size(first) == 120 and harness.cd_size(second) == 128
    assert harness.gemms_of(first) == [first]
