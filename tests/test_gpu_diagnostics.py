"""The diagnostics of the C ABI: the clock probe of the large-tile kernels and the bare matrix-instruction rate."""
import numpy as np
import pytest
import torch

from intel_gaudi3_software_amd import HipCalculator, MmeSimTensor, abi

pytestmark = pytest.mark.gpu


def test_clock_probe_reports_the_workgroups_of_a_large_tile_gemm():
    calc = HipCalculator()
    n = 1024
    rng = np.random.default_rng(11)
    a = torch.from_numpy(rng.integers(0x20, 0x50, n * n, dtype=np.uint8)).cuda()
    b = torch.from_numpy(rng.integers(0x20, 0x50, n * n, dtype=np.uint8)).cuda()
    out = torch.zeros(n * n, dtype=torch.float32, device="cuda")
    A, B, Y = MmeSimTensor([n, n], 2, abi.FP8_143, a, 7), MmeSimTensor([n, n], 2, abi.FP8_143, b, 7), MmeSimTensor([n, n], 2, abi.FP32, out)
    with pytest.raises(RuntimeError):
        calc.readClockProbe()  # switched off: an error, not zeros
    calc.doBatchGemm(Y, A, B, abi.OP_ABT)
    calc.synchronize()
    want = out.clone()
    calc.clockProbe(True)
    assert calc.readClockProbe()["workgroups"] == 0  # nothing has run since it was switched on
    calc.doBatchGemm(Y, A, B, abi.OP_ABT)
    r = calc.readClockProbe()
    tiles = (n // 256) ** 2
    assert r["workgroups"] >= tiles and r["workgroups"] % tiles == 0  # one workgroup per 256 x 256 tile (and k-slice, if any)
    assert 300.0 < r["shader_mhz"] < 3000.0
    assert 0.0 < r["workgroup_us_mean"] <= r["workgroup_us_max"] < 1e4
    assert torch.equal(out, want)  # the stamps do not touch the result
    assert calc.readClockProbe()["workgroups"] == 0  # a read clears the cells
    calc.clockProbe(False)
    calc.doBatchGemm(Y, A, B, abi.OP_ABT)
    calc.synchronize()
    assert torch.equal(out, want)
    calc.close()


@pytest.mark.parametrize("dtype", [abi.FP8_143, abi.BF16])
def test_matrix_core_rate_is_higher_on_zero_operands(dtype):
    calc = HipCalculator()
    zero_tf, zero_mhz = calc.matrixCoreRate(dtype, False, iters=1024, launches=4)
    rand_tf, rand_mhz = calc.matrixCoreRate(dtype, True, iters=1024, launches=4)
    peak = 5000.0 if dtype == abi.FP8_143 else 2500.0
    assert 0.2 * peak < rand_tf <= 1.05 * peak and 0.2 * peak < zero_tf <= 1.05 * peak
    assert zero_tf >= 0.95 * rand_tf  # operands that toggle the multipliers never run faster
    assert 300.0 < rand_mhz < 3000.0 and 300.0 < zero_mhz < 3000.0
    with pytest.raises(RuntimeError):
        calc.matrixCoreRate(abi.FP32, False)
    calc.close()
