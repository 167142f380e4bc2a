"""Writes tests/golden/contraction_forms.json: for every distinct contraction of the reference's Gaudi3 test configurations
(tests/golden/configs/gaudi3, read like tests/test_gpu_reference_configs.py reads them) the kernel form that the library
launched for it on an MI355X, as mme_hip_last_contraction_form reported it after the call.  Needs a GPU:

    python tests/golden/gen_contraction_forms.py

tests/test_planner.py holds the planner (mme_hip_plan_*, no GPU) to these records."""
import glob
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from intel_gaudi3_software_amd import abi, harness  # noqa: E402

CONFIG_DIR = os.path.join(ROOT, "tests", "golden", "configs", "gaudi3")
OUT = os.path.join(ROOT, "tests", "golden", "contraction_forms.json")


def cases():
    """(file name, test) for every distinct contraction the calculator path covers, in a fixed order."""
    out, seen = [], set()
    for path in sorted(glob.glob(os.path.join(CONFIG_DIR, "*", "*.json"))):
        seeds = (1, 2, 3, 4, 5, 6, 7, 8) if os.path.basename(os.path.dirname(path)) == "random_tests" else (7,)
        for sd in seeds:
            for test in harness.load_tests(path, seed=sd):
                if test["masked_bgemm"] or harness.supported(test) is not None:
                    continue
                if any(v <= 0 for v in test["x_sizes"] + test["w_sizes"] + test["y_sizes"]):
                    continue
                for t in harness.gemms_of(test):
                    key = (t["operation"], t["in_type"], t["in2_type"], tuple(t["x_sizes"]), tuple(t["w_sizes"]), tuple(t["y_sizes"]),
                           tuple(t["x_strides"] or ()), tuple(t["w_strides"] or ()), tuple(t["y_strides"] or ()), tuple(t["padding"]),
                           tuple(t["conv_strides"]), tuple(t["dilation"]))
                    if key in seen:
                        continue
                    seen.add(key)
                    out.append((os.path.basename(path), t))
    return out


def record(name, t, form):
    return {"file": name, "op": t["operation_name"], "in_type": t["in_type"], "in2_type": t["in2_type"], "x": t["x_sizes"], "w": t["w_sizes"],
            "y": t["y_sizes"], "x_strides": t["x_strides"], "w_strides": t["w_strides"], "y_strides": t["y_strides"], "padding": t["padding"],
            "conv_strides": t["conv_strides"], "dilation": t["dilation"], "flops": harness.contraction_flops(t), "form": form}


def main():
    import torch
    from intel_gaudi3_software_amd import ConvolutionParams, HipCalculator, MmeSimTensor
    calc = HipCalculator()
    rows = []
    for name, t in cases():
        types = harness.tensor_types(t)
        a_l, b_l, o_l = harness.operand_roles(t)
        tens = {}
        for letter in (a_l, b_l):
            dt, bias, mode = types[letter]
            n = harness._span(t[letter + "_sizes"], t[letter + "_strides"])
            td = {abi.FP32: torch.float32, abi.TF32: torch.float32, abi.BF16: torch.int16, abi.FP16: torch.int16, abi.UFP16: torch.int16}.get(dt, torch.uint8)
            tens[letter] = MmeSimTensor(t[letter + "_sizes"], 5, dt, torch.zeros(n, dtype=td, device="cuda"), bias, mode, t[letter + "_strides"])
        n = harness._span(t[o_l + "_sizes"], t[o_l + "_strides"])
        acc = MmeSimTensor(t[o_l + "_sizes"], 5, abi.FP32, torch.zeros(n, dtype=torch.float32, device="cuda"), 0, 0, t[o_l + "_strides"])
        if t["operation"] in harness._CONV_OPS:
            cp = ConvolutionParams(3, t["padding"] + [0], t["conv_strides"] + [1], t["dilation"] + [1])
            calc.doConvolution(acc, tens.get("x", acc), tens.get("w", acc), tens.get("y", acc), cp, t["operation"], 0, 0, 0)
        else:
            calc.doBatchGemm(acc, tens[a_l], tens[b_l], t["operation"], 0, 0, 0)
        calc.synchronize()
        rows.append(record(name, t, calc.lastContractionForm()))
    with open(OUT, "w") as f:
        json.dump(rows, f, indent=0)
    print("%d cases, %d on a large-tile kernel" % (len(rows), sum(1 for r in rows if r["form"]["large_tile"] == 1)))


if __name__ == "__main__":
    main()
