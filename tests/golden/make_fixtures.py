"""Collect the known-answer fixtures that the reference's own tests hold for the
Gemm / Conv / ConvTranspose / MaxPool / AveragePool path into tests/golden/.

Run in the authoring container only (it reads /root/reference, which does not exist
on the GPU box):   python tests/golden/make_fixtures.py

What is written:
  tests/golden/onnx/<name>.onnx      byte copies of the reference's binary test models
                                     (data files: graph + weights)
  tests/golden/expected.json         the expected output arrays of the reference's
                                     <name>.ref.hxx headers (numbers only) together with
                                     the input each test feeds (ones / iota / literal list,
                                     from TestCustomModelsFromONNX.cxx:330-349,372-391,
                                     693-712,860-967,992-1085,1086-1114,2047-2152); for the Einsum models
                                     the literal inputs and outputs of the tests themselves
                                     (TestCustomModelsFromONNX.cxx:3028-3103)
"""
import json
import os
import re
import shutil

REF = "/root/reference/src/SOFIE_core/test/input_models"
HERE = os.path.dirname(os.path.abspath(__file__))

# name -> (input kind, input shape, array name inside the ref header)
CASES = {
    "Linear_16": ("ones", [16, 100], "all_ones"),
    "Linear_32": ("ones", [32, 100], "all_ones"),
    "Linear_64": ("ones", [64, 100], "all_ones"),
    "ConvWithPadding": ("iota", [1, 1, 5, 5], "all_ones"),
    "ConvWithoutPadding": ("iota", [1, 1, 5, 5], "all_ones"),
    "ConvWithAutopadSameLower": ("iota", [1, 1, 5, 5], "all_ones"),
    "ConvWithStridesPadding": ("iota", [1, 1, 7, 5], "all_ones"),
    "ConvWithStridesNoPadding": ("iota", [1, 1, 7, 5], "all_ones"),
    "ConvWithAsymmetricPadding": ("iota", [1, 1, 7, 5], "all_ones"),
    "MaxPool1d": ("literal", [1, 6, 10], "output"),
    "MaxPool2d": ("literal", [1, 1, 5, 10], "output"),
    "MaxPool3d": ("literal", [1, 1, 3, 3, 3], "output"),
    "AvgPool": ("literal", [1, 1, 5, 10], "output"),
    "ConvTranspose1d": ("iota", [1, 1, 3], "output"),
    "ConvTranspose2d": ("iota", [1, 1, 3, 3], "output"),
    "ConvTransposeBias2d": ("iota", [1, 1, 3, 3], "output"),
    "ConvTransposeBias2dBatched": ("iota", [2, 1, 3, 3], "output"),
}

# Input of the reference's MaxPool2d test (TestCustomModelsFromONNX.cxx:1027-1038).
MAXPOOL2D_INPUT = [
    0.6266, 0.1656, 0.2753, -0.4558, -1.4592, 0.9285, -1.3410, 1.3223, -0.5936, -1.3648,
    -0.2989, 0.5901, -0.8845, -0.0433, 0.8314, -1.7159, -0.5765, 0.8678, 1.0257, 0.7847,
    -0.3421, -1.2364, -0.5805, 0.4421, 1.2184, 0.5043, 1.6823, -1.0483, -2.2798, -1.8927,
    0.7716, 0.0405, 0.3121, -0.3011, -0.3266, -1.9660, 1.0837, 0.2317, 0.9084, -0.3285,
    -0.9398, -0.2065, -0.9499, -0.9739, -0.1288, -0.1375, -1.2612, 0.8810, 0.8506, 0.4455,
]


# Input of the reference's MaxPool1d test (TestCustomModelsFromONNX.cxx:996-1007).
MAXPOOL1D_INPUT = [
    0.0907, 0.1029, 0.8143, 1.4497, -0.7785, 0.3825, -0.3764, 1.5785, -0.0835, 0.1622,
    1.5867, 0.9823, -0.8821, 0.4439, -0.1378, -0.2273, -0.0198, -2.0230, 0.0905, 0.6674,
    -1.4290, -1.3100, -0.9439, -0.0833, -0.1919, 0.6886, 0.9389, -1.2914, -1.3584, -2.0341,
    -0.3269, 0.1704, 1.1776, 1.3972, -1.8874, -1.5334, 1.1541, 0.3011, 0.6569, -2.3504,
    0.4033, 0.1142, 2.2846, -1.3948, -0.8573, 0.5756, -1.0864, 0.2283, 0.8947, 1.7627,
    -0.1657, 0.0649, -1.6066, 0.4162, -1.1525, -0.8184, 1.1324, -1.1086, 0.1061, 1.0071,
]

# Input of the reference's MaxPool3d test (TestCustomModelsFromONNX.cxx:1058-1070).
MAXPOOL3D_INPUT = [
    -2.6496, 1.0476, -0.5153, 0.3771, 0.4129, -0.3077, -0.8717, -0.8040, -0.3525,
    -0.1765, -0.3364, 0.8737, -0.2381, -0.8297, 0.4666, 0.6984, -0.6760, 0.6298,
    1.3833, 0.1101, 0.2039, -0.5477, 0.2341, 0.9181, 0.3842, 0.2428, 1.7924,
]


# Input of the reference's AvgPool test (TestCustomModelsFromONNX.cxx:1090-1101).
AVGPOOL_INPUT = [
    0.4764, -0.1976, 1.6506, -0.2421, 0.6412, 1.9985, 0.3938, 0.1347, 0.2204, -0.7503,
    0.2139, 0.7285, -0.0210, -0.4585, -1.5333, -0.4772, 0.5560, 0.6323, -2.5372, 1.4906,
    -1.1062, -0.9703, 0.2366, -0.9184, 0.3014, 0.7985, -0.6841, -2.2854, -2.7728, -1.2806,
    -1.0947, -0.5990, -0.3033, -1.9042, -0.5403, 0.2332, 0.9215, -0.1549, 0.0557, -0.5567,
    -1.4971, 0.5386, -0.2922, 0.4860, -0.3973, -0.4624, 0.4514, 0.2385, 0.3783, -1.0500,
]


# The reference's Einsum tests carry inputs and answers as literals (TestCustomModelsFromONNX.cxx:3028-3103).
EINSUM_CASES = {
    "Einsum_matmul": ([[1, 2, 3, 4], [5, 6, 7, 8]], [19, 22, 43, 50]),
    "Einsum_dotprod": ([[1, 2, 3], [5, 6, 7]], [5 + 12 + 21]),
    "Einsum_3": ([[1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12], [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12]],
                 [66, 87, 108, 498, 555, 612]),
    "Einsum_4": ([[1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12], [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16, 17, 18]],
                 [14, 32, 50, 32, 77, 122, 266, 338, 410, 365, 464, 563]),
}


def numbers_of(header_text, array):
    m = re.search(r"float\s+%s\s*\[\s*\]\s*=\s*\{(.*?)\}" % re.escape(array), header_text, re.S)
    body = re.sub(r"//[^\n]*", "", m.group(1))
    return [float(t.rstrip("f")) for t in re.findall(r"[-+]?(?:\d+\.?\d*|\.\d+)(?:[eE][-+]?\d+)?f?", body)]


def main():
    os.makedirs(os.path.join(HERE, "onnx"), exist_ok=True)
    expected = {}
    for name, (kind, shape, arr) in CASES.items():
        shutil.copyfile(os.path.join(REF, name + ".onnx"), os.path.join(HERE, "onnx", name + ".onnx"))
        os.chmod(os.path.join(HERE, "onnx", name + ".onnx"), 0o644)
        with open(os.path.join(REF, "references", name + ".ref.hxx")) as f:
            vals = numbers_of(f.read(), arr)
        entry = {"input_kind": kind, "input_shape": shape, "expected": vals}
        if kind == "literal":
            entry["input"] = {"AvgPool": AVGPOOL_INPUT, "MaxPool1d": MAXPOOL1D_INPUT, "MaxPool2d": MAXPOOL2D_INPUT,
                              "MaxPool3d": MAXPOOL3D_INPUT}[name]
        expected[name] = entry
    for name, (inputs, answer) in EINSUM_CASES.items():
        shutil.copyfile(os.path.join(REF, name + ".onnx"), os.path.join(HERE, "onnx", name + ".onnx"))
        os.chmod(os.path.join(HERE, "onnx", name + ".onnx"), 0o644)
        # one literal list per graph input, in the order of the graph's inputs; shapes come from the model file
        expected[name] = {"input_kind": "literals", "inputs": [[float(v) for v in x] for x in inputs],
                          "expected": [float(v) for v in answer]}
    with open(os.path.join(HERE, "expected.json"), "w") as f:
        json.dump(expected, f, indent=0)
    print({k: len(v["expected"]) for k, v in expected.items()})


if __name__ == "__main__":
    main()
