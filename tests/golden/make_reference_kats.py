"""Writes reference_kats.json: the known-answer vectors held by the reference's own tests for
the quantized Dense / Gather path, transcribed as data (inputs and expected outputs).

Sources (gomlx/gomlx):
  ml/nn/quantized_dense_test.go:272-334   Q8_0 basic / with_bias / batch
  ml/nn/quantized_dense_test.go:340-401   Q4_0 basic / with_silu
  ml/nn/quantized_dense_test.go:406-452   IQ4_NL basic
  ml/nn/quantized_gather_test.go:17-74    Q8_0 gather basic / single
  ml/nn/quantized_gather_test.go:78-121   Q4_0 gather
  ml/nn/quantized_gather_test.go:125-169  IQ4_NL gather
  ml/layers/activation/activation_test.go:17-112  Relu, Swish, Gelu (exact), GeluApproximate, HardSwish on
                                          x = [0, -1, 2, -3, 4, -5, 6]; tolerances as in the tests
                                          (xslices.Epsilon is defined outside the repository: 1e-4 is used here)
  ml/layers/norm/rmsnorm_test.go:16-45    RMSNorm over the last two axes of a [2, 3, 2] input (gain = ones),
                                          stored flattened: rows of 6 values

Nothing from the reference is imported or executed; run `python make_reference_kats.py`
to regenerate the JSON next to this script.
"""
import json
import os

Q4_0, Q8_0, IQ4_NL = 2, 8, 20
NONE, SILU = 0, 3


def q8_row(scale_hi, ones):
    row = [0] * 34
    row[0], row[1] = 0x00, scale_hi
    for i in ones:
        row[2 + i] = 1
    return row


def q4_row(scale_hi, byte_with_9):
    row = [0x88] * 18
    row[0], row[1] = 0x00, scale_hi
    row[2 + byte_with_9] = 0x89
    return row


ACT_X = [0, -1, 2, -3, 4, -5, 6]
x_basic = [1.0, 1.0] + [0.0] * 30
x_half = [0.5] + [0.0] * 31
q8_w = [q8_row(0x40, [0]), q8_row(0x42, [1])]
q4_w = [q4_row(0x40, 0), q4_row(0x42, 1)]
iq_w = [q4_row(0x3C, 0), q4_row(0x40, 1)]


def unit(values):
    v = [0.0] * 32
    for i, a in values.items():
        v[i] = a
    return v


kats = {
    "fp16": [  # little-endian byte pairs -> value
        {"bytes": [0x00, 0x40], "value": 2.0},
        {"bytes": [0x00, 0x42], "value": 3.0},
        {"bytes": [0x00, 0x3C], "value": 1.0},
    ],
    "dense": [
        {"name": "q8_0_basic", "type": Q8_0, "w": q8_w, "x": [x_basic], "bias": None, "act": NONE,
         "want": [[2.0, 3.0]], "tol": 1e-4},
        {"name": "q8_0_with_bias", "type": Q8_0, "w": q8_w, "x": [x_basic], "bias": [0.5, -0.5], "act": NONE,
         "want": [[2.5, 2.5]], "tol": 1e-4},
        {"name": "q8_0_batch", "type": Q8_0, "w": q8_w, "x": [x_basic, x_half], "bias": None, "act": NONE,
         "want": [[2.0, 3.0], [1.0, 0.0]], "tol": 1e-4},
        {"name": "q4_0_basic", "type": Q4_0, "w": q4_w, "x": [x_basic], "bias": None, "act": NONE,
         "want": [[2.0, 3.0]], "tol": 1e-4},
        {"name": "q4_0_with_silu", "type": Q4_0, "w": q4_w, "x": [x_basic], "bias": None, "act": SILU,
         "want": [[1.7616, 2.8577]], "tol": 1e-3},
        {"name": "iq4_nl_basic", "type": IQ4_NL, "w": iq_w, "x": [x_basic], "bias": None, "act": NONE,
         "want": [[14.0, 28.0]], "tol": 1e-4},
    ],
    # act = compute.ActivationType the type maps to (activation.go:58-75): GeluApproximate also maps to Gelu (exact)
    "activation": [
        {"name": "relu", "act": 2, "x": ACT_X, "want": [0, 0, 2, 0, 4, 0, 6], "tol": 1e-4},
        {"name": "swish", "act": 3, "x": ACT_X,
         "want": [0, -0.26894143, 1.7615942, -0.14227763, 3.928055, -0.03346425, 5.9851646], "tol": 1e-4},
        {"name": "gelu_exact", "act": 1, "x": ACT_X,
         "want": [0, -0.15865526, 1.9544997, -4.0496886e-03, 3.9998736, -1.3411045e-06, 6], "tol": 1e-5},
        {"name": "gelu_approximate_through_the_backend_enum", "act": 1, "x": ACT_X,
         "want": [0, -0.15880796, 1.9545977, -3.6375225e-03, 3.9999294, 0, 6], "tol": 0.01},
        {"name": "hard_swish", "act": 4, "x": ACT_X, "want": [0, -0.33333334, 1.6666666, 0, 4, 0, 6], "tol": 1e-4},
    ],
    "rmsnorm": [
        {"name": "rmsnorm_two_axes", "x": [[3, 4, 5, 6, 7, 8], [6, 8, 10, 12, 14, 16]], "eps": 1e-6,
         "want": [[0.52091914, 0.6945589, 0.86819863, 1.0418383, 1.2154781, 1.3891178]] * 2, "tol": 1e-3},
    ],
    "gather": [
        {"name": "q8_0_gather_basic", "type": Q8_0,
         "table": [q8_row(0x40, [0]), q8_row(0x42, [1]), q8_row(0x3C, [0, 1])],
         "indices": [[2], [0]], "want": [unit({0: 1.0, 1: 1.0}), unit({0: 2.0})], "tol": 1e-4},
        {"name": "q8_0_gather_single", "type": Q8_0,
         "table": [q8_row(0x40, [0]), q8_row(0x42, [1]), q8_row(0x3C, [0, 1])],
         "indices": [[1]], "want": [unit({1: 3.0})], "tol": 1e-4},
        {"name": "q4_0_gather_basic", "type": Q4_0, "table": q4_w,
         "indices": [[1], [0]], "want": [unit({1: 3.0}), unit({0: 2.0})], "tol": 1e-4},
        {"name": "iq4_nl_gather_basic", "type": IQ4_NL, "table": iq_w,
         "indices": [[0]], "want": [[13.0] + [1.0] * 31], "tol": 1e-4},
    ],
}

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_kats.json"), "w") as f:
    json.dump(kats, f, indent=1)
print("wrote reference_kats.json")
