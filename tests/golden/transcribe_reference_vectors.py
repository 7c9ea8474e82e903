"""Transcribes the input/expected-output constants that the reference's own
tests hold for this path into small JSON fixtures (data only).

Run once in a container that has the reference checkout; the fixtures it writes
are committed beside it and the tests read only those.

    python tests/golden/transcribe_reference_vectors.py [/root/reference]
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))
NUM = r"[-+]?(?:\d+\.\d*(?:[eE][-+]?\d+)?|\d+(?:[eE][-+]?\d+)?)"


def read(rel):
    with open(os.path.join(REF, rel)) as f:
        return f.read()


def dense_literals(text):
    """Every `dense<[...]>` literal, flattened to a list of floats."""
    out = []
    for m in re.finditer(r"dense<\s*(\[.*?\])\s*>", text, re.S):
        out.append([float(x) for x in re.findall(NUM, m.group(1))])
    return out


def check_rows(text):
    """Numbers on `CHECK-NEXT: [..]` lines, one list per line."""
    rows = []
    for line in text.splitlines():
        m = re.search(r"CHECK(?:-NEXT)?:\s*\[(.*?)\]?\s*$", line)
        if m and re.search(r"\d", m.group(1)):
            rows.append([float(x) for x in re.findall(NUM, m.group(1))])
    return rows


def check_scalars(text):
    vals = []
    for line in text.splitlines():
        m = re.match(r"\s*//\s*CHECK:\s+(" + NUM + r")\s*$", line)
        if m:
            vals.append(float(m.group(1)))
    return vals


fx = {}

t = read("test/PlaidML/OpTest.Relu.mlir")
fx["relu_olt_f32_4x5"] = {"source": "test/PlaidML/OpTest.Relu.mlir:17,41-62", "shape": [4, 5],
                          "input": dense_literals(t)[0], "expected": check_scalars(t)}
t = read("test/PlaidML/OpTest.Relu_BF16.mlir")
fx["relu_olt_bf16_4x5"] = {"source": "test/PlaidML/OpTest.Relu_BF16.mlir:17,43-64", "shape": [4, 5],
                           "input": dense_literals(t)[0], "expected": check_scalars(t)}
t = read("test/SPIRV/OpTest.Relu_FLOAT32.mlir")
d = dense_literals(t)
fx["relu_f32_4x5_spirv"] = {"source": "test/SPIRV/OpTest.Relu_FLOAT32.mlir:12-23", "shape": [4, 5],
                            "input": d[0], "expected": d[1]}

t = read("test/PlaidML/OpTest.Softmax.mlir")
fx["softmax_f32_10x20"] = {"source": "test/PlaidML/OpTest.Softmax.mlir:17-26,98-109", "shape": [10, 20],
                           "input": dense_literals(t)[0],
                           "expected": [v for row in check_rows(t) for v in row]}
t = read("test/SPIRV/OpTest.Softmax_FLOAT32.mlir")
d = dense_literals(t)
fx["softmax_f32_10x20_spirv"] = {"source": "test/SPIRV/OpTest.Softmax_FLOAT32.mlir:12-35", "shape": [10, 20],
                                 "input": d[0], "expected": d[1]}

t = read("test/PlaidML/OpTest.Transpose.mlir")
fx["transpose_f32_10x20"] = {"source": "test/PlaidML/OpTest.Transpose.mlir:27-61", "shape": [10, 20],
                             "input": dense_literals(t)[0],
                             "expected": [v for row in check_rows(t) for v in row]}
t = read("test/PlaidML/OpTest.Transpose_BF16.mlir")
fx["transpose_bf16_10x20"] = {"source": "test/PlaidML/OpTest.Transpose_BF16.mlir:27-61", "shape": [10, 20],
                              "input": dense_literals(t)[0],
                              "expected": [v for row in check_rows(t) for v in row]}

t = read("test/PlaidML/OpTest.Sum.mlir")
fx["sum_f32_10x20"] = {"source": "test/PlaidML/OpTest.Sum.mlir:28-43", "shape": [10, 20],
                       "input": dense_literals(t)[0], "expected": check_rows(t)[0]}

t = read("test/PlaidML/OpTest.GEMM_FLOAT32.mlir")
d = dense_literals(t)
fx["gemm_f32_3x3"] = {"source": "test/PlaidML/OpTest.GEMM_FLOAT32.mlir:17-32", "A": d[0], "B": d[1], "C0": d[2],
                      "expected": [v for row in check_rows(t)[:3] for v in row]}
for key, rel in (("gemm_f16_acc_f32_3x3", "test/SPIRV/OpTest.GEMM_F16_ACC_F32.mlir"),
                 ("gemm_bf16_acc_f32_3x3", "test/SPIRV/OpTest.GEMM_BF16_ACC_F32.mlir")):
    t = read(rel)
    d = dense_literals(t)
    # order in the file: C0 is dense<1.0> (a splat, not matched), then B, A, expected
    fx[key] = {"source": rel + ":11-15", "C0": [1.0] * 9, "B": d[0], "A": d[1], "expected": d[2]}

fx["dot_f16_acc_f32_8x16x32"] = {"source": "test/PlaidML/CppEdsl.DotF16_AccF32.mlir:50-57",
                                 "A_fill": 1.0, "B_fill": 2.0, "M": 8, "K": 16, "N": 32, "expected_fill": 32.0}
fx["wg_reduction_rows"] = {"source": "test/Integration/Dialect/XeGPU/WG/reduction_2D_1D_cross_sg_cross_lane.mlir:92-103,115",
                           "rows": 8, "cols": 256, "row_value_is_row_index": True,
                           "expected": [256.0 * i for i in range(8)]}

with open(os.path.join(OUT, "reference_vectors.json"), "w") as f:
    json.dump(fx, f, indent=1)
for k, v in fx.items():
    print(k, {kk: (len(vv) if isinstance(vv, list) else vv) for kk, vv in v.items() if kk != "source"})
