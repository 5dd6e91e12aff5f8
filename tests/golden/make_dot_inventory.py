#!/usr/bin/env python3
"""Extracts the Dot known-answer vectors that the reference's own kernel tests hold
(test/nnfusion/inventory/dot.cpp in the nnfusion tree: shapes :26-176, inputs :182-301, expected
outputs :305-402) into tests/golden/dot_inventory.json.  The reference file is read as text; only the
numbers (shapes, input values, expected values) are kept.  Run in the build container, where the tree
is mounted:   python tests/golden/make_dot_inventory.py [/root/reference]
"""
import json
import os
import re
import sys

ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
src = open(os.path.join(ref, "test/nnfusion/inventory/dot.cpp")).read()


def section(name):
    start = src.index(name)
    end = src.index("default:", start)
    return src[start:end]


def cases(text):
    parts = re.split(r"case\s+(\d+)\s*:", text)
    return {int(parts[i]): parts[i + 1] for i in range(1, len(parts), 2)}


def numbers(s):
    return [float(x) for x in re.findall(r"-?\d+(?:\.\d+)?", s)]


create = cases(section("create_object<op::Dot, float>"))
inputs = cases(section("generate_input<op::Dot, float>"))
outputs = cases(section("generate_output<op::Dot, float>"))

out = []
for c in sorted(create):
    shapes = re.findall(r"Shape\s+(\w+)\s*\{([^}]*)\}", create[c])
    named = {name: [int(v) for v in re.findall(r"\d+", body)] for name, body in shapes}
    if "shape" in named:
        shape_a = shape_b = named["shape"]
    else:
        shape_a, shape_b = named["shape_a"], named["shape_b"]
    dot_args = re.search(r"make_shared<op::Dot>\(([^)]*)\)", create[c]).group(1).strip()
    assert dot_args == "", "a case with explicit reduction axes appeared: extend this script"
    def vec(text, name):
        # either  vector<float> a = vector<float>{...};  or  vector<float> a_data{...};
        m = re.search(r"vector<float>\s+%s\s*=\s*vector<float>\s*\{([^}]*)\}" % name, text)
        if m is None:
            m = re.search(r"vector<float>\s+%s_data\s*\{([^}]*)\}" % name, text)
        return numbers(m.group(1))

    a, b, r = vec(inputs[c], "a"), vec(inputs[c], "b"), vec(outputs[c], "result")
    out.append({"case": c, "shape_a": shape_a, "shape_b": shape_b, "a": a, "b": b, "expected": r})

dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dot_inventory.json")
with open(dst, "w") as f:
    json.dump({"source": "test/nnfusion/inventory/dot.cpp (nnfusion v0.4.0)", "cases": out}, f, indent=1)
print(f"wrote {len(out)} cases to {dst}")

# ---- the ONNX Gemm vector the reference's frontend tests hold (test/nnfusion/frontend/onnx_import.cpp:823-871):
# a (4,3), b (5,4), c (1,5) -> (3,5) with transA = transB = 1; the model file (test/models/onnx/gemm_op.onnx)
# carries alpha = 0.25 and beta = 0.35 (the ONNX "gemm_all_attributes" node test).
osrc = open(os.path.join(ref, "test/nnfusion/frontend/onnx_import.cpp")).read()
blk = osrc[osrc.index("TEST(nnfusion_onnx_import, gemm_op)"):]
blk = blk[:blk.index("EXPECT_EQ")]
vecs = [numbers(v) for v in re.findall(r"\{\{?([0-9.,\s-]+)\}", blk)]
vecs = [v for v in vecs if len(v) >= 5]
assert [len(v) for v in vecs] == [12, 20, 5, 15], [len(v) for v in vecs]
gemm = {"source": "test/nnfusion/frontend/onnx_import.cpp:823-871", "a_shape": [4, 3], "b_shape": [5, 4],
        "c_shape": [1, 5], "trans_a": 1, "trans_b": 1, "alpha": 0.25, "beta": 0.35,
        "a": vecs[0], "b": vecs[1], "c": vecs[2], "expected": vecs[3]}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "onnx_gemm_op.json"), "w") as f:
    json.dump(gemm, f, indent=1)
print("wrote onnx_gemm_op.json")
