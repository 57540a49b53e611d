#!/usr/bin/env python3
"""Extracts known-answer vectors from the reference's own Go test files into
small JSON fixtures.  The Go files are read as TEXT (nothing is compiled, run or
imported); only numeric literals - inputs and expected outputs - are kept.

    python tests/golden/extract_fixtures.py [/root/reference]

Writes next to this script:
    maxpool_asym.json  nn_test.go TestMaxPool2D_asymmetricPadding (float32 case)
    leaky_relu.json    nn_test.go TestLeakyRelu (float32 case)
    conv.json          known_issues_test.go TestIssue233_F32, blas_test.go TestUse
    softmax_do.json    op_softmax_test.go testCasesSoftMaxDo
    binop.json         op_math_test.go binOpTests (operands, result, the two derivatives)
    batchnorm.json     nn_amd64_test.go bnAllCases (float32 cases)
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.dirname(os.path.abspath(__file__))

LIT = re.compile(r"\[\]float(32|64)\{([^{}]*)\}", re.S)


def read(name):
    with open(os.path.join(REF, name), encoding="utf-8") as f:
        return f.read()


def func_body(text, header):
    """Text from `header` to the next top-level `func ` / `var ` declaration."""
    i = text.index(header)
    m = re.search(r"\n(func |var )", text[i + len(header):])
    return text[i:i + len(header) + (m.start() if m else len(text))]


def nums(s):
    return [float(t) for t in re.split(r"[,\s]+", s.strip()) if t]


def literals(text):
    return [(int(m.group(1)), nums(m.group(2))) for m in LIT.finditer(text)]


def dump(name, obj):
    with open(os.path.join(OUT, name), "w") as f:
        json.dump(obj, f, separators=(",", ":"))
    print("wrote", name, os.path.getsize(os.path.join(OUT, name)), "bytes")


def maxpool():
    body = func_body(read("nn_test.go"), "func TestMaxPool2D_asymmetricPadding")
    lits = literals(body)
    (b0, x), (b1, y) = lits[0], lits[1]
    assert b0 == 32 and b1 == 32 and len(x) == 3072 and len(y) == 3072
    dump("maxpool_asym.json", {
        "source": "nn_test.go:91-138 TestMaxPool2D_asymmetricPadding",
        "shape": [1, 3, 32, 32], "kernel": [2, 2], "pad": [1, 0, 1, 0], "stride": [1, 1],
        "x": x, "y": y})


def leaky():
    body = func_body(read("nn_test.go"), "func TestLeakyRelu")
    lits = literals(body)
    (b0, x), (b1, y) = lits[0], lits[1]
    assert b0 == 32 and b1 == 32 and len(x) == 60 and len(y) == 60
    dump("leaky_relu.json", {"source": "nn_test.go:538-588 TestLeakyRelu", "alpha": 0.1,
                             "shape": [3, 4, 5], "x": x, "y": y, "tolerance": 1e-6})


def conv():
    b1 = literals(func_body(read("known_issues_test.go"), "func TestIssue233_F32"))
    b2 = literals(func_body(read("blas_test.go"), "func TestUse"))
    assert len(b1[0][1]) == 25 and len(b1[1][1]) == 9 and len(b1[2][1]) == 25
    assert len(b2[0][1]) == 35 and len(b2[1][1]) == 9
    dump("conv.json", [
        {"source": "known_issues_test.go:160-199 TestIssue233_F32", "x_shape": [1, 1, 5, 5],
         "w_shape": [1, 1, 3, 3], "pad": [1, 1], "stride": [1, 1], "dilation": [1, 1],
         "x": b1[0][1], "w": b1[1][1], "y": b1[2][1], "y_shape": [1, 1, 5, 5]},
        {"source": "blas_test.go:426-460 TestUse; ops/nn/conv_test.go:13-37 ExampleConv2d",
         "x_shape": [1, 1, 7, 5], "w_shape": [1, 1, 3, 3], "pad": [0, 0], "stride": [2, 2],
         "dilation": [1, 1], "x": b2[0][1], "w": b2[1][1], "y": [54, 72, 144, 162, 234, 252],
         "y_shape": [1, 1, 3, 2]},
    ])


def softmax():
    body = func_body(read("op_softmax_test.go"), "var testCasesSoftMaxDo")
    cases = []
    # each case: input literal, tensor.Shape{...}, expected literal
    pos = 0
    while True:
        m1 = LIT.search(body, pos)
        if not m1:
            break
        ms = re.compile(r"tensor\.Shape\{([^}]*)\}").search(body, m1.end())
        m2 = LIT.search(body, ms.end())
        cases.append({"input": nums(m1.group(2)), "shape": [int(v) for v in nums(ms.group(1))],
                      "expected": nums(m2.group(2))})
        pos = m2.end()
    assert len(cases) >= 5
    for c in cases:
        n = 1
        for d in c["shape"]:
            n *= d
        assert len(c["input"]) == n == len(c["expected"]), (len(c["input"]), n)
    dump("softmax_do.json", {"source": "op_softmax_test.go:13-100 testCasesSoftMaxDo", "cases": cases})


VAL = re.compile(r"NewF(32|64)\(([^)]*)\)|\[\]float(32|64)\{([^{}]*)\}")


def binop():
    body = func_body(read("op_math_test.go"), "var binOpTests")
    entries = re.split(r"\n\t\{(\w+),\n", body)[1:]
    out = []
    for op, rest in zip(entries[0::2], entries[1::2]):
        vals = []
        for m in VAL.finditer(rest):
            if m.group(1):
                vals.append({"bits": int(m.group(1)), "scalar": True, "v": [float(m.group(2))]})
            else:
                vals.append({"bits": int(m.group(3)), "scalar": False, "v": nums(m.group(4))})
            if len(vals) == 5:
                break
        a, b, correct, deriv_a, deriv_b = vals
        out.append({"op": op, "a": a, "b": b, "correct": correct, "deriv_a": deriv_a, "deriv_b": deriv_b})
    assert len(out) == 32, len(out)
    dump("binop.json", {"source": "op_math_test.go:23-360 binOpTests (a, b, correct, correctDerivA, correctDerivB)", "cases": out})


def batchnorm():
    text = read("nn_amd64_test.go")
    body = func_body(text, "var bnAllCases")
    blocks = re.split(r"\n\t\{\n", body)[1:]
    out = []
    for blk in blocks:
        if "tensor.Float32" not in blk.split("XShape")[0]:
            continue

        def field(name):
            m = re.search(name + r":\s*(.*)", blk)
            return m.group(1).strip().rstrip(",") if m else None

        def shape(name):
            return [int(v) for v in nums(re.search(name + r":\s*tensor\.Shape\{([^}]*)\}", blk).group(1))]

        def lit(name):
            m = re.search(name + r":\s*\[\]float32\{([^{}]*)\}", blk)
            return nums(m.group(1)) if m else None

        x = field("X")
        case = {"desc": field("desc").strip('"'), "x_shape": shape("XShape"),
                "scale_shape": shape("ScaleShape"), "bias_shape": shape("BiasShape"),
                "scale_init": field("ScaleInit"), "bias_init": field("BiasInit"),
                "expected_mean": lit("ExpectedMean"), "expected_variance": lit("ExpectedVariance"),
                "expected_train_result": lit("ExpectedTrainResult"),
                "expected_eval_result": lit("ExpectedEvalResult"),
                "expected_scale_grad": lit("ExpectedScaleGrad"),
                "expected_bias_grad": lit("ExpectedBiasGrad"),
                "expected_output_grad": lit("ExpectedOutputGrad"),
                "expected_input_grad": lit("ExpectedInputGrad")}
        m = re.match(r"RangedFromWithStep\(([^,]*),\s*([^)]*)\)", x)
        if m:
            case["x_ranged"] = [float(m.group(1)), float(m.group(2))]
        else:
            case["x"] = nums(LIT.search(x).group(2))
        out.append(case)
    assert len(out) >= 5, len(out)
    dump("batchnorm.json", {
        "source": "nn_amd64_test.go:8-205 bnAllCases (float32 cases); test body nn_test.go:319-440: "
                  "momentum 0.9, eps 1e-5, one training run, one Adam step (lr 0.02) on "
                  "fcWeight/scale/bias, then an EvalMode run",
        "cases": out})


if __name__ == "__main__":
    maxpool()
    leaky()
    conv()
    softmax()
    binop()
    batchnorm()
