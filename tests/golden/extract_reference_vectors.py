#!/usr/bin/env python3
"""Collect the known-answer vectors held by the reference's own unit tests.

Run in the build container (the reference checkout is not present on the GPU
box):

    python tests/golden/extract_reference_vectors.py [/root/reference]

It reads the reference's gtest sources as text, pulls out every numeric array
initialiser, the size_t scalars and every EXPECT_NEAR / EXPECT_FLOAT_EQ line of
each TEST_F, and writes them as data to tests/golden/reference_vectors.json.
No reference code is executed or stored; only numbers are kept.
"""
import json
import math
import os
import re
import sys

FILES = [
    "test/cuBERT/op/DenseTest.cpp",
    "test/cuBERT/op/EmbeddingTest.cpp",
    "test/cuBERT/op/GELUTest.cpp",
    "test/cuBERT/op/LayerNormTest.cpp",
    "test/cuBERT/op/SoftmaxTest.cpp",
    "test/cuBERT/op_att/AttentionMaskTest.cpp",
    "test/cuBERT/op_att/BatchMatMulTest.cpp",
    "test/cuBERT/op_att/AttentionSelfTest.cpp",
    "test/cuBERT/op_att/TransformerTest.cpp",
    "test/cuBERT/op_bert/BertEmbeddingsTest.cpp",
    "test/cuBERT/op_bert/BertPoolerTest.cpp",
    "test/cuBERT/op_out/AdditionalOutputLayerTest.cpp",
]

ARRAY_RE = re.compile(
    r"\b(float|int|int8_t)\s+(\w+)\s*\[\s*\d*\s*\]\s*=\s*\{([^}]*)\}\s*;", re.S)
SCALAR_RE = re.compile(r"\bsize_t\s+(\w+)\s*=\s*(\d+)\s*;")
EXPECT_RE = re.compile(r"EXPECT_(NEAR|FLOAT_EQ)\s*\(\s*(\w+)\[(\d+)\]\s*,\s*(.*)\)\s*;")
TEST_RE = re.compile(r"TEST_F\s*\(\s*\w+\s*,\s*(\w+)\s*\)")

SAFE = {"sqrt": math.sqrt, "tanhf": math.tanh, "erf": math.erf}


def evaluate(expr):
    """Evaluate a C arithmetic literal expression such as `1 - std::sqrt(1.5)`."""
    e = expr.strip().replace("std::", "")
    e = re.sub(r"(\d+\.?\d*(?:[eE][-+]?\d+)?)[fF]\b", r"\1", e)   # 1.f -> 1.
    e = re.sub(r"(\d+\.)(?=\s|$|[-+*/)])", r"\g<1>0", e)
    if not re.fullmatch(r"[\w\s.+\-*/()eE]*", e):
        raise ValueError("unexpected expression: %r" % expr)
    return float(eval(e, {"__builtins__": {}}, SAFE))  # literals and the three functions above only


def numbers(body):
    return [evaluate(tok) for tok in body.replace("\n", " ").split(",") if tok.strip()]


def split_top_level(text):
    """Split 'a, b' at the last top-level comma (for EXPECT_NEAR's tolerance)."""
    depth = 0
    cut = None
    for i, ch in enumerate(text):
        if ch == "(":
            depth += 1
        elif ch == ")":
            depth -= 1
        elif ch == "," and depth == 0:
            cut = i
    return (text, None) if cut is None else (text[:cut], text[cut + 1:])


def parse(path):
    src = open(path).read()
    src = re.sub(r"//[^\n]*", "", src)
    # file-scope arrays precede the first TEST_F
    marks = [(m.start(), m.group(1)) for m in TEST_RE.finditer(src)]
    out = {"globals": {}, "tests": {}}
    head = src[: marks[0][0]] if marks else src
    for m in ARRAY_RE.finditer(head):
        out["globals"][m.group(2)] = numbers(m.group(3))
    for i, (pos, name) in enumerate(marks):
        end = marks[i + 1][0] if i + 1 < len(marks) else len(src)
        body = src[pos:end]
        t = {"arrays": {}, "scalars": {}, "expect": []}
        for m in ARRAY_RE.finditer(body):
            t["arrays"][m.group(2)] = numbers(m.group(3))
        for m in SCALAR_RE.finditer(body):
            t["scalars"][m.group(1)] = int(m.group(2))
        for m in EXPECT_RE.finditer(body):
            kind, var, idx, rest = m.group(1), m.group(2), int(m.group(3)), m.group(4)
            val, tol = split_top_level(rest) if kind == "NEAR" else (rest, None)
            try:
                value = evaluate(val)
            except (ValueError, NameError):
                # the expected value is computed in the test body (GELUTest's
                # double-precision closed form): keep the expression as text
                value = val.strip()
            t["expect"].append([var, idx, value, None if tol is None else evaluate(tol)])
        out["tests"][name] = t
    return out


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    result = {}
    for rel in FILES:
        result[rel] = parse(os.path.join(ref, rel))
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(dst, "w") as f:
        json.dump(result, f, indent=1, sort_keys=True)
    n = sum(len(t["expect"]) for r in result.values() for t in r["tests"].values())
    print("wrote %s: %d files, %d expectations" % (dst, len(result), n))


if __name__ == "__main__":
    main()
