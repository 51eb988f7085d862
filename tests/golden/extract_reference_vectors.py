#!/usr/bin/env python3
"""Collect the known-answer vectors held by the reference's own unit tests.

Run in the build container (the reference checkout is not present on the GPU
box):

    python tests/golden/extract_reference_vectors.py [/root/reference]

It reads the reference's gtest sources as text, pulls out every numeric array
initialiser, the size_t scalars and every EXPECT_NEAR / EXPECT_FLOAT_EQ line of
each TEST_F, and writes them as data to tests/golden/reference_vectors.json.
The tokenizer tests (input strings, expected tokens and ids, character-class
expectations, and the 11-line test vocabulary) go to
tests/golden/tokenization_vectors.json.
No reference code is executed or stored; only inputs and expected outputs are kept.
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


TOKENIZATION_TEST = "test/cuBERT/tokenization_test.cpp"
STRING_RE = r'(?:u8)?"((?:[^"\\]|\\.)*)"'


def c_string(literal):
    """Value of a C/C++ string literal body with \\uXXXX, \\t, \\n, \\r escapes."""
    simple = {"t": "\t", "n": "\n", "r": "\r", "\\": "\\", '"': '"', "0": "\0"}

    def one(m):
        e = m.group(1)
        return chr(int(e[1:], 16)) if e[0] in "uU" else simple[e]

    return re.sub(r"\\(u[0-9A-Fa-f]{4}|U[0-9A-Fa-f]{8}|.)", one, literal)


def char_literal(text):
    text = text.strip()
    m = re.fullmatch(r"'(\\?.)'", text)
    if m:
        return ord(c_string(m.group(1)))
    return int(text, 0)


def parse_tokenization(path):
    """Per TEST_F of the tokenizer tests: the tokenize calls in order (receiver, input text) with the tokens and
    ids expected afterwards, and the character-class expectations."""
    text = open(path, encoding="utf8").read()
    out = {}
    marks = list(TEST_RE.finditer(text))
    for i, m in enumerate(marks):
        body = text[m.end():marks[i + 1].start() if i + 1 < len(marks) else len(text)]
        steps, classes = [], []
        ctor = re.search(r"cuBERT::(\w+)\s+tokenizer\s*(?:\(([^)]*)\))?\s*;", body)
        for line in body.splitlines():
            call = re.search(r"tokenizer\.tokenize\(\s*" + STRING_RE + r"\s*,\s*&tokens(?:\s*,\s*(\d+))?\s*\)", line)
            if call:
                steps.append({"op": "tokenize", "text": c_string(call.group(1)),
                              "max_length": int(call.group(2)) if call.group(2) else None})
                continue
            if re.search(r"tokens\.clear\(\)", line):
                steps.append({"op": "clear"})
                continue
            init = re.search(r"std::vector<std::string>\s+tokens\s*=\s*\{(.*)\}\s*;", line)
            if init:
                steps.append({"op": "set", "tokens": [c_string(x) for x in re.findall(STRING_RE, init.group(1))]})
                continue
            streq = re.search(r"EXPECT_STREQ\(\s*tokens\[(\d+)\]\.c_str\(\)\s*,\s*" + STRING_RE + r"\s*\)", line)
            if streq:
                steps.append({"op": "expect_token", "index": int(streq.group(1)), "token": c_string(streq.group(2))})
                continue
            size = re.search(r"EXPECT_EQ\(\s*tokens\.size\(\)\s*,\s*(\d+)\s*\)", line)
            if size:
                steps.append({"op": "expect_size", "size": int(size.group(1))})
                continue
            ident = re.search(r"EXPECT_EQ\(\s*ids\[(\d+)\]\s*,\s*(\d+)\s*\)", line)
            if ident:
                steps.append({"op": "expect_id", "index": int(ident.group(1)), "id": int(ident.group(2))})
                continue
            cls = re.search(r"EXPECT_(TRUE|FALSE)\(\s*cuBERT::(_is_\w+)\((.*)\)\s*\)\s*;", line)
            if cls:
                classes.append({"function": cls.group(2), "code_point": char_literal(cls.group(3)),
                                "expect": cls.group(1) == "TRUE"})
        out[m.group(1)] = {"receiver": ctor.group(1) if ctor else None,
                           "constructor_args": (ctor.group(2) or "").strip() if ctor else "",
                           "steps": steps, "char_classes": classes}
    vocab = open(os.path.join(os.path.dirname(os.path.dirname(os.path.dirname(path))), "test_vocab.txt"),
                 encoding="utf8").read().split("\n")
    return {"tests": out, "test_vocab": [v for v in vocab if v != ""]}


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    result = {}
    for rel in FILES:
        result[rel] = parse(os.path.join(ref, rel))
    here = os.path.dirname(os.path.abspath(__file__))
    dst = os.path.join(here, "reference_vectors.json")
    with open(dst, "w") as f:
        json.dump(result, f, indent=1, sort_keys=True)
    n = sum(len(t["expect"]) for r in result.values() for t in r["tests"].values())
    print("wrote %s: %d files, %d expectations" % (dst, len(result), n))
    tok = parse_tokenization(os.path.join(ref, TOKENIZATION_TEST))
    dst = os.path.join(here, "tokenization_vectors.json")
    with open(dst, "w") as f:
        json.dump(tok, f, indent=1, sort_keys=True, ensure_ascii=True)
    print("wrote %s: %d tests, %d steps, %d character classes" % (
        dst, len(tok["tests"]), sum(len(t["steps"]) for t in tok["tests"].values()),
        sum(len(t["char_classes"]) for t in tok["tests"].values())))


if __name__ == "__main__":
    main()
