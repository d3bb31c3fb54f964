"""Extracts the golden vectors that the reference's own unit tests hold and writes
them as JSON fixtures next to this script.

Reads the reference's test sources as text only (nothing is compiled, imported or
run).  Only numeric data leaves the files: the brace-initialised float arrays, the
Scale shapes and the ConvInfo / PoolingInfo arguments of each TEST body.

  tests/unittest_conv_forward.cpp:7-68      -> conv_forward.json
  tests/unittest_pooling_forward.cpp:7-81   -> pooling_forward.json

Usage (in the build container, where /root/reference is mounted):
  python tests/golden/extract_reference_vectors.py [/root/reference]
"""
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def _tests(text):
    """Yield (name, body) for every TEST(...) { ... } block."""
    for m in re.finditer(r"TEST\((\w+),\s*(\w+)\)\s*\{", text):
        start = m.end()
        nxt = text.find("\nTEST(", start)
        body = text[start: nxt if nxt >= 0 else len(text)]
        yield m.group(2), body


def _array(body, name):
    m = re.search(r"float\s+%s\[\]\s*=\s*\{([^}]*)\}" % name, body)
    if not m:
        return None
    return [float(tok) for tok in m.group(1).replace("\n", " ").split(",") if tok.strip()]


def _scale(body, name):
    m = re.search(r"Scale\s+%s\s*\{([^}]*)\}" % name, body)
    return [int(t) for t in m.group(1).split(",")] if m else None


def conv(ref):
    text = open(os.path.join(ref, "tests/unittest_conv_forward.cpp")).read()
    cases = []
    for name, body in _tests(text):
        if not name.startswith("Gpu"):
            continue  # the DISABLED_Cpu twins repeat the same data
        info = re.search(r"ConvInfo\s+conv_info\(([^)]*)\)", body).group(1)
        ph, pw, sv, sh = [int(t) for t in info.split(",")]
        cases.append({
            "name": name,
            "input_size": _scale(body, "input_size"),
            "weight_size": _scale(body, "weight_size"),
            "correct_size": _scale(body, "correct_size"),
            "pad_height": ph, "pad_width": pw,
            "stride_vertical": sv, "stride_horizontal": sh,
            "input": _array(body, "input_raw"),
            "weight": _array(body, "weight_raw"),
            "bias": _array(body, "bias_raw"),
            # the test compares against correct_raw[i] + bias[(i / 16) % 5]
            "correct_without_bias": _array(body, "correct_raw"),
            "tolerance": 1e-3,
        })
    return cases


def pooling(ref):
    text = open(os.path.join(ref, "tests/unittest_pooling_forward.cpp")).read()
    cases = []
    for name, body in _tests(text):
        info = re.search(r"PoolingInfo\s+pooling_info\(PoolingInfo::Algorithm::kMax,([^)]*)\)",
                         body).group(1)
        a = [int(t) for t in info.split(",")]
        a += [1, 1, 0, 0][len(a) - 2:] if len(a) < 6 else []
        # constructor order (convolution_info.h:24-31): h, w, sv, sh, ph, pw
        h, w, sv, sh, ph, pw = (a + [0, 0])[:6]
        cases.append({
            "name": name,
            "input_size": _scale(body, "input_size"),
            "correct_size": _scale(body, "correct_size"),
            "height": h, "width": w, "stride_vertical": sv, "stride_horizontal": sh,
            "pad_height": ph, "pad_width": pw,
            "input": _array(body, "input_raw"),
            "correct": _array(body, "correct_raw"),
        })
    return cases


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    with open(os.path.join(HERE, "conv_forward.json"), "w") as f:
        json.dump(conv(ref), f)
    with open(os.path.join(HERE, "pooling_forward.json"), "w") as f:
        json.dump(pooling(ref), f)


if __name__ == "__main__":
    main()
