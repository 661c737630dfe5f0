#!/usr/bin/env python3
"""Writes the known-answer fixtures of this directory from the literal input/expected vectors
the reference's own backend tests hold (ngraph/test/backend/*.in.cpp).  Only the numbers are
taken: every test body is scanned for brace-initialised Shape / Strides / CoordinateDiff /
vector<float> declarations, which become one JSON record per test.  Runs only where the
reference checkout is present; the JSON it writes is what travels.

    python tests/golden/extract_reference_vectors.py [/root/reference]
"""
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
DECL = re.compile(
    r"(?:const\s+)?(?:std::)?(Shape|Strides|CoordinateDiff|size_t|vector<float>|vector<int64_t>)"
    r"\s*&?\s+(\w+)\s*(?:\{([^{}]*)\}|=\s*([^;{}]+));", re.S)
CONST = re.compile(
    r"auto\s+(\w+)\s*=\s*op::Constant::create\(\s*element::f32\s*,\s*Shape\{([^{}]*)\}\s*,"
    r"\s*\{([^{}]*)\}\s*\)", re.S)
EXPECTED = re.compile(r"add_expected_output<float>\(\s*\w+\s*,\s*(?:std::)?vector<float>\{([^{}]*)\}", re.S)


def nums(text, as_float):
    vals = []
    for tok in text.replace("\n", " ").split(","):
        tok = tok.strip()
        if not tok:
            continue
        tok = re.sub(r"[fFuUlL]+$", "", tok) if not tok.lower().endswith("inf") else tok
        vals.append(float(tok) if as_float else int(float(tok)))
    return vals


def tests_of(path):
    src = open(path).read()
    src = re.sub(r"//[^\n]*", "", src)  # comments inside the literal vectors
    parts = re.split(r"NGRAPH_TEST\(\$\{BACKEND_NAME\},\s*(\w+)\)", src)
    for i in range(1, len(parts), 2):
        yield parts[i], parts[i + 1]


def extract(path):
    out = {}
    for name, body in tests_of(path):
        rec = {}
        for kind, var, braces, assign in DECL.findall(body):
            text = braces if braces is not None and braces != "" or assign == "" else assign
            try:
                if kind == "size_t":
                    rec[var] = int(text.strip())
                else:
                    rec[var] = nums(text, kind == "vector<float>")
            except ValueError:
                pass
        for var, shape, data in CONST.findall(body):
            rec[var] = {"shape": nums(shape, False), "data": nums(data, True)}
        m = EXPECTED.search(body)
        if m:
            rec["expected"] = nums(m.group(1), True)
        if "PDPD" in body:
            ax = re.search(r"AutoBroadcastType::PDPD\s*,\s*(-?\d+)", body)
            rec["pdpd_axis"] = int(ax.group(1))
        if "RoundingType::CEIL" in body:
            rec["ceil"] = True
        if "exclude_pad = " in body:
            rec["exclude_pad"] = "exclude_pad = true" in body
        for k in ("SAME_UPPER", "SAME_LOWER"):
            if "PadType::" + k in body:
                rec["auto_pad"] = k
        out[name] = rec
    return out


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    backend = os.path.join(ref, "ngraph", "test", "backend")
    for stem in ("fake_quantize", "convolution", "group_convolution", "max_pool", "avg_pool", "prelu"):
        rec = extract(os.path.join(backend, stem + ".in.cpp"))
        dst = os.path.join(HERE, stem + ".json")
        with open(dst, "w") as f:
            json.dump({"source": "ngraph/test/backend/%s.in.cpp" % stem, "tests": rec}, f, indent=1)
        print(stem, len(rec), "tests ->", dst)


if __name__ == "__main__":
    main()
