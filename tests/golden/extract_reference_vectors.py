#!/usr/bin/env python3
"""Transcribe the known-answer vectors held by the reference's own unit tests into
tests/golden/reference_vectors.json.

Runs only where the reference tree is mounted (it reads the test files as TEXT and pulls
out the numeric literals: inputs, filters, expected outputs and descriptor arguments; no
reference code is compiled, imported or run).  The JSON it writes is committed; the tests
read the JSON only.

Sources (relative to the reference tree):
  tests/layers/conv/test_conv2d.cpp        7 conv2d forward cases (+ their backward maps)
  tests/layers/pool/test_mpool.cpp         6 max-pool cases (forward values, backward maps)
  tests/layers/pool/test_avgpool.cpp       6 avg-pool cases
  tests/layers/conv/test_convol_sizes.cpp  72-entry output-size table
  tests/tensor/test_tensor_da.cpp          tensor_da_pad
  tests/tensor/nn/test_tensor_nn.cpp       tensor_nn_full_softmax (forward)
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")


def strip_comments(src):
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return re.sub(r"//[^\n]*", "", src)


def numbers(body):
    return [float(t.rstrip("f")) for t in re.findall(r"-?\d+\.?\d*(?:[eE][-+]?\d+)?f?", body)]


def ints(body):
    return [int(t) for t in re.findall(r"-?\d+", body)]


def test_blocks(src):
    """Yield (name, body, first_line) for every TEST(suite, name) block."""
    heads = [(m.start(), m.group(1)) for m in re.finditer(r"TEST\(\s*\w+\s*,\s*(\w+)\s*\)", src)]
    for n, (pos, name) in enumerate(heads):
        end = heads[n + 1][0] if n + 1 < len(heads) else len(src)
        yield name, src[pos:end], src.count("\n", 0, pos) + 1


def arrays_and_tensors(body):
    arrs = {m.group(1): numbers(m.group(2)) for m in re.finditer(r"\*\s*(\w+)\s*=\s*new float\[[^\]]*\]\s*\{(.*?)\};", body, flags=re.S)}
    tens = {}
    for m in re.finditer(r"(\w+)\s*=\s*new Tensor\(\s*\{([^}]*)\}\s*,\s*(\w+)\s*,", body):
        tens[m.group(1)] = {"shape": ints(m.group(2)), "data": arrs[m.group(3)]}
    return arrs, tens


def conv_cases(path):
    raw = open(os.path.join(REF, path)).read()
    cases = []
    for name, body, line in test_blocks(strip_comments(raw)):
        arrs, tens = arrays_and_tensors(body)
        m = re.search(r"new ConvolDescriptor\(\s*(\d+)\s*,\s*\{([^}]*)\}\s*,\s*\{([^}]*)\}\s*,\s*\"(\w+)\"\s*,\s*\{([^}]*)\}\s*,\s*(\d+)\s*,\s*\{([^}]*)\}\s*,\s*(\w+)\s*\)", body)
        if "t_image" not in tens or not m:
            continue  # device-differential tests hold no vectors
        case = {
            "name": name, "source": "%s:%d" % (path, line),
            "filters": int(m.group(1)), "kernel": ints(m.group(2)), "strides": ints(m.group(3)),
            "padding": m.group(4), "use_bias": m.group(8) == "true",
            "image": tens["t_image"], "forward": tens["t_fwrd"], "backward_of_ones": tens["t_bwrd"],
        }
        mk = re.search(r"cd->K\s*=\s*new Tensor\(\s*\{([^}]*)\}\s*,\s*(\w+)", body)
        case["filters_data"] = {"shape": ints(mk.group(1)), "data": arrs[mk.group(2)]} if mk else "ones"
        mb = re.search(r"cd->bias\s*=\s*new Tensor\(\s*\{([^}]*)\}\s*,\s*(\w+)", body)
        case["bias_data"] = {"shape": ints(mb.group(1)), "data": arrs[mb.group(2)]} if mb else "zeros"
        tol = re.search(r"equivalent\(t_fwrd,\s*cd->O,\s*([\d.e-]+)f?\s*,\s*([\d.e-]+)f?", body)
        case["atol"], case["rtol"] = float(tol.group(1)), float(tol.group(2))
        cases.append(case)
    return cases


def pool_cases(path):
    raw = open(os.path.join(REF, path)).read()
    cases = []
    for name, body, line in test_blocks(strip_comments(raw)):
        arrs, tens = arrays_and_tensors(body)
        m = re.search(r"new PoolDescriptor\(\s*\{([^}]*)\}\s*,\s*\{([^}]*)\}\s*,\s*\"(\w+)\"\s*\)", body)
        if "t_image" not in tens or not m or len(tens["t_image"]["shape"]) != 4:
            continue  # 3-D pooling and device-differential tests are outside the path
        tol = re.search(r"equivalent\(t_fwrd,\s*pd->O,\s*([\d.e-]+)f?\s*,\s*([\d.e-]+)f?", body)
        cases.append({
            "name": name, "source": "%s:%d" % (path, line),
            "kernel": ints(m.group(1)), "strides": ints(m.group(2)), "padding": m.group(3),
            "image": tens["t_image"], "forward": tens["t_fwrd"], "backward_of_ones": tens["t_bwrd"],
            "atol": float(tol.group(1)), "rtol": float(tol.group(2)),
        })
    return cases


def size_table(path):
    src = strip_comments(open(os.path.join(REF, path)).read())

    def vec(name, conv):
        m = re.search(r"%s\s*=\s*\{(.*?)\};" % name, src, flags=re.S)
        return conv(m.group(1))

    return {
        "source": path + ":10-55",
        "padding": re.findall(r'"(\w+)"', re.search(r"padding\s*=\s*\{(.*?)\};", src, flags=re.S).group(1)),
        "input_sizes": vec("input_sizes", ints), "strides": vec("strides", ints), "kernels": vec("kernels", ints),
        "output_sizes": vec(r"output_sizes", ints),
        "loop_order": ["padding", "input_sizes", "strides", "kernels"],
    }


def pad_case(path):
    src = strip_comments(open(os.path.join(REF, path)).read())
    body = [b for n, b, _ in test_blocks(src) if n == "tensor_da_pad"][0]
    m = re.search(r"t1_ref\s*=\s*new Tensor\(\s*\{(.*?)\}\s*,\s*\{\s*1\s*,\s*1\s*,\s*3\+pad\*2\s*,\s*3\+pad\*2\s*\}", body, flags=re.S)
    pad = int(re.search(r"pad\s*=\s*(\d+)\s*;", body).group(1))
    return {"source": path + ":14-31", "input": {"shape": [1, 1, 3, 3], "data": [1.0] * 9}, "pads": [pad] * 4,
            "expected": {"shape": [1, 1, 3 + 2 * pad, 3 + 2 * pad], "data": numbers(m.group(1))}, "atol": 1e-3}


def softmax_case(path):
    src = strip_comments(open(os.path.join(REF, path)).read())
    body = [b for n, b, _ in test_blocks(src) if n == "tensor_nn_full_softmax"][0]
    t1 = re.search(r"t1\s*=\s*new Tensor\(\s*\{(.*?)\}\s*,\s*\{([^}]*)\}", body, flags=re.S)
    ref = re.search(r"t1_ref\s*=\s*new Tensor\(\s*\{(.*?)\}\s*,\s*\{([^}]*)\}", body, flags=re.S)
    return {"source": path + ":13-24", "axis": int(re.search(r"axis\s*=\s*(\d+)", body).group(1)),
            "input": {"shape": ints(t1.group(2)), "data": numbers(t1.group(1))},
            "expected": {"shape": ints(ref.group(2)), "data": numbers(ref.group(1))}, "atol": 1e-3}


def main():
    doc = {
        "_about": "Numeric literals transcribed from the unit tests of deephealthproject/eddl v1.1 "
                  "by tests/golden/extract_reference_vectors.py; data only.",
        "conv2d": conv_cases("tests/layers/conv/test_conv2d.cpp"),
        "maxpool2d": pool_cases("tests/layers/pool/test_mpool.cpp"),
        "avgpool2d": pool_cases("tests/layers/pool/test_avgpool.cpp"),
        "output_sizes": size_table("tests/layers/conv/test_convol_sizes.cpp"),
        "pad": pad_case("tests/tensor/test_tensor_da.cpp"),
        "softmax": softmax_case("tests/tensor/nn/test_tensor_nn.cpp"),
    }
    assert len(doc["conv2d"]) == 7 and len(doc["maxpool2d"]) == 6 and len(doc["avgpool2d"]) == 6
    assert len(doc["output_sizes"]["output_sizes"]) == 72
    for group in ("conv2d", "maxpool2d", "avgpool2d"):
        for c in doc[group]:
            for key in ("image", "forward", "backward_of_ones"):
                n = 1
                for d in c[key]["shape"]:
                    n *= d
                assert n == len(c[key]["data"]), (c["name"], key)
    with open(OUT, "w") as fh:
        json.dump(doc, fh, indent=1)
    print("wrote", OUT)


if __name__ == "__main__":
    main()
