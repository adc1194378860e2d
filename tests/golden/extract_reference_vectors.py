#!/usr/bin/env python3
"""Collects known-answer vectors held by the reference's own C++ unit tests into reference_vectors.json.

The reference's test sources are read as TEXT: array literals (order, shape, data), linspace/assign
fills, the op's integer/float arguments and the expected arrays are parsed out of the matmul, softmax
and argmax test cases.  Nothing of the reference is imported, compiled or executed.  Only data ends up
in the fixture: every case is {inputs, args, expected}.

Sources (relative to <reference>/libnd4j/tests_cpu/layers_tests/):
  DeclarableOpsTests14.cpp  matmul_test1..38   (orders c/f, transX/Y/Z, vectors, batched)
  DeclarableOpsTests1.cpp   softmax_test1..12, ArgMax1..6
  DeclarableOpsTests19.cpp  test_matmul_ccc/fcf/cff/... (alpha/beta: 1*ones(10,10)^2 + 1*100 = 110)

Usage: python tests/golden/extract_reference_vectors.py [/root/reference]
"""
import json
import os
import re
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
TESTS = os.path.join(REF, "libnd4j", "tests_cpu", "layers_tests")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")

NUM = r"[-+]?(?:\d+\.?\d*(?:[eE][-+]?\d+)?|\.\d+(?:[eE][-+]?\d+)?)"


def numbers(text):
    text = re.sub(r"(?<=[\d.])[fFL]\b", "", text)
    return [float(t) for t in re.findall(NUM, text)]


def test_bodies(path, prefix):
    src = open(path).read()
    out = {}
    for m in re.finditer(r"TEST_F\(\s*\w+\s*,\s*(%s\w*)\s*\)\s*\{" % prefix, src):
        depth, i = 1, m.end()
        while depth and i < len(src):
            depth += {"{": 1, "}": -1}.get(src[i], 0)
            i += 1
        out[m.group(1)] = src[m.end():i - 1]
    return out


DT = {"double": "float64", "float": "float32", "LongType": "int64", "sd::LongType": "int64", "int": "int32",
      "FLOAT32": "float32", "DOUBLE": "float64", "INT64": "int64", "INT32": "int32"}


def parse_arrays(body):
    """name -> {order, shape, data|None, dtype}; data is in buffer order, as the literals are."""
    arrays = {}
    # auto x = NDArrayFactory::create<T>('c', {shape}[, {data}]);
    for m in re.finditer(r"auto\s+(\w+)\s*=\s*NDArrayFactory::create<\s*([\w:]+)\s*>\(\s*'(\w)'\s*,\s*\{([^}]*)\}\s*(?:,\s*\{([^}]*)\})?\s*\)\s*;", body, re.S):
        name, t, order, shp, data = m.groups()
        arrays[name] = {"order": order, "shape": [int(v) for v in numbers(shp)], "data": numbers(data) if data is not None else None, "dtype": DT.get(t)}
    # auto e = NDArrayFactory::create<T>(scalar);
    for m in re.finditer(r"auto\s+(\w+)\s*=\s*NDArrayFactory::create<\s*([\w:]+)\s*>\(\s*(%s)[fF]?\s*\)\s*;" % NUM, body):
        name, t, v = m.groups()
        arrays[name] = {"order": "c", "shape": [], "data": [float(v)], "dtype": DT.get(t)}
    # NDArray x('c', {shape}, {data}, FLOAT32);
    for m in re.finditer(r"NDArray\s+(\w+)\(\s*'(\w)'\s*,\s*\{([^}]*)\}\s*,\s*\{([^}]*)\}\s*(?:,\s*(?:sd::)?(?:DataType::)?(\w+))?\s*\)\s*;", body, re.S):
        name, order, shp, data, t = m.groups()
        arrays[name] = {"order": order, "shape": [int(v) for v in numbers(shp)], "data": numbers(data), "dtype": DT.get(t or "DOUBLE")}
    return arrays


def fill(arrays, body):
    """Apply x.linspace(a[, b]) / x.assign(v): values in LOGICAL row-major order (NDArray::linspace walks
    linear indices), flagged so the consumer lays them out by `order`."""
    for m in re.finditer(r"(\w+)(?:\.|->)linspace\(\s*(%s)[fF]?\s*(?:,\s*(%s)[fF]?\s*)?\)" % (NUM, NUM), body):
        name, a, b = m.groups()
        if name in arrays and arrays[name]["data"] is None:
            n = 1
            for s in arrays[name]["shape"]:
                n *= s
            step = float(b) if b is not None else 1.0
            arrays[name]["logical"] = [float(a) + step * i for i in range(n)]
    for m in re.finditer(r"(\w+)\.assign\(\s*(%s)[fF]?\s*\)" % NUM, body):
        name, v = m.groups()
        if name in arrays and arrays[name]["data"] is None:
            n = 1
            for s in arrays[name]["shape"]:
                n *= s
            arrays[name]["logical"] = [float(v)] * n
    for a in arrays.values():
        if a["data"] is None and "logical" not in a:
            return False
    return True


def pack(a):
    d = {"order": a["order"], "shape": a["shape"], "dtype": a["dtype"]}
    if a["data"] is not None:
        d["buffer"] = a["data"]      # buffer order
    else:
        d["logical"] = a["logical"]  # row-major logical order
    return d


def evaluate_call(body):
    """op.evaluate({&a, &b}, {targs}, {iargs}[, {bargs}]) / op.execute({&a,&b}, {&z}, {targs}[, {iargs}])"""
    m = re.search(r"op\.evaluate\(\s*\{([^}]*)\}\s*(?:,\s*\{([^}]*)\}\s*)?(?:,\s*\{([^}]*)\}\s*)?(?:,\s*\{([^}]*)\}\s*)?\)", body)
    if m:
        ins = re.findall(r"&(\w+)", m.group(1))
        return {"inputs": ins, "outputs": None, "targs": numbers(m.group(2) or ""), "iargs": [int(v) for v in numbers(m.group(3) or "")],
                "bargs": [t.strip() == "true" for t in (m.group(4) or "").split(",") if t.strip()]}
    m = re.search(r"op\.execute\(\s*\{([^}]*)\}\s*,\s*\{([^}]*)\}\s*(?:,\s*\{([^}]*)\}\s*)?(?:,\s*\{([^}]*)\}\s*)?", body)
    if m:
        return {"inputs": re.findall(r"&(\w+)", m.group(1)), "outputs": re.findall(r"&(\w+)", m.group(2)),
                "targs": numbers(m.group(3) or ""), "iargs": [int(v) for v in numbers(m.group(4) or "")], "bargs": []}
    return None


def collect(path, prefix, op, exp_names):
    cases = []
    for name, body in sorted(test_bodies(path, prefix).items()):
        arrays = parse_arrays(body)
        call = evaluate_call(body)
        exp = next((n for n in exp_names if n in arrays), None)
        if not call or exp is None or not fill(arrays, body):
            continue
        if any(i not in arrays for i in call["inputs"]):
            continue
        case = {"name": name, "op": op, "source": os.path.basename(path), "inputs": [pack(arrays[i]) for i in call["inputs"]],
                "targs": call["targs"], "iargs": call["iargs"], "bargs": call["bargs"], "expected": pack(arrays[exp])}
        if call["outputs"]:
            case["initial_output"] = pack(arrays[call["outputs"][0]])
        cases.append(case)
    return cases


def main():
    cases = []
    cases += collect(os.path.join(TESTS, "DeclarableOpsTests14.cpp"), "matmul_test", "matmul", ["exp"])
    cases += collect(os.path.join(TESTS, "DeclarableOpsTests19.cpp"), "test_matmul_", "matmul", ["e"])
    cases += collect(os.path.join(TESTS, "DeclarableOpsTests1.cpp"), "softmax_test", "softmax", ["expOutput", "exp"])
    cases += collect(os.path.join(TESTS, "DeclarableOpsTests1.cpp"), "ArgMax", "argmax", ["exp"])
    with open(OUT, "w") as f:
        json.dump({"comment": "known-answer vectors parsed from the reference's C++ unit tests (data only)", "cases": cases}, f, indent=0)
    by_op = {}
    for c in cases:
        by_op[c["op"]] = by_op.get(c["op"], 0) + 1
    print("wrote", OUT, by_op)


if __name__ == "__main__":
    main()
