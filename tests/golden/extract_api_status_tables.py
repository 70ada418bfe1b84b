#!/usr/bin/env python3
"""Writes tests/golden/api_status_tables.json from the reference's api_gtest tables.

The reference pins the status code of every hot-path entry point with value-parameterised
gtest tables (`INSTANTIATE_TEST_CASE_P(name, suite, testing::Combine(testing::Values(...), ...))`)
in test/mlu_op_gtest/api_gtest/src/gtest/<op>/<op>_general.cpp.  This script reads those files
as text, parses the parameter tuples and writes them out as plain data (descriptor shapes,
dtypes, layouts, scalar parameters, expected status).  It copies no code; it is run by hand in
the build container, where /root/reference exists, and its JSON output is what the tests load.

    python tests/golden/extract_api_status_tables.py [/root/reference]
"""
import itertools
import json
import os
import re
import sys

OPS = {
    "get_indice_pairs": "get_indice_pairs/get_indice_pairs_general.cpp",
    "indice_convolution_forward": "indice_convolution_forward/indice_convolution_forward_general.cpp",
    "indice_convolution_backward_data":
        "indice_convolution_backward_data/indice_convolution_backward_data_general.cpp",
    "indice_convolution_backward_filter":
        "indice_convolution_backward_filter/indice_convolution_backward_filter_general.cpp",
    "voxelization": "voxelization/voxelization_general.cpp",
    "dynamic_point_to_voxel_forward":
        "dynamic_point_to_voxel_forward/dynamic_point_to_voxel_forward_general.cpp",
    "dynamic_point_to_voxel_backward":
        "dynamic_point_to_voxel_backward/dynamic_point_to_voxel_backward_general.cpp",
}

TOKEN = re.compile(r"\s*([A-Za-z_][A-Za-z_0-9:<> ]*[A-Za-z_0-9>]|[A-Za-z_]|-?\d+|[(){},])")


def tokenize(text):
    pos, out = 0, []
    text = text.strip()
    while pos < len(text):
        m = TOKEN.match(text, pos)
        if not m:
            raise ValueError("cannot tokenize at: %r" % text[pos:pos + 40])
        out.append(m.group(1).strip())
        pos = m.end()
    return out


def parse_expr(tokens, i):
    """expr := INT | NAME | NAME '(' args ')' | NAME '{' args '}' | '{' args '}'.
    Returns (value, next_index); calls become {"call": name, "args": [...]}."""
    t = tokens[i]
    if re.fullmatch(r"-?\d+", t):
        return int(t), i + 1
    if t == "{":
        args, i = parse_args(tokens, i + 1, "}")
        return args, i
    name = t
    if i + 1 < len(tokens) and tokens[i + 1] in "({":
        close = ")" if tokens[i + 1] == "(" else "}"
        args, j = parse_args(tokens, i + 2, close)
        return {"call": name, "args": args}, j
    return name, i + 1


def parse_args(tokens, i, close):
    args = []
    if tokens[i] == close:
        return args, i + 1
    while True:
        v, i = parse_expr(tokens, i)
        args.append(v)
        if tokens[i] == ",":
            i += 1
            continue
        if tokens[i] == close:
            return args, i + 1
        raise ValueError("unexpected token %r" % tokens[i])


def simplify(v):
    """std::vector<..>({..}) -> list; MLUOpTensorParam(..) -> dict; other tuples -> list."""
    if isinstance(v, dict):
        name, args = v["call"], [simplify(a) for a in v["args"]]
        if name.startswith("std::vector"):
            return args[0] if args and isinstance(args[0], list) else args
        if name == "MLUOpTensorParam":
            d = {"layout": args[0], "dtype": args[1], "dim_nb": args[2], "dims": args[3]}
            if len(args) > 4:
                d["strides"] = args[4]
            if len(args) > 5:
                d["onchip_dtype"] = args[5]
            return d
        return args
    if isinstance(v, list):
        return [simplify(a) for a in v]
    return v


def extract_blocks(text):
    """Yields (case_name, suite, combine_argument_text) per INSTANTIATE_TEST_CASE_P."""
    for m in re.finditer(r"INSTANTIATE_TEST_CASE_P\s*\(", text):
        depth, j = 1, m.end()
        while depth:
            c = text[j]
            depth += c == "("
            depth -= c == ")"
            j += 1
        body = text[m.end():j - 1]
        name, suite, rest = body.split(",", 2)
        yield name.strip(), suite.strip(), rest.strip()


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    base = os.path.join(ref, "test/mlu_op_gtest/api_gtest/src/gtest")
    out = {}
    for op, rel in OPS.items():
        text = open(os.path.join(base, rel)).read()
        text = re.sub(r"//[^\n]*", "", text)
        cases = []
        for name, suite, rest in extract_blocks(text):
            tree, _ = parse_expr(tokenize(rest), 0)
            assert tree["call"] == "testing::Combine", tree["call"]
            axes = []
            for values in tree["args"]:
                assert values["call"] == "testing::Values"
                axes.append([simplify(a) for a in values["args"]])
            for idx, combo in enumerate(itertools.product(*axes)):
                last = combo[-1]
                if isinstance(last, list) and len(last) == 2 and str(last[1]).startswith("MLUOP_STATUS"):
                    combo = tuple(combo[:-1]) + (last[0], last[1])  # PublicParam{device, status}
                cases.append({"name": "%s/%d" % (name, idx), "params": list(combo[:-2]),
                              "device": combo[-2], "expected": combo[-1]})
        out[op] = {"source": "test/mlu_op_gtest/api_gtest/src/gtest/" + rel, "cases": cases}
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "api_status_tables.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
    print({k: len(v["cases"]) for k, v in out.items()})


if __name__ == "__main__":
    main()
