"""Writes tests/golden/reference_vectors.json from the golden vectors the reference's own C++
tests hold for sort and argsort.

    python tests/golden/extract_reference_vectors.py [/root/reference]

Only data is taken: the literal input arrays, the shapes/axes they are tried on and the literal
expected outputs in
    tests/cpp/integration/test_sort.cc          (int32 :26-60, double :62-96, inputs :541-555)
    tests/cpp/integration/test_argsort.cc       (12-element :26-60, 4-D..7-D :62-204, inputs :282-377)
    tests/cpp/integration/test_sort_complex.cc  (complex :27-126, from integers :141-152, 4-D..7-D
                                                 :154-195, inputs and shapes :257-345)
The reference is read as text, never imported, built or run.  Cases the reference generates by
formula (10 000 reversed elements :379-410, empty :412-433, single item :435-455; test_sort_complex.cc
:347-390) are restated as formulas in tests/test_oracle.py instead of being stored.  Complex values are stored as
[real, imag] pairs (test_sort.cc:98-134,557-571, test_argsort.cc:298-311,330-344).
"""
from __future__ import annotations

import json
import re
import sys
from pathlib import Path


def function_body(text: str, name: str) -> str:
    start = text.index(name + "()")
    brace = text.index("{", start)
    depth, i = 0, brace
    while True:
        c = text[i]
        if c == "{":
            depth += 1
        elif c == "}":
            depth -= 1
            if depth == 0:
                return text[brace : i + 1]
        i += 1


def parse_expect_table(body: str) -> list[dict[str, list[float]]]:
    """`{ {{axis, {v...}}, {axis, {v...}}}, ... }` -> one {axis: values} dict per shape.
    A brace initialiser of numbers is JSON once braces become brackets."""
    init = body[body.index("= {") + 2 : body.rindex("};") + 1]
    nested = json.loads(init.replace("{", "[").replace("}", "]"))
    return [{str(axis): vals for axis, vals in per_shape} for per_shape in nested]


COMPLEX = re.compile(r"legate::Complex<\w+>\(\s*([-0-9.eE]+)\s*,\s*([-0-9.eE]+)\s*\)")


def decomplex(text: str) -> str:
    """`legate::Complex<float>(a, b)` -> `{a, b}` so that the generic brace parser applies."""
    return COMPLEX.sub(lambda m: "{" + m.group(1) + "," + m.group(2) + "}", text)


def parse_complex_array(text: str, decl: str) -> list[list[float]]:
    i = text.index(decl)
    j = text.index("{", i)
    k = text.index("};", j)
    return [[float(a), float(b)] for a, b in COMPLEX.findall(text[j:k])]


def parse_shapes(text: str, anchor: str) -> list[list[int]]:
    i = text.index(anchor)
    j = text.index("=", i)
    k = text.index(";", j)
    return [[int(v) for v in re.findall(r"\d+", grp)] for grp in re.findall(r"\{([\d\s,]+)\}", text[j:k])]


def parse_array(text: str, decl: str) -> list[float]:
    i = text.index(decl)
    j = text.index("{", i)
    k = text.index("}", j)
    return [float(v) if "." in v else int(v) for v in re.split(r"\s*,\s*", text[j + 1 : k].strip())]


def main() -> None:
    ref = Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    tdir = ref / "tests" / "cpp" / "integration"
    sort_cc = (tdir / "test_sort.cc").read_text()
    argsort_cc = (tdir / "test_argsort.cc").read_text()

    shapes12 = parse_shapes(sort_cc[sort_cc.index("void sort_basic_axis()") :], "test_shapes")
    out: dict = {"source": "tests/cpp/integration/test_sort.cc, test_argsort.cc", "cases": []}

    def add(op, dtype, data, shapes, table, stable_only, where):
        assert len(shapes) == len(table), (where, len(shapes), len(table))
        for shape, per_axis in zip(shapes, table):
            ndim = len(shape)
            assert sorted(int(a) for a in per_axis) == list(range(-ndim + 1, ndim)), (where, shape, per_axis.keys())
            for axis, expect in per_axis.items():
                out["cases"].append(
                    {
                        "op": op,
                        "dtype": dtype,
                        "input": data,
                        "shape": shape,
                        "axis": int(axis),
                        "expect": expect,
                        "stable_only": stable_only,
                        "where": where,
                    }
                )

    # sort: test_sort.cc
    body = sort_cc[sort_cc.index("void sort_basic_axis()") :]
    add("sort", "int32", parse_array(body, "in_array1"), shapes12,
        parse_expect_table(function_body(sort_cc, "get_expect_result_int")), False, "test_sort.cc:26-60,547")
    add("sort", "float64", parse_array(body, "in_array2"), shapes12,
        parse_expect_table(function_body(sort_cc, "get_expect_result_double")), False, "test_sort.cc:62-96,552")

    add("sort", "complex64", parse_complex_array(body, "in_array3"), shapes12,
        parse_expect_table(decomplex(function_body(sort_cc, "get_expect_result_complex"))), False,
        "test_sort.cc:98-134,557")

    # argsort: test_argsort.cc
    table12 = parse_expect_table(function_body(argsort_cc, "get_argsort_expect_result"))
    body = argsort_cc[argsort_cc.index("void argsort_basic_axis()") :]
    add("argsort", "int32", parse_array(body, "in_array1"), shapes12, table12, False, "test_argsort.cc:26-60,290")
    add("argsort", "float64", parse_array(body, "in_array2"), shapes12, table12, False, "test_argsort.cc:26-60,294")
    add("argsort", "complex64", parse_complex_array(body, "in_array3"), shapes12, table12, False,
        "test_argsort.cc:26-60,298")
    body = argsort_cc[argsort_cc.index("void argsort_basic_axis_stable()") :]
    add("argsort", "int32", parse_array(body, "in_array1"), shapes12, table12, True, "test_argsort.cc:26-60,321")
    add("argsort", "float64", parse_array(body, "in_array2"), shapes12, table12, True, "test_argsort.cc:26-60,326")
    add("argsort", "complex64", parse_complex_array(body, "in_array3"), shapes12, table12, True,
        "test_argsort.cc:26-60,330")

    body = argsort_cc[argsort_cc.index("void argsort_basic_axis_max_dim()") :]
    data16 = parse_array(body, "in_array")
    for nd in (4, 5, 6, 7):
        shapes = parse_shapes(body, f"test_shapes_{nd}d")
        table = parse_expect_table(function_body(argsort_cc, f"get_argsort_expect_result_{nd}d"))
        add("argsort", "int32", data16, shapes, table, False, f"test_argsort.cc get_argsort_expect_result_{nd}d")

    # sort_complex: test_sort_complex.cc.  One expected array per shape (the sort is along the last axis).
    cplx_cc = (tdir / "test_sort_complex.cc").read_text()
    out["source"] += ", test_sort_complex.cc"
    out["sort_complex_cases"] = []

    def add_complex(in_dtype, out_dtype, data, shapes, table, where):
        assert len(shapes) == len(table), (where, len(shapes), len(table))
        for shape, expect in zip(shapes, table):
            out["sort_complex_cases"].append({"in_dtype": in_dtype, "out_dtype": out_dtype, "input": data,
                                              "shape": shape, "expect": expect, "where": where})

    def int_table(fn_name):
        body = function_body(cplx_cc, fn_name)
        init = body[body.index("= {") + 2 : body.index("};") + 1]
        return [[[float(v), 0.0] for v in row] for row in json.loads(init.replace("{", "[").replace("}", "]"))]

    def complex_table(fn_name):
        body = decomplex(function_body(cplx_cc, fn_name))
        init = body[body.index("= {") + 2 : body.index("};") + 1]
        return json.loads(init.replace("{", "[").replace("}", "]"))

    body = cplx_cc[cplx_cc.index("void sort_complex_basic()") : cplx_cc.index("void sort_complex_basic_max_dim()")]
    shapes_int = parse_shapes(body, "test_shapes_int")
    from_int = int_table("get_sort_complex_expect_result_from_int")
    ints = parse_array(body, "in_array1")
    assert ints == parse_array(body, "in_array2") == parse_array(body, "int_array3")
    add_complex("int8", "complex64", ints, shapes_int, from_int, "test_sort_complex.cc:141-152,257-274")
    add_complex("int16", "complex64", ints, shapes_int, from_int, "test_sort_complex.cc:141-152,265-268")
    add_complex("int32", "complex128", ints, shapes_int, from_int, "test_sort_complex.cc:141-152,271-274")
    shapes_c = parse_shapes(body[body.index("// Test complex type") :], "test_shapes")
    table_c = complex_table("get_sort_complex_expect_result")
    in4 = parse_complex_array(body, "in_array4")
    assert in4 == parse_complex_array(body, "in_array5")
    add_complex("complex64", "complex64", in4, shapes_c, table_c, "test_sort_complex.cc:27-126,277-295")
    add_complex("complex128", "complex128", in4, shapes_c, table_c, "test_sort_complex.cc:27-126,297-312")
    body = cplx_cc[cplx_cc.index("void sort_complex_basic_max_dim()") : cplx_cc.index("void sort_complex_large_array()")]
    data16c = parse_array(body, "in_array")
    for nd in (4, 5, 6, 7):
        add_complex("int16", "complex64", data16c, parse_shapes(body, f"test_shapes_{nd}d"),
                    int_table(f"get_sort_complex_expect_result_{nd}d"),
                    f"test_sort_complex.cc get_sort_complex_expect_result_{nd}d")

    dst = Path(__file__).resolve().parent / "reference_vectors.json"
    dst.write_text(json.dumps(out, separators=(",", ":")) + "\n")
    print(f"{len(out['cases'])} sort/argsort cases, {len(out['sort_complex_cases'])} sort_complex cases -> {dst}")


if __name__ == "__main__":
    main()
