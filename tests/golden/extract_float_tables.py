"""Writes tests/golden/float_tables.json: the value tables the reference's own test holds for the
low-precision formats on the block-scaled matmul path.

The reference file test/test_float_encoding.py (lines 49-186) is parsed as TEXT with ``ast`` (it is
neither imported nor executed); only the list literals f4e2m1fn_values, f8e4m3fn_values and
f8e8m0fnu_values are evaluated (``math.nan`` -> the string "nan").  Index = bit pattern.

Run once in the build container:  python tests/golden/extract_float_tables.py
"""
import ast
import json
import math
import pathlib

SRC = pathlib.Path("/root/reference/test/test_float_encoding.py")
OUT = pathlib.Path(__file__).with_name("float_tables.json")
WANTED = ("f4e2m1fn_values", "f8e4m3fn_values", "f8e8m0fnu_values")


def _value(node):
    if isinstance(node, ast.Constant):
        return float(node.value)
    if isinstance(node, ast.UnaryOp) and isinstance(node.op, ast.USub):
        v = _value(node.operand)
        return "nan" if v == "nan" else -v
    if isinstance(node, ast.Attribute) and node.attr == "nan":
        return "nan"
    raise ValueError(ast.dump(node))


def main():
    tree = ast.parse(SRC.read_text())
    tables = {}
    for node in tree.body:
        if isinstance(node, ast.Assign) and isinstance(node.targets[0], ast.Name) \
                and node.targets[0].id in WANTED:
            vals = [_value(e) for e in node.value.elts]
            # keep the sign of -0.0 visible in JSON
            tables[node.targets[0].id] = [
                v if v == "nan" else ("-0.0" if (v == 0 and math.copysign(1, v) < 0) else v)
                for v in vals]
    assert set(tables) == set(WANTED)
    assert len(tables["f4e2m1fn_values"]) == 16
    assert len(tables["f8e4m3fn_values"]) == 256 and len(tables["f8e8m0fnu_values"]) == 256
    OUT.write_text(json.dumps({"source": "test/test_float_encoding.py:49-186", **tables}, indent=0))
    print("wrote", OUT)


if __name__ == "__main__":
    main()
