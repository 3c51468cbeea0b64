"""Writes the golden fixtures under tests/golden/ from the data the reference's own tests hold.

Run in the build container (needs /root/reference as TEXT only; nothing of the reference is imported
or executed). The fixtures are data: expected output vectors and the parameters that produce them.
"""
import json
import os
import re

REF = "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def numbers_between(text, start_marker, end_marker):
    s = text.index(start_marker) + len(start_marker)
    e = text.index(end_marker, s)
    return [float(t) for t in re.findall(r"-?\d+\.?\d*(?:[eE]-?\d+)?", text[s:e])]


def polynomial_value(text, variables):
    """Value of an arithmetic expression taken from the reference's source text. The text is parsed, never executed: only
    numbers, the given variable names, unary +/- and the operators + - * / are accepted; anything else raises."""
    import ast
    import operator

    binary = {ast.Add: operator.add, ast.Sub: operator.sub, ast.Mult: operator.mul, ast.Div: operator.truediv}
    unary = {ast.UAdd: operator.pos, ast.USub: operator.neg}

    def value(node):
        if isinstance(node, ast.Expression):
            return value(node.body)
        if isinstance(node, ast.Constant) and type(node.value) in (int, float):
            return float(node.value)
        if isinstance(node, ast.Name) and node.id in variables:
            return variables[node.id]
        if isinstance(node, ast.BinOp) and type(node.op) in binary:
            return binary[type(node.op)](value(node.left), value(node.right))
        if isinstance(node, ast.UnaryOp) and type(node.op) in unary:
            return unary[type(node.op)](value(node.operand))
        raise ValueError(f"not a polynomial in {sorted(variables)}: {ast.dump(node)[:80]}")

    return value(ast.parse(text, mode="eval"))


def main():
    # test/doctest_packing.cpp:21-46 : get_packed_weights of the vector 1..512 (two 16x16 matrices)
    txt = open(os.path.join(REF, "test/doctest_packing.cpp")).read()
    vals = numbers_between(txt, "std::vector<float> reference_values = {", "};")
    assert len(vals) == 512
    json.dump(
        {
            "source": "test/doctest_packing.cpp:21-46",
            "input_width": 16, "network_width": 16, "output_width": 16, "n_hidden_layers": 1,
            "unpacked": "1..512",
            "packed": [int(v) for v in vals],
        },
        open(os.path.join(HERE, "packing_16x16x2.json"), "w"),
    )

    # test/doctest_encodings.cpp:234-285 : 3-D hash grid, x = (1,1,1), params i/(n/2) - 1
    txt = open(os.path.join(REF, "test/doctest_encodings.cpp")).read()
    s = txt.index("Test grid encoding using create_grid_encoding instead of factory")
    vals = numbers_between(txt[s:], "const std::vector<float> reference_out = {", "};")
    assert len(vals) == 32
    json.dump(
        {
            "source": "test/doctest_encodings.cpp:234-285",
            "n_dims": 3, "n_levels": 16, "n_features_per_level": 2, "log2_hashmap_size": 19,
            "base_resolution": 16, "per_level_scale": 2.0, "grid_type": "Hash",
            "hash": "CoherentPrime", "interpolation": "Linear", "padded_output_width": 32,
            "input": [1.0, 1.0, 1.0], "params": "i / (n_params / 2) - 1 (test/doctest_encodings.cpp:27-34)",
            "tolerance": 1.0e-3, "tolerance_metric": "max|a-b| / max(max|a|, max|b|)  (include/common/result_check.h:83-102)",
            "expected": vals,
        },
        open(os.path.join(HERE, "grid_forward_3d.json"), "w"),
    )

    # toPackedLayoutCoord / fromPackedLayoutCoord point values: test/doctest_common.cpp:25-119
    json.dump(
        {
            "source": "test/doctest_common.cpp:25-119",
            "to_packed": [[0, 1, 1, 0], [1, 2, 2, 2], [2, 2, 2, 1], [4, 4, 2, 4], [5, 4, 2, 6], [6, 4, 2, 5]],
            "from_packed": [[0, 1, 1, 0], [1, 2, 2, 2], [2, 2, 2, 1], [4, 4, 2, 4], [5, 4, 2, 6], [6, 4, 2, 5]],
            "columns": "idx, rows, cols, expected",
            # test/python/test_packing.py:9-48
            "pack_4x4": {"unpacked": [[1, 2, 3, 4], [5, 6, 7, 8], [9, 10, 11, 12], [13, 14, 15, 16]],
                         "packed": [[1, 5, 2, 6], [3, 7, 4, 8], [9, 13, 10, 14], [11, 15, 12, 16]]},
        },
        open(os.path.join(HERE, "packed_coords.json"), "w"),
    )

    # test/python/test_encodings.py:377-573 : spherical harmonics of degree 4 at the input (1, 1, 1) (ten equal rows)
    txt = open(os.path.join(REF, "test/python/test_encodings.py")).read()
    s = txt.index("def test_spherical():")
    vals = numbers_between(txt[s:], "spherical_output = torch.Tensor(", ").to(")
    assert len(vals) == 160 and vals[:16] == vals[16:32]
    json.dump(
        {
            "source": "test/python/test_encodings.py:377-573",
            "degree": 4, "input": [1.0, 1.0, 1.0], "n_rows": 10, "atol": 1.0e-3,
            "expected_row": vals[:16],
        },
        open(os.path.join(HERE, "spherical_harmonics_degree4.json"), "w"),
    )

    # include/common/common_device.h:33-206 : the 64 polynomials of sh_enc (bands 0-7), evaluated from the reference's own
    # text at seeded points. The fixture holds encoding inputs in [0, 1]^3 (the encoding maps them to 2x - 1,
    # include/encodings/spherical_harmonics.h:38-72) and the 64 values per point.
    import random
    import re
    src = open(os.path.join(REF, "include/common/common_device.h")).read()
    body = src[src.index("void sh_enc("):src.index("} // namespace kernels") if "} // namespace kernels" in src else len(src)]
    body = re.sub(r"//[^\n]*", "", body)  # the comments repeat the formulas in another notation
    stmts = re.findall(r"data_out\[(\d+) \+ offset\]\s*=\s*\(T\)\((.*?)\);", body, flags=re.S)
    assert [int(i) for i, _ in stmts] == list(range(64)), "expected the 64 assignments of sh_enc in order"
    exprs = [re.sub(r"(?<=[0-9.])f\b", "", " ".join(e.split())) for _, e in stmts]
    rnd = random.Random(2024)
    inputs = [[rnd.random(), rnd.random(), rnd.random()] for _ in range(24)] + [[1.0, 1.0, 1.0], [0.0, 0.5, 1.0], [0.5, 0.5, 0.5]]
    expected = []
    for p in inputs:
        x, y, z = (2.0 * c - 1.0 for c in p)
        env = dict(x=x, y=y, z=z, xy=x * y, xz=x * z, yz=y * z, x2=x * x, y2=y * y, z2=z * z)
        env.update(x4=env["x2"] ** 2, y4=env["y2"] ** 2, z4=env["z2"] ** 2)
        env.update(x6=env["x4"] * env["x2"], y6=env["y4"] * env["y2"], z6=env["z4"] * env["z2"])
        expected.append([polynomial_value(e, env) for e in exprs])
    json.dump(
        {
            "source": "include/common/common_device.h:33-206 (the polynomials of sh_enc, evaluated in double precision)",
            "degree": 8, "atol": 2.0e-5, "inputs": inputs, "expected": expected,
        },
        open(os.path.join(HERE, "spherical_harmonics_degree8.json"), "w"),
    )


if __name__ == "__main__":
    main()
