"""Writes tests/golden/jax_custom_primitives.json: the input / expected arrays that the reference's JAX
custom-primitive tests hold as literals, read from the test files as TEXT (nothing is imported or run):
  mlir-tensorrt/integrations/PJRT/test/JAX/CustomPrimitives/test_dynamic_quantize.py  (x, expected)
  mlir-tensorrt/integrations/PJRT/test/JAX/CustomPrimitives/test_quantize.py:60-83
  mlir-tensorrt/integrations/PJRT/test/JAX/CustomPrimitives/test_dequantize.py:62-101
Run in the container that has /root/reference mounted:  python tests/golden/make_jax_known_answers.py
"""
import ast
import json
import os
import re

REF = "/root/reference/mlir-tensorrt/integrations/PJRT/test/JAX/CustomPrimitives"
HERE = os.path.dirname(os.path.abspath(__file__))


def array_literals(path, func):
    """The nested-list literals of `np.array([...])` calls inside function `func`, in order."""
    text = open(path).read()
    body = text[text.index("def %s(" % func):]
    nxt = re.search(r"\n(?:def |@|if __name__)", body[1:])
    body = body[: nxt.start() + 1] if nxt else body
    out = []
    for m in re.finditer(r"np\.array\(\s*(\[)", body):
        depth, i = 0, m.start(1)
        for j in range(i, len(body)):
            depth += body[j] == "["
            depth -= body[j] == "]"
            if depth == 0:
                out.append(ast.literal_eval(body[i:j + 1]))
                break
    return out


def main():
    dq = array_literals(os.path.join(REF, "test_dynamic_quantize.py"), "test_dynamic_quantize_pt")
    q_pt = array_literals(os.path.join(REF, "test_quantize.py"), "test_quantize_pt")
    q_pc = array_literals(os.path.join(REF, "test_quantize.py"), "test_quantize_pc")
    q_bl = array_literals(os.path.join(REF, "test_quantize.py"), "test_quantize_block")
    d_pt = array_literals(os.path.join(REF, "test_dequantize.py"), "test_dequantize_pt")
    d_pc = array_literals(os.path.join(REF, "test_dequantize.py"), "test_dequantize_pc")
    d_bl = array_literals(os.path.join(REF, "test_dequantize.py"), "test_dequantize_block")
    doc = {
        "dynamic_quantize_pt": {"double_quant_scale": 1.0, "axis": 1, "x": dq[0], "expected": dq[1]},
        "quantize_pt": {"scale": 1.0, "x": q_pt[0], "expected": q_pt[1]},
        "quantize_pc": {"scale": [2.0, 10.0], "axis": 0, "x": q_pc[0], "expected": q_pc[1]},
        "quantize_block": {"scale": [[1.0, 1.0, 1.0, 1.0]], "x": q_bl[0], "expected": q_bl[1]},
        "dequantize_pt": {"scale": 0.5, "x": d_pt[0], "expected": d_pt[1]},
        "dequantize_pc": {"scale": [0.5, 0.1], "axis": 0, "x": d_pc[0], "expected": d_pc[1]},
        "dequantize_block": {"scale": [[2.0, 2.0, 2.0, 2.0]], "x": d_bl[0], "expected": d_bl[1]},
    }
    with open(os.path.join(HERE, "jax_custom_primitives.json"), "w") as f:
        json.dump(doc, f, indent=1)
    print({k: (len(v["x"]), len(v["x"][0])) for k, v in doc.items()})


if __name__ == "__main__":
    main()
