"""Extracts the numeric test vectors that Ferrox's own unit tests hold for the hot path and writes them
to reference_vectors.json (data only: inputs and expected outputs).

Run in the build container, where the reference checkout is mounted:
    python tests/golden/extract_reference_vectors.py /root/reference
The reference sources are read as text; nothing is imported or executed.
"""
import json
import os
import re
import sys


def _body(src, fn_name):
    i = src.index(f"fn {fn_name}()")
    j = src.index("#[test]", i) if "#[test]" in src[i:] else len(src)
    return src[i:j]


def _floats(text):
    text = re.sub(r"//[^\n]*", "", text)
    return [float(t) for t in re.findall(r"-?\d+\.\d+(?:e-?\d+)?", text)]


def _vec_blocks(body):
    return [_floats(m) for m in re.findall(r"vec!\[(.*?)\];", body, flags=re.S)]


def main(ref):
    src = open(os.path.join(ref, "src/ops/mod.rs")).read()
    out = {}

    b = _body(src, "conv2d_test")
    blocks = [v for v in _vec_blocks(b) if len(v) > 10]
    x, w, y = blocks[0], blocks[1], blocks[2]
    assert (len(x), len(w), len(y)) == (75, 108, 100), (len(x), len(w), len(y))
    out["conv2d_test"] = {"source": "src/ops/mod.rs:743-801", "x_shape": [1, 3, 5, 5], "x": x, "w_shape": [4, 3, 3, 3],
                          "w": w, "stride": [1, 1], "padding": [1, 1], "y_shape": [1, 4, 5, 5], "y": y, "tol": 1e-3}
    out["conv2d_simple_forward"] = {"source": "src/ops/mod.rs:724-740", "x_shape": [1, 1, 2, 2], "x": [1.0, 2.0, 3.0, 4.0],
                                    "w_shape": [1, 1, 2, 2], "w": [0.5, 0.5, 0.5, 0.5], "stride": [1, 1],
                                    "padding": [0, 0], "y_shape": [1, 1, 1, 1], "y": [5.0], "tol": 1e-5}
    out["conv2d_edge_cases"] = {"source": "src/ops/mod.rs:972-988", "x_shape": [1, 1, 2, 2], "x": [1.0, 2.0, 3.0, 4.0],
                                "w_shape": [1, 1, 1, 1], "w": [2.0], "stride": [1, 1], "padding": [0, 0],
                                "y_shape": [1, 1, 2, 2], "y": [2.0, 4.0, 6.0, 8.0], "tol": 1e-6}

    def simple(fn, n_in):
        body = _body(src, fn)
        arrays = [_floats(m) for m in re.findall(r"&\[([^\]]*)\]", body)]
        arrays = [a for a in arrays if a]
        return arrays

    # (name, function) -> arrays in order of appearance: inputs..., expected
    for key, fn in [("relu", "relu_activation"), ("sigmoid", "sigmoid_activation"), ("tanh", "tanh_activation"),
                    ("matmul", "matrix_multiply"), ("sum_all", "sum_all_elements"), ("sum_axis0", "sum_along_axes"),
                    ("mean_all", "mean_all_elements"), ("mean_axis1", "mean_along_axes"), ("max_all", "max_all_elements"),
                    ("max_axis0", "max_along_axes"), ("softmax_axis1", "softmax_last_axis"),
                    ("softmax_axis0", "softmax_first_axis"), ("neg", "neg_function"), ("min_all", "min_all_elements"),
                    ("min_axis1", "min_along_axes"), ("max_elementwise", "max_elementwise"),
                    ("min_elementwise", "min_elementwise"), ("reciprocal", "reciprocal_operation"),
                    ("maxpool1d", "test_maxpool1d_forward"), ("avgpool1d", "test_avgpool1d_forward"),
                    ("maxpool2d", "test_maxpool2d_forward"), ("avgpool2d", "test_avgpool2d_forward")]:
        arrs = simple(fn, 1)
        out[key] = {"source": f"src/ops/mod.rs fn {fn}", "arrays": arrs}

    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", dst, "keys:", sorted(out))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
