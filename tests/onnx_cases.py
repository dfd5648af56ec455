"""The quantized-path ONNX node tests the reference runs (scripts/runtests.py:556-563), rebuilt
as test directories (model.onnx + test_data_set_0/{input,output}_i.pb) from the known-answer
vectors of tests/golden/onnx_node_vectors.json.  As in the ONNX backend test suite, every node
input -- scales and zero points included -- is a graph input with its own input_i.pb."""
import os

import numpy as np


def _case(ol, op, names, arrays, out, attrs=None):
    g = ol.Graph()
    g.name = "test_" + op.lower()
    g.nodes.append(ol.Node(op, names, ["y"], attrs or {}))
    g.inputs = [(n, ol.ONNX_OF[a.dtype], list(a.shape)) for n, a in zip(names, arrays)]
    g.outputs = [("y", ol.ONNX_OF[out.dtype], list(out.shape))]
    return g, arrays, [out]


def build_cases(ol, vec):
    f32, u8, i32 = np.float32, np.uint8, np.int32
    cases = {}
    t = vec["test_quantizelinear"]
    cases["test_quantizelinear"] = _case(ol, "QuantizeLinear", ["x", "y_scale", "y_zero_point"],
                                         [np.array(t["x"], f32), np.array(t["y_scale"], f32), np.array(t["y_zero_point"], u8)],
                                         np.array(t["y"], u8))
    t = vec["test_dequantizelinear"]
    cases["test_dequantizelinear"] = _case(ol, "DequantizeLinear", ["x", "x_scale", "x_zero_point"],
                                           [np.array(t["x"], u8), np.array(t["x_scale"], f32), np.array(t["x_zero_point"], u8)],
                                           np.array(t["y"], f32))
    for k in ("test_qlinearmatmul_2D", "test_qlinearmatmul_3D"):
        t = vec[k]
        cases[k] = _case(ol, "QLinearMatMul",
                         ["a", "a_scale", "a_zero_point", "b", "b_scale", "b_zero_point", "y_scale", "y_zero_point"],
                         [np.array(t["a"], u8), np.array(t["a_scale"], f32), np.array(t["a_zero_point"], u8),
                          np.array(t["b"], u8), np.array(t["b_scale"], f32), np.array(t["b_zero_point"], u8),
                          np.array(t["y_scale"], f32), np.array(t["y_zero_point"], u8)], np.array(t["y"], u8))
    t = vec["test_qlinearconv"]
    cases["test_qlinearconv"] = _case(
        ol, "QLinearConv", ["x", "x_scale", "x_zero_point", "w", "w_scale", "w_zero_point", "y_scale", "y_zero_point"],
        [np.array(t["x"], u8).reshape(t["x_shape"]), np.array(t["x_scale"], f32), np.array(t["x_zero_point"], u8),
         np.array(t["w"], u8).reshape(t["w_shape"]), np.array(t["w_scale"], f32), np.array(t["w_zero_point"], u8),
         np.array(t["y_scale"], f32), np.array(t["y_zero_point"], u8)], np.array(t["y"], u8).reshape(1, 1, 7, 7))
    for k in ("test_basic_convinteger", "test_convinteger_with_padding"):
        t = vec[k]
        attrs = {"pads": list(t["pads"]) * 2} if any(t["pads"]) else {}
        cases[k] = _case(ol, "ConvInteger", ["x", "w", "x_zero_point"],
                         [np.array(t["x"], u8).reshape(t["x_shape"]), np.array(t["w"], u8).reshape(t["w_shape"]),
                          np.array(t["x_zero_point"], u8)], np.array(t["y"], i32).reshape(t["y_shape"]), attrs)
    t = vec["test_matmulinteger"]
    cases["test_matmulinteger"] = _case(ol, "MatMulInteger", ["A", "B", "a_zero_point", "b_zero_point"],
                                        [np.array(t["a"], u8), np.array(t["b"], u8), np.array([t["a_zero_point"]], u8),
                                         np.array([t["b_zero_point"]], u8)], np.array(t["y"], i32))
    return cases


def write_case(ol, root, name, case):
    graph, inputs, outputs = case
    d = os.path.join(root, name)
    os.makedirs(os.path.join(d, "test_data_set_0"))
    with open(os.path.join(d, "model.onnx"), "wb") as f:
        f.write(ol.make_model(graph))
    for prefix, arrays, names in (("input", inputs, [i[0] for i in graph.inputs]), ("output", outputs, ["y"])):
        for i, (a, n) in enumerate(zip(arrays, names)):
            with open(os.path.join(d, "test_data_set_0", "%s_%d.pb" % (prefix, i)), "wb") as f:
                f.write(ol.make_tensor(n, a))
    return d
