"""The quantized-path ONNX node tests the reference runs (scripts/runtests.py:556-563,577-582), rebuilt
as test directories (model.onnx + test_data_set_0/{input,output}_i.pb) from the known-answer
vectors of tests/golden/onnx_node_vectors.json.  As in the ONNX backend test suite, every node
input -- scales and zero points included -- is a graph input with its own input_i.pb."""
import os

import numpy as np


def _case(ol, op, names, arrays, out, attrs=None, out_names=("y",)):
    outs = list(out) if isinstance(out, (list, tuple)) else [out]
    g = ol.Graph()
    g.name = "test_" + op.lower()
    g.nodes.append(ol.Node(op, names, list(out_names), attrs or {}))
    g.inputs = [(n, ol.ONNX_OF[a.dtype], list(a.shape)) for n, a in zip(names, arrays)]
    g.outputs = [(n, ol.ONNX_OF[o.dtype], list(o.shape)) for n, o in zip(out_names, outs)]
    return g, arrays, outs


def _dynamic_quantize_expanded(ol, x, outs):
    """The body of the ONNX function DynamicQuantizeLinear as nodes of the graph, which is what the
    *_expanded node tests hold."""
    f32 = np.float32
    g = ol.Graph()
    g.name = "test_dynamicquantizelinear_expanded"
    N = ol.Node
    g.nodes = [
        N("Constant", [], ["Q_Min"], {"value": np.array(0, f32)}), N("Constant", [], ["Q_Max"], {"value": np.array(255, f32)}),
        N("ReduceMin", ["x"], ["X_Min"], {"keepdims": 0}), N("Min", ["X_Min", "Q_Min"], ["X_Min_Adjusted"]),
        N("ReduceMax", ["x"], ["X_Max"], {"keepdims": 0}), N("Max", ["X_Max", "Q_Min"], ["X_Max_Adjusted"]),
        N("Sub", ["X_Max_Adjusted", "X_Min_Adjusted"], ["X_Range"]), N("Div", ["X_Range", "Q_Max"], ["Scale"]),
        N("Div", ["X_Min_Adjusted", "Scale"], ["Min_Scaled"]), N("Sub", ["Q_Min", "Min_Scaled"], ["Initial_ZeroPoint_FP"]),
        N("Clip", ["Initial_ZeroPoint_FP", "Q_Min", "Q_Max"], ["Clipped_ZeroPoint_FP"]),
        N("Round", ["Clipped_ZeroPoint_FP"], ["Rounded_ZeroPoint_FP"]),
        N("Cast", ["Rounded_ZeroPoint_FP"], ["Zeropoint"], {"to": ol.ONNX_OF[np.dtype(np.uint8)]}),
        N("Identity", ["Scale"], ["y_scale"]), N("Identity", ["Zeropoint"], ["y_zero_point"]),
        N("QuantizeLinear", ["x", "Scale", "Zeropoint"], ["y"])]
    g.inputs = [("x", ol.ONNX_OF[x.dtype], list(x.shape))]
    g.outputs = [(n, ol.ONNX_OF[o.dtype], list(o.shape)) for n, o in zip(("y", "y_scale", "y_zero_point"), outs)]
    return g, [x], list(outs)


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
    t = vec["test_round"]
    cases["test_round"] = _case(ol, "Round", ["x"], [np.array(t["x"], f32)], np.array(t["y"], f32))
    for k in ("test_dynamicquantizelinear", "test_dynamicquantizelinear_max_adjusted", "test_dynamicquantizelinear_min_adjusted"):
        t = vec[k]
        x = np.array(t["x"], f32).reshape(t["x_shape"])
        outs = [np.array(t["y"], u8).reshape(t["x_shape"]), np.array(t["y_scale"], f32), np.array(t["y_zero_point"], u8)]
        cases[k] = _case(ol, "DynamicQuantizeLinear", ["x"], [x], outs, out_names=("y", "y_scale", "y_zero_point"))
        cases[k + "_expanded"] = _dynamic_quantize_expanded(ol, x, outs)
    return cases


def write_case(ol, root, name, case):
    graph, inputs, outputs = case
    d = os.path.join(root, name)
    os.makedirs(os.path.join(d, "test_data_set_0"))
    with open(os.path.join(d, "model.onnx"), "wb") as f:
        f.write(ol.make_model(graph))
    for prefix, arrays, names in (("input", inputs, [i[0] for i in graph.inputs]), ("output", outputs, [o[0] for o in graph.outputs])):
        for i, (a, n) in enumerate(zip(arrays, names)):
            with open(os.path.join(d, "test_data_set_0", "%s_%d.pb" % (prefix, i)), "wb") as f:
                f.write(ol.make_tensor(n, a))
    return d
