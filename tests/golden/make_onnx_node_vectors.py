"""Writes tests/golden/onnx_node_vectors.json.

The reference pins its quantized ops with eight ONNX backend node tests and the three
DynamicQuantizeLinear ones
(scripts/runtests.py:556-563,577-582 in the chainer-compiler tree); their data
files live in an ONNX checkout that is not part of that tree.  The inputs and
expected outputs below are the ONNX operator-specification examples those node
tests are generated from.  Before writing, every expected output is re-derived
here in float64 / int64 from the ONNX operator definitions, so a typo in a
vector fails this script rather than a test.

Run:  python tests/golden/make_onnx_node_vectors.py
"""
import json
import os

import numpy as np

V = {}

V["test_quantizelinear"] = dict(
    x=[0, 2, 3, 1000, -254, -1000], y_scale=2.0, y_zero_point=128, zp_dtype="uint8",
    y=[128, 129, 130, 255, 1, 0])

V["test_dequantizelinear"] = dict(
    x=[0, 3, 128, 255], x_dtype="uint8", x_scale=2.0, x_zero_point=128,
    y=[-256, -250, 0, 254])

V["test_qlinearmatmul_2D"] = dict(
    a=[[208, 236, 0, 238], [3, 214, 255, 29]], a_scale=0.0066, a_zero_point=113,
    b=[[152, 51, 244], [60, 26, 255], [0, 127, 246], [127, 254, 247]], b_scale=0.00705, b_zero_point=114,
    y_scale=0.0107, y_zero_point=118,
    y=[[168, 115, 255], [1, 66, 151]])

V["test_qlinearmatmul_3D"] = dict(
    a=[V["test_qlinearmatmul_2D"]["a"]] * 2, a_scale=0.0066, a_zero_point=113,
    b=[V["test_qlinearmatmul_2D"]["b"]] * 2, b_scale=0.00705, b_zero_point=114,
    y_scale=0.0107, y_zero_point=118,
    y=[V["test_qlinearmatmul_2D"]["y"]] * 2)

V["test_qlinearconv"] = dict(
    x=[[255, 174, 162, 25, 203, 168, 58],
       [15, 59, 237, 95, 129, 0, 64],
       [56, 242, 153, 221, 168, 12, 166],
       [232, 178, 186, 195, 237, 162, 237],
       [188, 39, 124, 77, 80, 102, 43],
       [127, 230, 21, 83, 41, 40, 134],
       [255, 154, 92, 141, 42, 148, 247]],
    x_shape=[1, 1, 7, 7], x_scale=0.00369204697, x_zero_point=132,
    w=[0], w_shape=[1, 1, 1, 1], w_scale=[0.00172794575], w_zero_point=[255],
    y_scale=0.00162681262, y_zero_point=123,
    y=[[0, 81, 93, 230, 52, 87, 197],
       [240, 196, 18, 160, 126, 255, 191],
       [199, 13, 102, 34, 87, 243, 89],
       [23, 77, 69, 60, 18, 93, 18],
       [67, 216, 131, 178, 175, 153, 212],
       [128, 25, 234, 172, 214, 215, 121],
       [0, 101, 163, 114, 213, 107, 8]])

V["test_matmulinteger"] = dict(
    a=[[11, 7, 3], [10, 6, 2], [9, 5, 1], [8, 4, 0]], a_zero_point=12,
    b=[[1, 4], [2, 5], [3, 6]], b_zero_point=0,
    y=[[-38, -83], [-44, -98], [-50, -113], [-56, -128]])

V["test_basic_convinteger"] = dict(
    x=list(range(2, 11)), x_shape=[1, 1, 3, 3], x_zero_point=1,
    w=[1, 1, 1, 1], w_shape=[1, 1, 2, 2], pads=[0, 0],
    y=[12, 16, 24, 28], y_shape=[1, 1, 2, 2])

V["test_convinteger_with_padding"] = dict(
    x=list(range(2, 11)), x_shape=[1, 1, 3, 3], x_zero_point=1,
    w=[1, 1, 1, 1], w_shape=[1, 1, 2, 2], pads=[1, 1],
    y=[1, 3, 5, 3, 5, 12, 16, 9, 11, 24, 28, 15, 7, 15, 17, 9], y_shape=[1, 1, 4, 4])

# DynamicQuantizeLinear: y_scale and y_zero_point are outputs of the node
V["test_dynamicquantizelinear"] = dict(
    x=[0, 2, -3, -2.5, 1.34, 0.5], x_shape=[6],
    y=[153, 255, 0, 26, 221, 179], y_scale=0.0196078438, y_zero_point=153)

V["test_dynamicquantizelinear_max_adjusted"] = dict(
    x=[-1.0, -2.1, -1.3, -2.5, -3.34, -4.0], x_shape=[6],
    y=[191, 121, 172, 96, 42, 0], y_scale=0.0156862754, y_zero_point=255)

V["test_dynamicquantizelinear_min_adjusted"] = dict(
    x=[1, 2.1, 1.3, 2.5, 3.34, 4.0, 1.5, 2.6, 3.9, 4.0, 3.0, 2.345], x_shape=[3, 4],
    y=[64, 134, 83, 159, 213, 255, 96, 166, 249, 255, 191, 149], y_scale=0.0156862754, y_zero_point=0)

# Round (ties to even), which the DynamicQuantizeLinear body uses and the reference also runs on its own
V["test_round"] = dict(
    x=[0.1, 0.5, 0.9, 1.2, 1.5, 1.8, 2.3, 2.5, 2.7, -1.1, -1.5, -1.9, -2.2, -2.5, -2.8],
    y=[0.0, 0.0, 1.0, 1.0, 2.0, 2.0, 2.0, 2.0, 3.0, -1.0, -2.0, -2.0, -2.0, -2.0, -3.0])


def rne_sat(v, lo=0, hi=255):
    return np.clip(np.rint(v), lo, hi).astype(np.int64)


def check():
    t = V["test_quantizelinear"]
    got = np.clip(np.rint(np.array(t["x"], dtype=np.float64) / t["y_scale"]) + t["y_zero_point"], 0, 255)
    assert got.astype(int).tolist() == t["y"], got

    t = V["test_dequantizelinear"]
    got = (np.array(t["x"], dtype=np.float64) - t["x_zero_point"]) * t["x_scale"]
    assert got.tolist() == t["y"], got

    for name in ("test_qlinearmatmul_2D", "test_qlinearmatmul_3D"):
        t = V[name]
        a = np.array(t["a"], dtype=np.int64) - t["a_zero_point"]
        b = np.array(t["b"], dtype=np.int64) - t["b_zero_point"]
        acc = np.matmul(a, b)
        got = rne_sat(acc * (t["a_scale"] * t["b_scale"] / t["y_scale"]) + t["y_zero_point"])
        assert got.tolist() == t["y"], (name, got)

    t = V["test_qlinearconv"]
    x = np.array(t["x"], dtype=np.int64) - t["x_zero_point"]
    w = t["w"][0] - t["w_zero_point"][0]
    got = rne_sat(x * w * (t["x_scale"] * t["w_scale"][0] / t["y_scale"]) + t["y_zero_point"])
    assert got.tolist() == t["y"], got

    t = V["test_matmulinteger"]
    got = (np.array(t["a"], dtype=np.int64) - t["a_zero_point"]) @ (np.array(t["b"], dtype=np.int64) - t["b_zero_point"])
    assert got.tolist() == t["y"], got

    for name in ("test_basic_convinteger", "test_convinteger_with_padding"):
        t = V[name]
        x = np.array(t["x"], dtype=np.int64).reshape(3, 3) - t["x_zero_point"]
        p = t["pads"][0]
        xp = np.pad(x, p)
        oh = xp.shape[0] - 1
        got = [[int(xp[i:i + 2, j:j + 2].sum()) for j in range(oh)] for i in range(oh)]
        assert np.array(got).reshape(-1).tolist() == t["y"], (name, got)

    # DynamicQuantizeLinear, from the operator definition in float32 as the node test generator
    # evaluates it: range widened to contain 0, scale = range / 255, zero point = clip(round(0 - min /
    # scale)), y = clip(round(x / scale) + zero point)
    for name in ("test_dynamicquantizelinear", "test_dynamicquantizelinear_max_adjusted", "test_dynamicquantizelinear_min_adjusted"):
        t = V[name]
        x = np.array(t["x"], dtype=np.float32)
        x_min, x_max = np.minimum(np.float32(0), x.min()), np.maximum(np.float32(0), x.max())
        scale = np.float32((x_max - x_min) / np.float32(255))
        zp = np.clip(np.rint((np.float32(0) - x_min) / scale), 0, 255).astype(np.uint8)
        y = np.clip(np.rint(x / scale) + zp, 0, 255).astype(np.uint8)
        assert y.tolist() == t["y"] and int(zp) == t["y_zero_point"], (name, y, zp)
        assert np.float32(t["y_scale"]) == scale, (name, scale)
    t = V["test_round"]
    assert np.rint(np.array(t["x"], dtype=np.float32)).tolist() == t["y"]

if __name__ == "__main__":
    check()
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "onnx_node_vectors.json")
    with open(out, "w") as f:
        json.dump(V, f, indent=1, sort_keys=True)
    print("wrote", out)
