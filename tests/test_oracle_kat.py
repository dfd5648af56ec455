"""Pins the CPU oracle against the known-answer vectors of the eight ONNX node
tests the reference runs for this path (scripts/runtests.py:556-563,577-582 in the
chainer-compiler tree), under the reference's own rounding (+0.5f, truncate)."""
import numpy as np
import pytest


def test_quantizelinear(oracle, onnx_vectors):
    t = onnx_vectors["test_quantizelinear"]
    y = oracle.quantize_linear(np.array(t["x"], np.float32), t["y_scale"], t["y_zero_point"], np.uint8)
    assert y.dtype == np.uint8 and y.tolist() == t["y"]
    # the ONNX text (round-half-even) agrees on this vector too
    y2 = oracle.quantize_linear(np.array(t["x"], np.float32), t["y_scale"], t["y_zero_point"], np.uint8,
                                round_mode=oracle.ROUND_ONNX_RNE)
    assert y2.tolist() == t["y"]
    # multi-pass spelling == single pass
    assert oracle.quantize_linear_multipass(np.array(t["x"], np.float32), t["y_scale"], t["y_zero_point"]).tolist() == t["y"]


def test_dequantizelinear(oracle, onnx_vectors):
    t = onnx_vectors["test_dequantizelinear"]
    y = oracle.dequantize_linear(np.array(t["x"], np.uint8), t["x_scale"], t["x_zero_point"])
    assert y.dtype == np.float32 and y.tolist() == t["y"]
    assert oracle.dequantize_linear(np.array(t["x"], np.uint8), t["x_scale"], t["x_zero_point"], multipass=True).tolist() == t["y"]


@pytest.mark.parametrize("name", ["test_qlinearmatmul_2D", "test_qlinearmatmul_3D"])
def test_qlinearmatmul(oracle, onnx_vectors, name):
    t = onnx_vectors[name]
    a, b = np.array(t["a"], np.uint8), np.array(t["b"], np.uint8)
    args = (a, t["a_scale"], t["a_zero_point"], b, t["b_scale"], t["b_zero_point"], t["y_scale"], t["y_zero_point"])
    assert oracle.qlinear_matmul_int(*args).tolist() == t["y"]
    assert oracle.qlinear_matmul_literal(*args).tolist() == t["y"]


def test_qlinearconv(oracle, onnx_vectors):
    t = onnx_vectors["test_qlinearconv"]
    x = np.array(t["x"], np.uint8).reshape(t["x_shape"])
    w = np.array(t["w"], np.uint8).reshape(t["w_shape"])
    # w_scale / w_zero_point are 1-element 1-D here: the per-channel branch of
    # QLinearConvOp::RunImpl (runtime/ops/quantize.cc:78-84)
    args = (x, t["x_scale"], t["x_zero_point"], w, np.array(t["w_scale"], np.float32),
            np.array(t["w_zero_point"], np.uint8), t["y_scale"], t["y_zero_point"])
    want = np.array(t["y"]).reshape(1, 1, 7, 7)
    np.testing.assert_array_equal(oracle.qlinear_conv_int(*args), want)
    np.testing.assert_array_equal(oracle.qlinear_conv_literal(*args), want)


def test_matmulinteger(oracle, onnx_vectors):
    t = onnx_vectors["test_matmulinteger"]
    y = oracle.matmul_integer(np.array(t["a"], np.uint8), np.array(t["b"], np.uint8),
                              np.array([t["a_zero_point"]], np.uint8), np.array([t["b_zero_point"]], np.uint8))
    assert y.dtype == np.int32 and y.tolist() == t["y"]


@pytest.mark.parametrize("name", ["test_basic_convinteger", "test_convinteger_with_padding"])
def test_convinteger(oracle, onnx_vectors, name):
    t = onnx_vectors[name]
    x = np.array(t["x"], np.uint8).reshape(t["x_shape"])
    w = np.array(t["w"], np.uint8).reshape(t["w_shape"])
    y = oracle.conv_integer(x, w, t["x_zero_point"], None, pads=tuple(t["pads"]))
    assert y.dtype == np.int32 and list(y.shape) == t["y_shape"] and y.reshape(-1).tolist() == t["y"]
