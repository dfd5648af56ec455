"""ONNX reader/writer, the node emitter and the comparison rule of the test driver, without a GPU."""
import importlib
import os
import struct
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import __graft_entry__ as entry  # noqa: E402
import onnx_cases  # noqa: E402


@pytest.fixture(scope="module")
def mods():
    pkg = entry.load_package()
    get = lambda n: importlib.import_module(pkg.__name__ + "." + n)
    return get("onnx_lite"), None, get("chxvm"), get("run_onnx")


def _pb_tensor_class():
    """TensorProto as google.protobuf sees it (field numbers of onnx.proto), proto3 syntax so that
    repeated scalars are written packed."""
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    fd = descriptor_pb2.FileDescriptorProto(name="onnx_min.proto", package="onnx_min", syntax="proto3")
    m = fd.message_type.add(name="TensorProto")
    for name, num, typ, rep in (("dims", 1, F.TYPE_INT64, True), ("data_type", 2, F.TYPE_INT32, False),
                                ("float_data", 4, F.TYPE_FLOAT, True), ("int32_data", 5, F.TYPE_INT32, True),
                                ("int64_data", 7, F.TYPE_INT64, True), ("name", 8, F.TYPE_STRING, False),
                                ("raw_data", 9, F.TYPE_BYTES, False), ("double_data", 10, F.TYPE_DOUBLE, True)):
        m.field.add(name=name, number=num, type=typ, label=F.LABEL_REPEATED if rep else F.LABEL_OPTIONAL)
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    desc = pool.FindMessageTypeByName("onnx_min.TensorProto")
    get = getattr(message_factory, "GetMessageClass", None)
    return get(desc) if get else message_factory.MessageFactory(pool).GetPrototype(desc)


def test_tensor_reader_against_google_protobuf(mods):
    ol = mods[0]
    T = _pb_tensor_class()
    t = T(dims=[2, 3], data_type=ol.FLOAT, float_data=[0.5, -1, 2, 3, 4, 5.25], name="f")       # packed floats
    name, a = ol.parse_tensor(t.SerializeToString())
    assert name == "f" and a.dtype == np.float32 and a.tolist() == [[0.5, -1, 2], [3, 4, 5.25]]
    t = T(dims=[4], data_type=ol.UINT8, int32_data=[0, 3, 128, 255])                              # bytes travel as int32
    assert ol.parse_tensor(t.SerializeToString())[1].tolist() == [0, 3, 128, 255]
    t = T(dims=[3], data_type=ol.INT64, int64_data=[-1, 2 ** 40, 0])
    assert ol.parse_tensor(t.SerializeToString())[1].tolist() == [-1, 2 ** 40, 0]
    t = T(dims=[2, 2], data_type=ol.INT8, raw_data=np.array([-128, -1, 0, 127], np.int8).tobytes())
    assert ol.parse_tensor(t.SerializeToString())[1].tolist() == [[-128, -1], [0, 127]]
    t = T(data_type=ol.FLOAT, float_data=[2.0])                                                    # 0-d
    assert ol.parse_tensor(t.SerializeToString())[1].shape == ()


def test_tensor_writer_against_google_protobuf(mods):
    ol = mods[0]
    T = _pb_tensor_class()
    rng = np.random.default_rng(0)
    for a in (rng.standard_normal((2, 3, 4)).astype(np.float32), rng.integers(0, 256, (5,)).astype(np.uint8),
              np.array(7, np.int32), rng.integers(-9, 9, (2, 2)).astype(np.int64)):
        t = T()
        t.ParseFromString(ol.make_tensor("n", a))
        assert list(t.dims) == list(a.shape) and t.data_type == ol.ONNX_OF[a.dtype] and t.name == "n"
        assert t.raw_data == a.tobytes()
        name, back = ol.parse_tensor(ol.make_tensor("n", a))
        assert name == "n" and back.dtype == a.dtype and np.array_equal(back, a)


def test_model_round_trip(mods, onnx_vectors):
    ol = mods[0]
    for name, (graph, inputs, outputs) in onnx_cases.build_cases(ol, onnx_vectors).items():
        g2 = ol.parse_model(ol.make_model(graph))
        assert [(n.op_type, n.inputs, n.outputs) for n in g2.nodes] == [(n.op_type, n.inputs, n.outputs) for n in graph.nodes]
        assert g2.nodes[0].attrs == graph.nodes[0].attrs
        assert g2.inputs == graph.inputs and g2.outputs == graph.outputs, name
    g = ol.Graph()
    g.nodes.append(ol.Node("QLinearConv", list("abcdefgh"), ["y"],
                           {"strides": [2, 2], "pads": [1, 1, 1, 1], "group": 4, "auto_pad": "SAME_UPPER", "alpha": 0.5}))
    g.initializers["w"] = np.arange(6, dtype=np.int8).reshape(2, 3)
    g2 = ol.parse_model(ol.make_model(g))
    assert g2.nodes[0].attrs == {"strides": [2, 2], "pads": [1, 1, 1, 1], "group": 4, "auto_pad": "SAME_UPPER", "alpha": 0.5}
    assert np.array_equal(g2.initializers["w"], g.initializers["w"])


def _ops_of(vm, serialized):
    """Op names of a serialized program, decoded with the runtime's own reader via a round trip."""
    ol_fields = importlib.import_module(entry.load_package().__name__ + ".onnx_lite").fields
    names = []
    for f, w, v in ol_fields(vm.proto_roundtrip(serialized)):
        if f == 1:
            for f2, w2, v2 in ol_fields(v):
                if f2 == 1:
                    names.append(vm.op_name(v2))
    return names


def test_emitter_instruction_sequences(mods, onnx_vectors):
    ol, _, vm, _ = mods
    vm.runtime()
    cases = onnx_cases.build_cases(ol, onnx_vectors)

    def ops(name):
        return _ops_of(vm, vm.compile_onnx(ol.make_model(cases[name][0])))
    assert ops("test_quantizelinear") == ["In", "In", "In", "QuantizeLinear", "Free", "Free", "Free", "Out"]
    # ReplaceQLinearMatMul: DequantizeLinear x2, MatMul, QuantizeLinear
    assert ops("test_qlinearmatmul_2D") == ["In"] * 8 + ["DequantizeLinear", "DequantizeLinear", "MatMul", "QuantizeLinear",
                                                       "Free", "Free", "Free"] + ["Free"] * 8 + ["Out"]
    assert ops("test_qlinearconv") == ["In"] * 8 + ["QLinearConv"] + ["Free"] * 8 + ["Out"]
    assert ops("test_convinteger_with_padding") == ["In"] * 3 + ["ConvInteger"] + ["Free"] * 3 + ["Out"]


def test_emitter_initializers_and_rejections(mods):
    ol, _, vm, _ = mods
    vm.runtime()
    g = ol.Graph()
    g.inputs = [("x", ol.FLOAT, [1, 4]), ("s", ol.FLOAT, []), ("z", ol.UINT8, [1])]
    g.initializers["s"] = np.array(0.5, np.float32)
    g.initializers["z"] = np.array([3], np.uint8)
    g.nodes.append(ol.Node("QuantizeLinear", ["x", "s", "z"], ["q"]))
    g.nodes.append(ol.Node("Identity", ["q"], ["y"]))
    g.outputs = [("y", ol.UINT8, [1, 4])]
    # one-element initializers read as scale / zero point become scalar constants
    assert _ops_of(vm, vm.compile_onnx(ol.make_model(g))) == [
        "FloatScalarConstant", "IntScalarConstant", "In", "QuantizeLinear", "Free", "Free", "Free", "Identity", "Free", "Out"] or \
        sorted(_ops_of(vm, vm.compile_onnx(ol.make_model(g)))) == sorted(
            ["FloatScalarConstant", "IntScalarConstant", "In", "QuantizeLinear", "Free", "Free", "Free", "Identity", "Free", "Out"])
    bad = ol.Graph()
    bad.inputs = [("x", ol.UINT8, [1, 1, 4, 4]), ("w", ol.UINT8, [1, 1, 3, 3])]
    bad.outputs = [("y", ol.INT32, [1, 1, 2, 2])]
    bad.nodes.append(ol.Node("ConvInteger", ["x", "w"], ["y"], {"pads": [1, 0, 0, 0]}))
    with pytest.raises(vm.ChxVMError, match="beginning and end"):   # simple_node_emitter.cc:76-86
        vm.compile_onnx(ol.make_model(bad))
    bad.nodes[0].attrs = {"dilations": [2, 2]}
    with pytest.raises(vm.ChxVMError, match="Dilation"):
        vm.compile_onnx(ol.make_model(bad))
    bad.nodes[0] = ol.Node("LSTM", ["x", "w"], ["y"])
    with pytest.raises(vm.ChxVMError, match="LSTM"):
        vm.compile_onnx(ol.make_model(bad))


def test_comparison_rule(mods):
    run_onnx = mods[3]
    a = np.array([1.0, 100.0, 0.0], np.float32)
    assert run_onnx.mismatches(a, a.copy(), 1e-4, 1e-6) == 0
    assert run_onnx.mismatches(a + np.array([5e-5, 9e-3, 5e-7], np.float32), a, 1e-4, 1e-6) == 0   # inside atol + rtol*|b|
    assert run_onnx.mismatches(a + np.array([2e-4, 0, 0], np.float32), a, 1e-4, 1e-6) == 1
    assert run_onnx.mismatches(np.array([np.nan], np.float32), np.array([np.nan], np.float32), 1e-4, 1e-6) == 1
    with pytest.raises(ValueError):
        run_onnx.mismatches(a.astype(np.float64), a, 1e-4, 1e-6)       # dtype must match exactly
    with pytest.raises(ValueError):
        run_onnx.mismatches(a.reshape(3, 1), a, 1e-4, 1e-6)            # shape must match exactly
    assert run_onnx.mismatches(np.array([7], np.uint8), np.array([8], np.uint8), 1e-4, 1e-6) == 1


def test_test_directory_layout(mods, onnx_vectors, tmp_path):
    ol, _, _, run_onnx = mods
    cases = onnx_cases.build_cases(ol, onnx_vectors)
    d = onnx_cases.write_case(ol, str(tmp_path), "test_qlinearconv", cases["test_qlinearconv"])
    assert sorted(os.listdir(d)) == ["model.onnx", "test_data_set_0"]
    assert sorted(os.listdir(os.path.join(d, "test_data_set_0"))) == ["input_%d.pb" % i for i in range(8)] + ["output_0.pb"]
    graph, data_sets = run_onnx.load_test_case(d, ol)
    assert graph.nodes[0].op_type == "QLinearConv" and len(data_sets) == 1
    name, inputs, outputs = data_sets[0]
    assert name == "test_data_set_0" and len(inputs) == 8 and outputs[0].shape == (1, 1, 7, 7)
    assert inputs[0].dtype == np.uint8 and inputs[1].dtype == np.float32 and inputs[1].shape == ()
