"""The ChxVM boundary without a GPU: op numbering, generated RunImpl prototypes, the protobuf
wire format, BackendConfig, and the program builder -- each against facts taken from the text
of the chainer-compiler tree (tests/golden/chxvm_op_enum.json, chxvm_boundary.json) or against
google.protobuf as an independent implementation of the wire format."""
import json
import os
import random
import re
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
RUNTIME_DIR = os.path.join(ROOT, "chainer-compiler_amd", "runtime")

sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402


@pytest.fixture(scope="module")
def chxvm():
    pkg = entry.load_package()
    from importlib import import_module
    mod = import_module(pkg.__name__ + ".chxvm")
    if not os.path.exists(mod.RUNTIME_LIB):
        entry.build()
    mod.runtime()
    return mod


@pytest.fixture(scope="module")
def op_enum():
    return json.load(open(os.path.join(HERE, "golden", "chxvm_op_enum.json")))


@pytest.fixture(scope="module")
def boundary():
    return json.load(open(os.path.join(HERE, "golden", "chxvm_boundary.json")))


@pytest.fixture(scope="module")
def generated(tmp_path_factory):
    out = tmp_path_factory.mktemp("gen")
    subprocess.check_call([sys.executable, os.path.join(RUNTIME_DIR, "gen_chxvm_hip.py"), "--idl",
                           os.path.join(RUNTIME_DIR, "chxvm_ops.idl"), "--configs", os.path.join(RUNTIME_DIR, "configs"),
                           "--out", str(out)])
    return out


# ---- op numbering -----------------------------------------------------------------------------

def test_runtime_exports(chxvm):
    rt = chxvm.runtime()
    for name in chxvm.RUNTIME_EXPORTS:
        assert hasattr(rt, name), name


def test_op_table_order_matches_reference(chxvm, op_enum):
    table = [name for name, _, _ in chxvm.read_op_table()]
    assert table == op_enum["order"]


def test_op_numbers_in_library(chxvm, op_enum):
    assert chxvm.num_ops() == len(op_enum["order"])
    for name, number in op_enum["number"].items():
        assert chxvm.op_number(name) == number
        assert chxvm.op_name(number) == name
    assert chxvm.op_number("NoSuchOp") == -1
    assert chxvm.op_name(0) == "?" and chxvm.op_name(len(op_enum["order"]) + 1) == "?"


def test_generated_proto_enum(generated, op_enum):
    text = open(os.path.join(generated, "chxvm.proto")).read()
    body = re.search(r"enum Op \{(.*?)\}", text, flags=re.S).group(1)
    pairs = re.findall(r"(\w+) = (\d+);", body)
    assert [(n, int(v)) for n, v in pairs] == [(n, i + 1) for i, n in enumerate(op_enum["order"])]


# ---- prototypes -------------------------------------------------------------------------------

def _split_params(text):
    parts, depth, cur = [], 0, ""
    for ch in text:
        depth += ch == "<"
        depth -= ch == ">"
        if ch == "," and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += ch
    return [p for p in parts + [cur] if p.strip()]


def test_runimpl_prototypes_match_reference_definitions(generated, boundary):
    protos = {}
    for line in open(os.path.join(generated, "runimpl_prototypes.txt")):
        m = re.match(r"^(.*?)\s+(\w+)Op::RunImpl\((.*)\);$", line.strip())
        types = []
        for p in _split_params(m.group(3)):
            p = p.strip()
            types.append(re.match(r"^(.*[&*>])\s*\w+$", p).group(1).strip())
        protos[m.group(2)] = {"returns": m.group(1), "params": types}
    for op, want in boundary["runimpl"].items():
        assert protos[op] == want, op


def test_generated_members_follow_storage_rules(generated):
    """Field operands become members: Ints as StackVector<int64_t, kMaxNdim>, Int as int, String
    as std::string; slot operands are stored as ints (runtime/gen_chxvm.py:111-118)."""
    header = open(os.path.join(generated, "gen_chxvm_ops.h")).read()
    cls = re.search(r"class QLinearConvOp : public ChxVMOp \{(.*?)\n\};", header, flags=re.S).group(1)
    assert "chainerx::StackVector<int64_t, chainerx::kMaxNdim> strides;" in cls
    assert "chainerx::StackVector<int64_t, chainerx::kMaxNdim> pads;" in cls
    assert "int group;" in cls and "std::string auto_pad;" in cls
    assert "int x_scale;" in cls and "int b;" in cls and "int y;" in cls
    cls = re.search(r"class ElementWiseNvrtcOp : public ChxVMOp \{(.*?)\n\};", header, flags=re.S).group(1)
    for member in ("std::vector<int> inputs;", "int num_outputs;", "std::string code;", "int fusion_id;",
                   "std::vector<int> outputs;"):
        assert member in cls


def test_generated_run_glue_has_null_skip_and_trace(generated):
    src = open(os.path.join(generated, "gen_chxvm_ops.cc")).read()
    body = re.search(r"void QuantizeLinearOp::Run\(ChxVMState\* st\) \{(.*?)\n\}\n", src, flags=re.S).group(1)
    assert "trace_level" in body and "IsNull()" in body
    assert "st->SetArray(y, RunImpl(st, st->GetArray(x), st->GetScalar(y_scale), st->GetOptionalScalar(y_zero_point)))" in \
        body.replace("\n", " ").replace("  ", " ") or "RunImpl(st, st->GetArray(x)" in body
    assert "MakeChxVMOp" in src and "case 139:" in src or "QuantizeLinearOp(inst)" in src
    # the trace lines of runtime/gen_chxvm.py:190-236,309-318 and the scans of :321-328, after the call
    flat = body.replace("\n", " ")
    assert '"$" << y << " = " << "QuantizeLinear("' in flat and 'st->GetVarString(x) << " ->"' in flat
    call = flat.index("RunImpl(")
    assert flat.index('st->GetVarString(y) << std::endl', call) < flat.index("st->check_infs()", call) < flat.index("st->check_nans()", call)
    assert "st->CheckInfs({x}, {y});" in flat and "st->CheckNans({x}, {y});" in flat
    lst = re.search(r"void ElementWiseNvrtcOp::Run\(ChxVMState\* st\) \{(.*?)\n\}\n", src, flags=re.S).group(1)
    assert "st->CheckNans({}, outputs);" in lst and "ArrayListToString(inputs)" in lst


# ---- wire format ------------------------------------------------------------------------------

def _pb_classes(boundary, op_enum):
    from google.protobuf import descriptor_pb2, descriptor_pool, message_factory
    F = descriptor_pb2.FieldDescriptorProto
    scalar = {"int32": F.TYPE_INT32, "int64": F.TYPE_INT64, "double": F.TYPE_DOUBLE, "string": F.TYPE_STRING}
    label = {"required": F.LABEL_REQUIRED, "optional": F.LABEL_OPTIONAL, "repeated": F.LABEL_REPEATED}
    schema = boundary["proto"]
    fd = descriptor_pb2.FileDescriptorProto(name="chxvm_test.proto", package=schema["package"], syntax="proto2")
    for mname in ["ChxVMValueProto", "ChxVMTypeProto", "ChxVMInstructionProto", "ChxVMProgramProto"]:
        msg = fd.message_type.add(name=mname)
        if mname == "ChxVMValueProto":
            e = msg.enum_type.add(name="Type")
            for k, v in sorted(schema["value_types"].items(), key=lambda kv: kv[1]):
                e.value.add(name=k, number=v)
        if mname == "ChxVMInstructionProto":
            e = msg.enum_type.add(name="Op")
            for k in op_enum["order"]:
                e.value.add(name=k, number=op_enum["number"][k])
        for fname, number, lab, typ in schema["messages"][mname]:
            f = msg.field.add(name=fname, number=number, label=label[lab])
            if typ in scalar:
                f.type = scalar[typ]
            elif typ in ("Type", "Op"):
                f.type = F.TYPE_ENUM
                f.type_name = ".%s.%s.%s" % (schema["package"], mname, typ)
            else:
                f.type = F.TYPE_MESSAGE
                f.type_name = ".%s.%s" % (schema["package"], typ)
    pool = descriptor_pool.DescriptorPool()
    pool.Add(fd)
    get = getattr(message_factory, "GetMessageClass", None)
    desc = pool.FindMessageTypeByName(schema["package"] + ".ChxVMProgramProto")
    return get(desc) if get else message_factory.MessageFactory(pool).GetPrototype(desc)


def _random_program(Program, op_enum, rng, n_inst):
    prog = Program()
    for _ in range(n_inst):
        inst = prog.instructions.add()
        inst.op = rng.randrange(1, len(op_enum["order"]) + 1)
        for _ in range(rng.randrange(0, 6)):
            v = inst.inputs.add()
            v.type = rng.randrange(1, 17)
            kind = rng.randrange(0, 9)
            if kind == 0:
                v.array = rng.choice([-1, 0, 7, 2 ** 31 - 1])
            elif kind == 1:
                v.i = rng.choice([0, -1, -2 ** 63, 2 ** 63 - 1, 12345678901234])
            elif kind == 2:
                v.f = rng.choice([0.0, -0.0, 1.5, 3.0e-310, -1e300, float("inf")])
            elif kind == 3:
                v.ints.extend(rng.choice([[], [1, 2, 3], [-1, 2 ** 40], [0] * 5]))
            elif kind == 4:
                v.s = rng.choice(["", "SAME_UPPER", "x = Add a b\nout x:float32\n", "é中"])
            elif kind == 5:
                v.array_list.extend(rng.choice([[], [3, -1, 4], [2 ** 31 - 1]]))
            elif kind == 6:
                v.doubles.extend(rng.choice([[], [0.25, -7.0], [1e-320]]))
            elif kind == 7:
                v.strings.extend(rng.choice([[], ["a", ""], ["multi\nline"]]))
            else:
                v.sequence, v.opaque, v.shape, v.scalar = 1, 2, 3, -1
        inst.outputs.extend(rng.choice([[], [5], [1, 2, -1]]))
        if rng.random() < 0.5:
            inst.debug_info = "node %d" % rng.randrange(100)
        if rng.random() < 0.7:
            inst.id = rng.randrange(-5, 2 ** 40)
        for _ in range(rng.randrange(0, 3)):
            t = inst.output_types.add()
            t.dtype = rng.choice([-1, 0, 6, 8])
            t.shape.extend(rng.choice([[], [64, 3, 224, 224], [-1]]))
        inst.output_names.extend(rng.choice([[], ["y"], ["a", "b"]]))
        if rng.random() < 0.3:
            inst.flops = rng.randrange(0, 2 ** 50)
    prog.input_names.extend(["x", "w"][: rng.randrange(0, 3)])
    for _ in range(rng.randrange(0, 3)):
        t = prog.input_types.add()
        t.dtype = 8
        t.shape.extend([1, 2])
    return prog


def test_wire_format_against_google_protobuf(chxvm, boundary, op_enum):
    """google.protobuf writes, the C++ reader parses and the C++ writer re-serializes; the result
    parsed by google.protobuf must equal the original message, field by field."""
    Program = _pb_classes(boundary, op_enum)
    rng = random.Random(7)
    for n_inst in [0, 1, 3, 20]:
        for _ in range(10):
            prog = _random_program(Program, op_enum, rng, n_inst)
            again = Program()
            again.ParseFromString(chxvm.proto_roundtrip(prog.SerializeToString()))
            assert again == prog


def test_wire_format_accepts_packed_repeated_fields(chxvm, boundary, op_enum):
    Program = _pb_classes(boundary, op_enum)
    # ChxVMValueProto{type=INTS, ints packed [1, 300, -1]} written by hand
    packed = b"".join(chxvm._varint(v) for v in [1, 300, -1])
    value = chxvm._f_varint(1, 8) + chxvm._varint((5 << 3) | 2) + chxvm._varint(len(packed)) + packed
    inst = chxvm._f_varint(1, 1) + chxvm._f_bytes(2, value)
    again = Program()
    again.ParseFromString(chxvm.proto_roundtrip(chxvm._f_bytes(1, inst)))
    assert list(again.instructions[0].inputs[0].ints) == [1, 300, -1]


def test_malformed_program_is_rejected(chxvm):
    with pytest.raises(chxvm.ChxVMError):
        chxvm.proto_roundtrip(b"\x0a\x05\x08")           # length runs past the end
    with pytest.raises(chxvm.ChxVMError):
        chxvm.proto_roundtrip(b"\x0a\x02\x10\x01")       # instruction without the required `op`


def test_python_encoder_against_google_protobuf(chxvm, boundary, op_enum):
    Program = _pb_classes(boundary, op_enum)
    b = chxvm.ProgramBuilder()
    x = b.input("x", "float32", (1, 3, 8, 8))
    s = b.scalar(0.05, "float32")
    z = b.scalar(128, "uint8")
    q = b.QuantizeLinear(x, s, z)
    w = b.constant([[[[1, -2], [3, 4]]]] * 4)
    y = b.ConvInteger(q, w, z, None, [2, 2], [], 1, "SAME_UPPER")
    b.output("y", y)
    prog = Program()
    prog.ParseFromString(b.serialize())
    ops = [op_enum["order"][i.op - 1] for i in prog.instructions]
    assert ops == ["In", "FloatScalarConstant", "IntScalarConstant", "QuantizeLinear", "IntConstant", "ConvInteger", "Out"]
    ql = prog.instructions[3]
    assert [v.type for v in ql.inputs] == [1, 14, 14] and [v.array for v in ql.inputs][:1] == [x]
    assert [ql.inputs[1].scalar, ql.inputs[2].scalar] == [s, z] and list(ql.outputs) == [q]
    ci = prog.instructions[5]
    assert ci.inputs[3].array == -1 and list(ci.inputs[4].ints) == [2, 2] and ci.inputs[7].s == "SAME_UPPER"
    assert list(prog.input_names) == ["x"] and prog.input_types[0].dtype == 8
    assert list(prog.input_types[0].shape) == [1, 3, 8, 8]
    assert prog.instructions[1].inputs[0].f == 0.05 and prog.instructions[2].inputs[0].i == 128
    # and the C++ reader agrees with it
    again = Program()
    again.ParseFromString(chxvm.proto_roundtrip(b.serialize()))
    assert again == prog


def test_builder_rejects_unimplemented_and_miscounted_ops(chxvm):
    b = chxvm.ProgramBuilder()
    with pytest.raises(chxvm.ChxVMError):
        b.add("Conv", 1, 2)
    with pytest.raises(chxvm.ChxVMError):
        b.QuantizeLinear(1, 2)


def test_program_with_unimplemented_op_fails_loudly_at_load(chxvm, op_enum):
    inst = chxvm.encode_instruction(op_enum["number"]["Conv"], [("ARRAY", 1)], [2])
    with pytest.raises(chxvm.ChxVMError) as e:
        chxvm.Program(chxvm.encode_program([inst]))
    assert "Conv" in str(e.value)


# ---- BackendConfig (the cases of configs/backend_config_test.cc:9-32) --------------------------

def test_backend_config_chxvm(chxvm):
    config = chxvm.BackendConfig.FromName("chxvm")
    assert config.name == "chxvm"
    assert config.simplify_preproc_count("ReplaceLess") == 0
    assert config.simplify_preproc_count("NOT FOUND") == 0
    assert config.simplify_preproc_count("ReplaceChainerLinear") == 0
    assert config.simplify_preproc_count("ReplaceChainerSelectItem") == 1
    assert config.simplify_count("ReplaceLess") == 1
    assert config.simplify_count("NOT FOUND") == 0
    assert config.simplify_count("ReplaceChainerLinear") == 0
    assert config.simplify_count("ReplaceChainerSelectItem") == 1


def test_backend_config_chxvm_test(chxvm):
    config = chxvm.BackendConfig.FromName("chxvm_test")
    assert config.name == "chxvm_test"
    assert config.simplify_preproc_count("ReplaceLess") == 0
    assert config.simplify_preproc_count("NOT FOUND") == 0
    assert config.simplify_preproc_count("ReplaceChainerLinear") == 1
    assert config.simplify_preproc_count("ReplaceChainerSelectItem") == 0
    assert config.simplify_count("ReplaceLess") == 1
    assert config.simplify_count("NOT FOUND") == 0
    assert config.simplify_count("ReplaceChainerLinear") == 1
    assert config.simplify_count("ReplaceChainerSelectItem") == 0


def test_backend_config_hip_is_chxvm_patched(chxvm):
    hip = chxvm.BackendConfig.FromName("hip")
    assert hip.name == "hip"
    assert hip.simplify_count("ReplaceQLinearMatMul") == 1      # QLinearMatMul is rewritten, never an instruction
    assert hip.simplify_count("ReplaceConstant") == 0           # a false flag is not a member
    for op in ("QuantizeLinear", "DequantizeLinear", "QLinearConv", "ConvInteger", "MatMulInteger", "ChainerFusionGroup"):
        assert hip.HasOp(op)
    assert not hip.HasOp("LSTM")


def test_backend_config_from_json(chxvm):
    c = chxvm.BackendConfig.FromJSON('{"simplify": {"A": true, "B": false}, // comment\n "merge": {"M": true}}')
    assert c.name == "custom"
    assert c.simplify_count("A") == 1 and c.simplify_count("B") == 0 and c.merge_count("M") == 1
    assert c.HasOp("Anything")                                   # no supported_ops section: every op is taken
    patched = chxvm.BackendConfig.FromJSON('{"base": "chxvm", "supported_ops": {"Tanh": null}, "merge": {"MergeX": true}}')
    assert not patched.HasOp("Tanh") and patched.HasOp("Sigmoid")
    assert patched.merge_count("MergeX") == 1 and patched.merge_count("MergePadConv") == 1
    with pytest.raises(chxvm.ChxVMError):
        chxvm.BackendConfig.FromJSON('{"simplify": {"A": 1}}')   # flag values must be bool
    with pytest.raises(chxvm.ChxVMError):
        chxvm.BackendConfig.FromJSON('{"base": 3}')
    with pytest.raises(chxvm.ChxVMError):
        chxvm.BackendConfig.FromName("no_such_backend")


def test_runtime_options(chxvm):
    chxvm.set_option("qlinearconv_bias", "onnx_int32")
    chxvm.set_option("qlinearconv_bias", "reference")
    with pytest.raises(chxvm.ChxVMError, match="qlinearconv_bias"):
        chxvm.set_option("qlinearconv_bias", "int64")
    with pytest.raises(chxvm.ChxVMError, match="unknown option"):
        chxvm.set_option("no_such_switch", "1")
    chxvm.set_option("fuse_residual", "off")
    chxvm.set_option("fuse_residual", "on")
    assert chxvm.counter("qlinearconv_residual_fusions") >= 0 and chxvm.counter("no_such_counter") == -1


def test_whole_network_as_one_program(chxvm):
    """A reduced ResNet converted to one ChxVMProgramProto survives the C++ reader and writer byte
    for byte (loading it uploads its constants, so that part runs with the GPU tests); a pool
    outside the DequantizeLinear -> pool -> QuantizeLinear pattern loads as the float op, unless the
    program wants its backward context, which this backend does not produce."""
    pkg = entry.load_package()
    from importlib import import_module
    wl = import_module(pkg.__name__ + ".workloads")
    ops = import_module(pkg.__name__ + ".ops")
    model = wl.build_resnet50(batch=1, image=32, seed=2, width=16, blocks=(1, 1, 1, 1), classes=4, device="cpu")
    b = wl.program_to_chxvm(model, chxvm, ops)
    data = b.serialize()
    assert chxvm.proto_roundtrip(data) == data
    assert len(b.instructions) > 3 * len(model["program"]) and b.input_names == ["x"]
    lone = chxvm.ProgramBuilder()
    x = lone.input("x", "float32", (1, 1, 4, 4))
    y = lone.new_slot()
    lone.add_raw("AveragePool", [("ARRAY", x), ("INTS", [2, 2]), ("INTS", [2, 2]), ("INTS", [0, 0]), ("INT", 0)], [y, -1])
    lone.output("y", y)
    chxvm.Program(lone.serialize()).close()
    ctx = chxvm.ProgramBuilder()
    x = ctx.input("x", "float32", (1, 1, 4, 4))
    y, c = ctx.new_slot(), ctx.new_slot()
    ctx.add_raw("AveragePool", [("ARRAY", x), ("INTS", [2, 2]), ("INTS", [2, 2]), ("INTS", [0, 0]), ("INT", 0)], [y, c])
    ctx.output("y", y)
    with pytest.raises(chxvm.ChxVMError, match="backward context"):
        chxvm.Program(ctx.serialize())


def test_loader_marks_values_only_convolutions_read(chxvm):
    """Which variables a program's convolutions may keep as code - 128 between them is decided when the program is
    loaded: written by a QLinearConv, read only by QLinearConv without groups and with pads of at most 1 (as input),
    and by nothing else; not a program output."""
    def program(second_pads=(1, 1), second_group=1, extra_reader=False):
        b = chxvm.ProgramBuilder()
        x = b.input("x", "uint8", (1, 16, 8, 8))
        ws = [b.input("w%d" % i, "int8", (16, 16 // (second_group if i == 1 else 1), 3, 3)) for i in range(3)]
        sc, zp = b.input("w_scale", "float32", (16,)), b.input("w_zero_point", "int8", (16,))

        def conv(v, w, pads, group=1):
            return b.QLinearConv(v, b.scalar(0.02, "float32"), b.scalar(3, "uint8"), w, sc, zp, b.scalar(0.05, "float32"),
                                 b.scalar(7, "uint8"), None, [1, 1], list(pads), group, "")
        a = conv(x, ws[0], (1, 1))
        c = conv(a, ws[1], second_pads, second_group)
        d = conv(c, ws[2], (1, 1))
        if extra_reader:
            b.output("a_float", b.DequantizeLinear(a, b.scalar(0.05, "float32"), b.scalar(7, "uint8")))
        b.output("d", d)
        return b.serialize()

    def marked(data):
        prog = chxvm.Program(data)
        n = prog.counter("minus_128_variables")
        prog.close()
        return n
    assert marked(program()) == 2                       # a and c; x is the caller's, d goes back to the caller
    assert marked(program(second_pads=(2, 2))) == 1     # a's reader pads by two rows: a keeps plain codes
    assert marked(program(second_group=2)) == 1         # a grouped reader
    assert marked(program(extra_reader=True)) == 1      # a DequantizeLinear reads a as well
    chxvm.set_option("store_minus_128", "off")
    try:
        assert marked(program()) == 0
    finally:
        chxvm.set_option("store_minus_128", "on")


def test_loader_marks_the_operands_of_absorbed_residual_sums(chxvm):
    """A value that a residual-sum group reads as its other operand stays markable while the group is computed inside
    the convolution before it (the group's own result is then a convolution's result too); with that fusion switched
    off the group is a reader of its own and neither value is marked."""
    import numpy as np
    import torch
    pkg = entry.load_package()
    from importlib import import_module
    ops = import_module(pkg.__name__ + ".ops")
    u8 = torch.uint8

    def scale_bits(v):
        return "0x%08x" % np.float32(v).view(np.uint32)
    code = ops.fusion_program(
        [("a", u8), ("b", u8)],
        [("fa", "DequantizeLinear", "a", scale_bits(0.05), 7), ("fb", "DequantizeLinear", "b", scale_bits(0.05), 7),
         ("s", "Add", "fb", "fa"), ("r", "Relu", "s"), ("q", "QuantizeLinear", "r", scale_bits(0.05), 7, "uint8")], [("q", u8)])

    def marked():
        b = chxvm.ProgramBuilder()
        x = b.input("x", "uint8", (1, 16, 8, 8))
        ws = [b.input("w%d" % i, "int8", (16, 16, 1, 1)) for i in range(3)]
        sc, zp = b.input("w_scale", "float32", (16,)), b.input("w_zero_point", "int8", (16,))

        def conv(v, w):
            return b.QLinearConv(v, b.scalar(0.02, "float32"), b.scalar(3, "uint8"), w, sc, zp, b.scalar(0.05, "float32"),
                                 b.scalar(7, "uint8"), None, [1, 1], [0, 0], 1, "")
        a = conv(x, ws[0])
        y = conv(a, ws[1])
        out = b.ElementWiseNvrtc([y, a], 1, code, 3, num_list_outputs=1)[0]
        b.Free(y)
        b.Free(a)
        b.output("d", conv(out, ws[2]))
        prog = chxvm.Program(b.serialize())
        n = prog.counter("minus_128_variables")
        prog.close()
        return n
    assert marked() == 2            # a (input of a convolution, other operand of the absorbed sum) and the sum
    chxvm.set_option("fuse_residual", "off")
    try:
        assert marked() == 0
    finally:
        chxvm.set_option("fuse_residual", "on")
