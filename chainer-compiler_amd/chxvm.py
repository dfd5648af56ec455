"""Python face of the hip ChxVM runtime (lib/libchxvm_hip_runtime.so).

Three parts, all used by the tests and by hosts that drive the VM from Python:

  * a writer of the ChxVMProgramProto wire format (field numbers of runtime/chxvm.proto.tmpl:1-65
    of the chainer-compiler tree) and `ProgramBuilder`, which plays the part of the generated
    `AddXxxOp(prog, ...)` emitters (compiler/chxvm/gen_chxvm_codegen.py:18-101): operands are
    checked against the op table `runtime/chxvm_ops.idl` and encoded by their declared type;
  * `Program`: load a serialized program into the C++ VM and run it on device tensors;
  * `BackendConfig` queries (configs/backend_config.h of the chainer-compiler tree).
"""
import ctypes
import os
import struct

import numpy as np

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
RUNTIME_LIB = os.path.join(_HERE, "lib", "libchxvm_hip_runtime.so")
IDL_PATH = os.path.join(_HERE, "runtime", "chxvm_ops.idl")

RUNTIME_EXPORTS = [
    "chxvm_last_error", "chxvm_num_ops", "chxvm_op_name", "chxvm_op_number", "chxvm_proto_roundtrip", "chxvm_free",
    "chxvm_program_create", "chxvm_program_destroy", "chxvm_program_num_instructions", "chxvm_program_num_inputs",
    "chxvm_program_input_name", "chxvm_program_run", "chxvm_outputs_count", "chxvm_outputs_name", "chxvm_outputs_get",
    "chxvm_outputs_destroy", "chxvm_backend_config_has", "chxvm_backend_config_name", "chxvm_set_option", "chxvm_counter",
    "chxvm_program_set_option", "chxvm_program_counter", "chxvm_program_capture", "chxvm_replay_launch", "chxvm_replay_synchronize",
    "chxvm_replay_outputs", "chxvm_replay_info", "chxvm_replay_destroy",
    "chxc_compile", "chxc_transform", "chxc_fusion_program", "chxc_quantize_data", "chxc_free",
]

# ChxVMValueProto.Type
VALUE_TYPE = {"ARRAY": 1, "OPTIONAL_ARRAY": 2, "ARRAY_LIST": 3, "SEQUENCE": 4, "OPAQUE": 5, "INT": 6, "FLOAT": 7,
              "INTS": 8, "STRING": 9, "LONGS": 10, "DOUBLES": 11, "INT_VALUES": 12, "SHAPE": 13, "SCALAR": 14,
              "OPTIONAL_SCALAR": 15, "STRINGS": 16}

# IDL operand type -> (Type enum name, encoder)
_SLOT_TYPES = ("Array", "OptionalArray", "ArrayList", "Scalar", "OptionalScalar", "Shape")


class ChxVMError(RuntimeError):
    pass


_rt = None


def runtime():
    """The loaded runtime library; raises when it has not been built (no fallback)."""
    global _rt
    if _rt is None:
        if not os.path.exists(RUNTIME_LIB):
            raise ChxVMError("%s is missing: build it with `make -C chainer-compiler_amd/runtime`" % RUNTIME_LIB)
        capi.lib()  # libchx_hip.so first, so that the dependency resolves to the in-tree build
        rt = ctypes.CDLL(RUNTIME_LIB)
        rt.chxvm_last_error.restype = ctypes.c_char_p
        rt.chxvm_op_name.restype = ctypes.c_char_p
        rt.chxvm_op_name.argtypes = [ctypes.c_int32]
        rt.chxvm_op_number.argtypes = [ctypes.c_char_p]
        rt.chxvm_proto_roundtrip.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p),
                                             ctypes.POINTER(ctypes.c_size_t)]
        rt.chxvm_free.argtypes = [ctypes.c_void_p]
        rt.chxvm_free.restype = None
        rt.chxvm_program_create.argtypes = [ctypes.c_char_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
        rt.chxvm_program_destroy.argtypes = [ctypes.c_void_p]
        rt.chxvm_program_destroy.restype = None
        rt.chxvm_program_num_instructions.argtypes = [ctypes.c_void_p]
        rt.chxvm_program_num_inputs.argtypes = [ctypes.c_void_p]
        rt.chxvm_program_input_name.argtypes = [ctypes.c_void_p, ctypes.c_int32]
        rt.chxvm_program_input_name.restype = ctypes.c_char_p
        rt.chxvm_program_run.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(capi.Tensor),
                                         ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_void_p)]
        rt.chxvm_outputs_count.argtypes = [ctypes.c_void_p]
        rt.chxvm_outputs_name.argtypes = [ctypes.c_void_p, ctypes.c_int32]
        rt.chxvm_outputs_name.restype = ctypes.c_char_p
        rt.chxvm_outputs_get.argtypes = [ctypes.c_void_p, ctypes.c_int32, ctypes.POINTER(capi.Tensor)]
        rt.chxvm_outputs_destroy.argtypes = [ctypes.c_void_p]
        rt.chxvm_outputs_destroy.restype = None
        rt.chxvm_backend_config_has.argtypes = [ctypes.c_char_p, ctypes.c_int32, ctypes.c_char_p, ctypes.c_char_p,
                                                ctypes.POINTER(ctypes.c_int32)]
        rt.chxvm_set_option.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
        rt.chxc_free.argtypes = [ctypes.c_void_p]
        rt.chxc_free.restype = None
        rt.chxvm_counter.argtypes = [ctypes.c_char_p]
        rt.chxvm_counter.restype = ctypes.c_int64
        rt.chxvm_program_set_option.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.c_char_p]
        rt.chxvm_program_counter.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        rt.chxvm_program_counter.restype = ctypes.c_int64
        rt.chxvm_replay_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        rt.chxvm_replay_synchronize.argtypes = [ctypes.c_void_p]
        rt.chxvm_replay_outputs.argtypes = [ctypes.c_void_p]
        rt.chxvm_replay_outputs.restype = ctypes.c_void_p
        rt.chxvm_replay_info.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
        rt.chxvm_replay_info.restype = ctypes.c_int64
        rt.chxvm_replay_destroy.argtypes = [ctypes.c_void_p]
        rt.chxvm_replay_destroy.restype = None
        rt.chxvm_backend_config_name.argtypes = [ctypes.c_char_p, ctypes.c_int32, ctypes.c_char_p, ctypes.c_size_t]
        _rt = rt
    return _rt


def _check(rc):
    if rc != 0:
        raise ChxVMError(runtime().chxvm_last_error().decode("utf-8", "replace"))


# ---------------------------------------------------------------------------------------------
# wire format
# ---------------------------------------------------------------------------------------------

def _varint(v):
    v &= (1 << 64) - 1  # negative int32/int64 values take ten bytes, as protobuf writes them
    out = bytearray()
    while True:
        b = v & 0x7F
        v >>= 7
        if v:
            out.append(b | 0x80)
        else:
            out.append(b)
            return bytes(out)


def _f_varint(field, v):
    return _varint(field << 3) + _varint(v)


def _f_bytes(field, b):
    if isinstance(b, str):
        b = b.encode()
    return _varint((field << 3) | 2) + _varint(len(b)) + b


def _f_double(field, v):
    return _varint((field << 3) | 1) + struct.pack("<d", v)


def encode_value(type_name, v):
    """One ChxVMValueProto (runtime/chxvm.proto.tmpl:1-36)."""
    out = _f_varint(1, VALUE_TYPE[type_name])
    if type_name in ("ARRAY", "OPTIONAL_ARRAY"):
        out += _f_varint(2, v)
    elif type_name == "INT":
        out += _f_varint(3, v)
    elif type_name == "FLOAT":
        out += _f_double(4, v)
    elif type_name in ("INTS", "INT_VALUES", "LONGS"):
        out += b"".join(_f_varint(5, x) for x in v)
    elif type_name == "STRING":
        out += _f_bytes(6, v)
    elif type_name == "ARRAY_LIST":
        out += b"".join(_f_varint(7, x) for x in v)
    elif type_name == "SEQUENCE":
        out += _f_varint(8, v)
    elif type_name == "DOUBLES":
        out += b"".join(_f_double(10, x) for x in v)
    elif type_name == "OPAQUE":
        out += _f_varint(11, v)
    elif type_name == "SHAPE":
        out += _f_varint(12, v)
    elif type_name in ("SCALAR", "OPTIONAL_SCALAR"):
        out += _f_varint(13, v)
    elif type_name == "STRINGS":
        out += b"".join(_f_bytes(14, x) for x in v)
    else:
        raise ValueError(type_name)
    return out


def encode_type(dtype, shape):
    return _f_varint(1, dtype) + b"".join(_f_varint(2, d) for d in shape)


def encode_instruction(op, inputs, outputs, debug_info="", id=0, output_types=(), output_names=(), flops=None):
    """inputs: list of (type_name, value); outputs: list of slot numbers."""
    out = _f_varint(1, op)
    out += b"".join(_f_bytes(2, encode_value(t, v)) for t, v in inputs)
    out += b"".join(_f_varint(3, o) for o in outputs)
    if debug_info:
        out += _f_bytes(4, debug_info)
    out += _f_varint(5, id)
    out += b"".join(_f_bytes(6, encode_type(*t)) for t in output_types)
    out += b"".join(_f_bytes(7, n) for n in output_names)
    if flops is not None:
        out += _f_varint(8, flops)
    return out


def encode_program(instructions, input_names=(), input_types=()):
    out = b"".join(_f_bytes(1, i) for i in instructions)
    out += b"".join(_f_bytes(2, n) for n in input_names)
    out += b"".join(_f_bytes(3, encode_type(*t)) for t in input_types)
    return out


# ---------------------------------------------------------------------------------------------
# op table and program builder
# ---------------------------------------------------------------------------------------------

_IDL_TO_VALUE = {"Array": "ARRAY", "OptionalArray": "ARRAY", "ArrayList": "ARRAY_LIST", "Scalar": "SCALAR",
                 "OptionalScalar": "SCALAR", "Shape": "SHAPE", "Int": "INT", "Float": "FLOAT", "Ints": "INTS",
                 "IntValues": "INT_VALUES", "Doubles": "DOUBLES", "String": "STRING", "Strings": "STRINGS"}


def read_op_table(path=IDL_PATH):
    """[(name, inputs or None, outputs or None)] in op-number order (number = index + 1)."""
    table = []
    for raw in open(path):
        line = raw.split("#")[0].strip()
        if not line:
            continue
        if ":" not in line:
            table.append((line, None, None))
            continue
        head, sig = line.split(":", 1)
        ins, outs = sig.split("->")
        parse = lambda t: [tuple(p.split()) for p in (q.strip() for q in t.split(",")) if p]
        table.append((head.split()[0], parse(ins), parse(outs)))
    return table


# ChainerX dtype numbers (compiler/dtype.h:14-25)
DTYPE = {"bool": 1, "int8": 2, "int16": 3, "int32": 4, "int64": 5, "uint8": 6, "float16": 7, "float32": 8, "float64": 9}


class ProgramBuilder:
    """Assembles a ChxVMProgramProto instruction by instruction.

    `b.QuantizeLinear(x, scale, zp)` appends the instruction and returns the slot number(s) of
    its result(s); slot operands take slot numbers (-1 for an absent optional one), field
    operands take Python values.  `new_slot()` hands out fresh variable ids.
    """

    def __init__(self, table=None):
        self.table = table or read_op_table()
        self.index = {name: (i + 1, ins, outs) for i, (name, ins, outs) in enumerate(self.table)}
        self.instructions = []
        self.input_names = []
        self.input_types = []
        self.next_slot = 1
        self.next_id = 1

    def new_slot(self):
        s = self.next_slot
        self.next_slot += 1
        return s

    def __getattr__(self, name):
        if name.startswith("_") or name not in self.index:
            raise AttributeError(name)
        return lambda *args, **kw: self.add(name, *args, **kw)

    def add(self, name, *args, outputs=None, debug_info="", num_list_outputs=None, output_types=(), output_names=()):
        """output_types: (dtype number, shape) per output, output_names: their names; what a compiler
        declares for the run-time type check and the output dumps."""
        number, ins, outs = self.index[name]
        if ins is None:
            raise ChxVMError("op %s has no signature in the op table of this runtime" % name)
        if len(args) != len(ins):
            raise ChxVMError("%s takes %d operands (%s), got %d" % (name, len(ins), ", ".join(n for _, n in ins), len(args)))
        enc = []
        for (typ, opname), v in zip(ins, args):
            if typ in ("OptionalArray", "OptionalScalar") and v is None:
                v = -1
            if typ in ("Ints", "IntValues", "ArrayList"):
                v = [int(x) for x in v]
            elif typ == "Doubles":
                v = [float(x) for x in v]
            elif typ == "Float":
                v = float(v)
            elif typ not in ("String", "Strings"):
                v = int(v)
            enc.append((_IDL_TO_VALUE[typ], v))
        if outputs is None:
            outputs = []
            for typ, _ in outs:
                if typ == "ArrayList":
                    outputs.append([self.new_slot() for _ in range(num_list_outputs)])
                else:
                    outputs.append(self.new_slot())
        flat = []
        for o in outputs:
            flat.extend(o if isinstance(o, (list, tuple)) else [o])
        self.instructions.append(encode_instruction(number, enc, flat, debug_info=debug_info, id=self.next_id,
                                                    output_types=output_types, output_names=output_names))
        self.next_id += 1
        if not outputs:
            return None
        return outputs[0] if len(outputs) == 1 else tuple(outputs)

    def add_raw(self, name, inputs, outputs, debug_info=""):
        """An instruction of an op that has no signature in this runtime's table (it only exists
        fused with its neighbours): `inputs` is a list of (value type name, value) in the operand
        order of the reference's op table."""
        number = self.index[name][0]
        self.instructions.append(encode_instruction(number, inputs, outputs, debug_info=debug_info, id=self.next_id))
        self.next_id += 1

    # conveniences -----------------------------------------------------------------------
    def input(self, name, dtype="float32", shape=()):
        self.input_names.append(name)
        self.input_types.append((DTYPE[dtype], list(shape)))
        return self.add("In", name)

    def output(self, name, slot):
        self.add("Out", name, slot)

    def scalar(self, value, dtype):
        if dtype.startswith("float"):
            return self.add("FloatScalarConstant", value, DTYPE[dtype], 0)
        return self.add("IntScalarConstant", value, DTYPE[dtype], 0)

    def constant(self, array):
        a = np.asarray(array)
        dt = DTYPE[str(a.dtype)]
        if a.dtype.kind == "f":
            return self.add("FloatConstant", a.ravel().tolist(), dt, a.shape, 0)
        return self.add("IntConstant", a.ravel().tolist(), dt, a.shape, 0)

    def serialize(self):
        return encode_program(self.instructions, self.input_names, self.input_types)


# ---------------------------------------------------------------------------------------------
# running
# ---------------------------------------------------------------------------------------------

_NP_OF_CODE = {1: np.bool_, 2: np.int8, 3: np.int16, 4: np.int32, 5: np.int64, 6: np.uint8, 7: np.float16, 8: np.float32,
               9: np.float64}


def _to_numpy(desc):
    """Host copy of the device array a descriptor names, with its shape and element order."""
    dt = np.dtype(_NP_OF_CODE[desc.dtype])
    nd = desc.ndim
    shape = [desc.shape[i] for i in range(nd)]
    strides = [desc.strides[i] for i in range(nd)]
    span = dt.itemsize + sum((s - 1) * st for s, st in zip(shape, strides)) if all(shape) else 0
    buf = np.empty(max(span, 1), dtype=np.uint8)
    if span:
        capi.check(capi.lib().chx_hip_memcpy_d2h(buf.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(desc.data),
                                                 ctypes.c_size_t(span), None))
    view = np.lib.stride_tricks.as_strided(buf[:dt.itemsize].view(dt), shape=shape, strides=strides) if span else \
        np.empty(shape, dt)
    return np.array(view, order="C")  # a copy that keeps 0-d arrays 0-d (ascontiguousarray would make them 1-d)


class Program:
    """A serialized ChxVMProgramProto loaded into the C++ VM."""

    def __init__(self, serialized):
        self._h = ctypes.c_void_p()
        self.serialized = bytes(serialized)
        _check(runtime().chxvm_program_create(self.serialized, len(self.serialized), ctypes.byref(self._h)))

    @property
    def num_instructions(self):
        return runtime().chxvm_program_num_instructions(self._h)

    @property
    def input_names(self):
        rt = runtime()
        return [rt.chxvm_program_input_name(self._h, i).decode() for i in range(rt.chxvm_program_num_inputs(self._h))]

    def run(self, inputs, trace_level=0):
        """inputs: {name: torch device tensor}.  Returns {name: numpy array}."""
        rt = runtime()
        names = list(inputs)
        c_names = (ctypes.c_char_p * len(names))(*[n.encode() for n in names])
        descs = (capi.Tensor * len(names))(*[capi.desc(inputs[n]) for n in names])
        out = ctypes.c_void_p()
        _check(rt.chxvm_program_run(self._h, c_names, descs, len(names), trace_level, ctypes.byref(out)))
        try:
            result = {}
            for i in range(rt.chxvm_outputs_count(out)):
                d = capi.Tensor()
                _check(rt.chxvm_outputs_get(out, i, ctypes.byref(d)))
                result[rt.chxvm_outputs_name(out, i).decode()] = _to_numpy(d)
            return result
        finally:
            rt.chxvm_outputs_destroy(out)

    def capture(self, inputs):
        """Records one run on the device buffers of `inputs` ({name: torch device tensor}; keep them alive,
        refill them before a launch) and returns the Replay."""
        rt = runtime()
        names = list(inputs)
        c_names = (ctypes.c_char_p * len(names))(*[n.encode() for n in names])
        descs = (capi.Tensor * len(names))(*[capi.desc(inputs[n]) for n in names])
        out = ctypes.c_void_p()
        _check(rt.chxvm_program_capture(self._h, c_names, descs, len(names), ctypes.byref(out)))
        return Replay(out, dict(inputs))

    def set_option(self, name, value):
        """Options of this program, overriding the process-wide ones of set_option():
        "qlinearconv_bias" = "reference" | "onnx_int32" | "default"."""
        _check(runtime().chxvm_program_set_option(self._h, name.encode(), value.encode()))

    def counter(self, name):
        """Event counts of this program over all its runs, e.g. "qlinearconv_residual_fusions"; "minus_128_variables" is
        the number of variables the loader marked to be kept as code - 128 between convolutions."""
        return runtime().chxvm_program_counter(self._h, name.encode())

    def close(self):
        if self._h:
            runtime().chxvm_program_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Replay:
    """A recorded run of a Program (chxvm_program_capture): launch() replays it on a stream."""

    def __init__(self, handle, inputs):
        self._h = handle
        self.inputs = inputs  # keeps the input buffers alive

    def launch(self, stream=None):
        """Enqueues the recorded run; stream: a raw stream pointer (e.g. capi.stream_ptr()), None = the replay's own."""
        _check(runtime().chxvm_replay_launch(self._h, stream))

    def synchronize(self):
        """Waits for launches on the replay's own stream."""
        _check(runtime().chxvm_replay_synchronize(self._h))

    def outputs(self):
        """{name: numpy array} of the last launch; the device must be done with it (synchronize())."""
        rt = runtime()
        out = rt.chxvm_replay_outputs(self._h)
        result = {}
        for i in range(rt.chxvm_outputs_count(out)):
            d = capi.Tensor()
            _check(rt.chxvm_outputs_get(out, i, ctypes.byref(d)))
            result[rt.chxvm_outputs_name(out, i).decode()] = _to_numpy(d)
        return result

    def info(self, name):
        """"pool_bytes", "pool_blocks", "warm_runs"."""
        return runtime().chxvm_replay_info(self._h, name.encode())

    def close(self):
        if self._h:
            runtime().chxvm_replay_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def decode_program(data):
    """[(op name, [(value type name, value)], outputs)] of a serialized program: the listing that
    --dump_chxvm of run_onnx prints."""
    from . import onnx_lite
    names = {v: k for k, v in VALUE_TYPE.items()}
    out = []
    for f, w, v in onnx_lite.fields(data):
        if f != 1:
            continue
        op, ins, outs = None, [], []
        for f2, w2, v2 in onnx_lite.fields(v):
            if f2 == 1:
                op = op_name(v2)
            elif f2 == 2:
                typ, val, lst = None, None, []
                for f3, w3, v3 in onnx_lite.fields(v2):
                    if f3 == 1:
                        typ = names[v3]
                    elif f3 in (2, 3, 8, 11, 12, 13):
                        val = v3 - (1 << 64) if v3 >= 1 << 63 else v3
                    elif f3 == 4:
                        val = np.frombuffer(v3, "<f8")[0]
                    elif f3 == 6:
                        val = bytes(v3).decode()
                    elif f3 in (5, 7):
                        lst.append(v3 - (1 << 64) if v3 >= 1 << 63 else v3)
                    elif f3 == 10:
                        lst.append(float(np.frombuffer(v3, "<f8")[0]))
                ins.append((typ, lst if typ in ("INTS", "INT_VALUES", "ARRAY_LIST", "DOUBLES") else val))
            elif f2 == 3:
                outs.append(v2 - (1 << 64) if v2 >= 1 << 63 else v2)
        out.append((op, ins, outs))
    return out


def set_option(name, value):
    """Runtime switches: "qlinearconv_bias" = "reference" (default) | "onnx_int32";
    "fuse_residual" = "on" (default) | "off" (applies to programs loaded afterwards);
    "pair_convolutions" = "on" (default) | "off": two QLinearConv of one value with the same geometry as one launch
    (applies to programs loaded afterwards);
    "store_minus_128" = "on" (default) | "off": uint8 values that only QLinearConv with pads of at most 1 read are kept as
    code - 128 in int8 arrays between them (applies to programs loaded afterwards);
    "chrome_tracing" = file that every later run writes its per-instruction timeline to, "" = off;
    "dump_outputs_dir" = directory that every later run writes the instructions' named array
    outputs to as .npy files, "" = off;
    "check_nans" / "check_infs" = "on" | "off" (default): every later run scans the results of each
    instruction and fails, naming the instruction's operands and results, at the first NaN / Inf;
    "check_types" = "on" | "off" (default): the inputs are checked against the program's input types
    and every typed result against the dtype and shape its instruction declares;
    "dump_memory_usage" = "0" (default) | "1" (bytes per variable slot and the peak, after the run) |
    "2" (also the bytes held after every instruction)."""
    _check(runtime().chxvm_set_option(name.encode(), value.encode()))


# ---------------------------------------------------------------------------------------------
# compiler side (compiler/compiler_capi.h)
# ---------------------------------------------------------------------------------------------

def _options(options):
    import json
    return json.dumps(options or {}).encode()


def compile_onnx(model_bytes, options=None):
    """ONNX ModelProto bytes -> serialized ChxVMProgramProto, through the quantizer and fusion passes
    that `options` selects (see compiler_capi.h)."""
    rt = runtime()
    out, n = ctypes.c_void_p(), ctypes.c_size_t()
    _check(rt.chxc_compile(bytes(model_bytes), len(model_bytes), _options(options), ctypes.byref(out), ctypes.byref(n)))
    try:
        return ctypes.string_at(out, n.value)
    finally:
        rt.chxc_free(out)


def transform_onnx(model_bytes, options=None):
    """Runs the passes only: (ONNX ModelProto bytes of the rewritten graph, one-line-per-node description)."""
    rt = runtime()
    out, n, desc = ctypes.c_void_p(), ctypes.c_size_t(), ctypes.c_void_p()
    _check(rt.chxc_transform(bytes(model_bytes), len(model_bytes), _options(options), ctypes.byref(out), ctypes.byref(n),
                             ctypes.byref(desc)))
    try:
        return ctypes.string_at(out, n.value), ctypes.string_at(desc).decode()
    finally:
        rt.chxc_free(out)
        rt.chxc_free(desc)


def fusion_program(model_bytes, group, options=None):
    """Program text of fusion group number `group` (1-based) after the passes."""
    rt = runtime()
    text = ctypes.c_void_p()
    _check(rt.chxc_fusion_program(bytes(model_bytes), len(model_bytes), _options(options), int(group), ctypes.byref(text)))
    try:
        return ctypes.string_at(text).decode()
    finally:
        rt.chxc_free(text)


def quantize_data(data, dtype):
    """The weight quantization of the quantizer pass on one float32 array: (codes, scale, zero_point)."""
    a = np.ascontiguousarray(data, dtype=np.float32).ravel()
    codes = np.empty(a.size, np.int32)
    scale, zp = ctypes.c_float(), ctypes.c_int64()
    dt = np.dtype(dtype)
    _check(runtime().chxc_quantize_data(a.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(a.size), DTYPE[str(dt)], ctypes.byref(scale),
                                        ctypes.byref(zp), codes.ctypes.data_as(ctypes.c_void_p)))
    return codes.reshape(np.shape(data)).astype(dt), np.float32(scale.value), zp.value


def counter(name):
    """Process-wide event counts of the runtime, e.g. "qlinearconv_residual_fusions"."""
    return runtime().chxvm_counter(name.encode())


def proto_roundtrip(serialized):
    """Parse with the C++ reader and serialize again with the C++ writer."""
    rt = runtime()
    out = ctypes.c_void_p()
    n = ctypes.c_size_t()
    _check(rt.chxvm_proto_roundtrip(bytes(serialized), len(serialized), ctypes.byref(out), ctypes.byref(n)))
    try:
        return ctypes.string_at(out, n.value)
    finally:
        rt.chxvm_free(out)


def op_name(number):
    return runtime().chxvm_op_name(number).decode()


def op_number(name):
    return runtime().chxvm_op_number(name.encode())


def num_ops():
    return runtime().chxvm_num_ops()


class BackendConfig:
    """BackendConfig.FromName / FromJSON of the C++ runtime."""

    def __init__(self, config, is_json):
        self._config = config.encode()
        self._is_json = 1 if is_json else 0
        buf = ctypes.create_string_buffer(256)
        _check(runtime().chxvm_backend_config_name(self._config, self._is_json, buf, 256))
        self.name = buf.value.decode()

    @classmethod
    def FromName(cls, name):
        return cls(name, False)

    @classmethod
    def FromJSON(cls, text):
        return cls(text, True)

    def _has(self, section, key):
        out = ctypes.c_int32()
        _check(runtime().chxvm_backend_config_has(self._config, self._is_json, section.encode(), key.encode(), ctypes.byref(out)))
        return out.value

    def simplify_preproc_count(self, key):
        return self._has("simplify_preproc", key)

    def simplify_count(self, key):
        return self._has("simplify", key)

    def merge_count(self, key):
        return self._has("merge", key)

    def expanding_functions_count(self, key):
        return self._has("expanding_functions", key)

    def HasOp(self, key):
        return bool(self._has("supported_ops", key))
