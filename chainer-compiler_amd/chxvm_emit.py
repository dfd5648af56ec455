"""ONNX graph -> ChxVM program for the node types of the quantized-inference path, the way the
reference lowers them:

  QuantizeLinear / DequantizeLinear / QLinearConv / ConvInteger / MatMulInteger
      one instruction each, operand order and optional operands as
      compiler/chxvm/simple_node_emitter.cc:640-680; pads must be symmetric and are halved,
      auto_pad NOTSET -> "" and otherwise only SAME_UPPER (:76-100); dilations must be 1
  QLinearMatMul
      DequantizeLinear, DequantizeLinear, MatMul, QuantizeLinear (ReplaceQLinearMatMul,
      compiler/simplifier.cc:675-694); the VM fuses the four back into one quantized product
  Identity
      one Identity instruction
  graph inputs / initializers / outputs
      In / constant instructions / Out; a 0-d or 1-element initializer used as a scale or zero
      point becomes a scalar constant, as the emitter's constant folding does

Anything else raises UnsupportedNode: this is the emitter of one backend path, not a compiler.
"""
import numpy as np

from . import chxvm, onnx_lite


class UnsupportedNode(ValueError):
    pass


_DTYPE_NAME = {onnx_lite.FLOAT: "float32", onnx_lite.UINT8: "uint8", onnx_lite.INT8: "int8", onnx_lite.INT32: "int32",
               onnx_lite.INT64: "int64", onnx_lite.BOOL: "bool", onnx_lite.DOUBLE: "float64"}

# positions of scalar operands (scale / zero point read through StrictScalar) per node type
_SCALAR_OPERANDS = {"QuantizeLinear": (1, 2), "DequantizeLinear": (1, 2), "QLinearConv": (1, 2, 6, 7),
                    "QLinearMatMul": (1, 2, 4, 5, 6, 7), "ConvInteger": (2,)}


def _conv_attrs(node, nd):
    for d in node.attrs.get("dilations", []):
        if d != 1:
            raise UnsupportedNode("Dilation is not supported yet")
    pads = list(node.attrs.get("pads", []))
    if len(pads) % 2:
        raise UnsupportedNode("pads must list begin and end values")
    half = len(pads) // 2
    if pads[:half] != pads[half:]:
        raise UnsupportedNode("paddings for beginning and end must be the same: %s" % pads)
    auto_pad = node.attrs.get("auto_pad", "NOTSET")
    if auto_pad == "NOTSET":
        auto_pad = ""
    elif auto_pad != "SAME_UPPER":
        raise UnsupportedNode("auto_pad %s is not supported" % auto_pad)
    return list(node.attrs.get("strides", [])), pads[:half], int(node.attrs.get("group", 1)), auto_pad


def emit_program(graph):
    """Returns (serialized ChxVMProgramProto, input names, output names)."""
    b = chxvm.ProgramBuilder()
    slot = {}
    scalar_uses = set()
    for n in graph.nodes:
        for pos in _SCALAR_OPERANDS.get(n.op_type, ()):
            if pos < len(n.inputs) and n.inputs[pos]:
                scalar_uses.add(n.inputs[pos])
    input_names = []
    for name, elem, shape in graph.inputs:
        if name in graph.initializers:
            continue
        slot[name] = b.input(name, _DTYPE_NAME.get(elem, "float32"), [d if d > 0 else -1 for d in shape])
        input_names.append(name)
    for name, a in graph.initializers.items():
        if name in scalar_uses and a.size == 1:
            slot[name] = b.scalar(a.reshape(()).item(), str(a.dtype))
        else:
            slot[name] = b.constant(a)

    def operand(node, i, optional=False):
        if i >= len(node.inputs) or node.inputs[i] == "":
            if optional:
                return None
            raise UnsupportedNode("%s: missing input %d" % (node.op_type, i))
        return slot[node.inputs[i]]

    for n in graph.nodes:
        t, nin = n.op_type, len(n.inputs)
        dbg = "%s(%s)" % (t, n.name or ",".join(n.outputs))
        if len(n.outputs) != 1:
            raise UnsupportedNode("%s with %d outputs" % (t, len(n.outputs)))
        if t == "QuantizeLinear" and 2 <= nin <= 3:
            y = b.QuantizeLinear(operand(n, 0), operand(n, 1), operand(n, 2, True), debug_info=dbg)
        elif t == "DequantizeLinear" and 2 <= nin <= 3:
            y = b.DequantizeLinear(operand(n, 0), operand(n, 1), operand(n, 2, True), debug_info=dbg)
        elif t == "QLinearConv" and 8 <= nin <= 9:
            strides, pads, group, auto_pad = _conv_attrs(n, 2)
            y = b.QLinearConv(*([operand(n, i) for i in range(8)] + [operand(n, 8, True), strides, pads, group, auto_pad]),
                              debug_info=dbg)
        elif t == "ConvInteger" and 2 <= nin <= 4:
            strides, pads, group, auto_pad = _conv_attrs(n, 2)
            y = b.ConvInteger(operand(n, 0), operand(n, 1), operand(n, 2, True), operand(n, 3, True), strides, pads, group,
                              auto_pad, debug_info=dbg)
        elif t == "MatMulInteger" and 2 <= nin <= 4:
            y = b.MatMulInteger(operand(n, 0), operand(n, 1), operand(n, 2, True), operand(n, 3, True), debug_info=dbg)
        elif t == "QLinearMatMul" and nin == 8:
            a_dl = b.DequantizeLinear(operand(n, 0), operand(n, 1), operand(n, 2), debug_info=dbg)
            b_dl = b.DequantizeLinear(operand(n, 3), operand(n, 4), operand(n, 5), debug_info=dbg)
            mm = b.MatMul(a_dl, b_dl, debug_info=dbg)
            y = b.QuantizeLinear(mm, operand(n, 6), operand(n, 7), debug_info=dbg)
            for tmp in (a_dl, b_dl, mm):
                b.Free(tmp)
        elif t == "Identity" and nin == 1:
            y = b.new_slot()
            b.add("Identity", operand(n, 0), outputs=[y], debug_info=dbg)
        else:
            raise UnsupportedNode("node type %s (%d inputs) is not on the quantized-inference path" % (t, nin))
        slot[n.outputs[0]] = y
    output_names = [name for name, _, _ in graph.outputs]
    for name in output_names:
        b.output(name, slot[name])
    return b.serialize(), input_names, output_names
