"""Writes tests/golden/chxvm_boundary.json: two facts about the ChxVM op boundary, taken from
the TEXT of files of the chainer-compiler tree (nothing is imported or executed):

  "runimpl": for the ops of the quantized-inference path, the return type and the parameter
      types (names dropped, whitespace normalised) of the hand-written `XxxOp::RunImpl`
      definitions in runtime/ops/{quantize,nvrtc,creation,generic}.cc -- what a generator of
      the op classes has to declare for those bodies to compile;
  "proto": the messages of runtime/chxvm.proto.tmpl: per message the fields as
      [name, number, label, type], and the values of ChxVMValueProto.Type.

Run in the build container only:  python tests/golden/make_chxvm_boundary.py /root/reference
"""
import json
import os
import re
import sys

OPS = ["QuantizeLinear", "DequantizeLinear", "QLinearConv", "MatMulInteger", "ConvInteger", "ElementWiseNvrtc",
       "IntScalarConstant", "FloatScalarConstant", "IntConstant", "FloatConstant", "In", "Out", "Free", "Identity",
       "NullConstant"]
FILES = ["quantize.cc", "nvrtc.cc", "creation.cc", "generic.cc"]


def split_params(text):
    parts, depth, cur = [], 0, ""
    for ch in text:
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        if ch == "," and depth == 0:
            parts.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        parts.append(cur)
    return parts


def param_type(p):
    p = " ".join(p.split())
    m = re.match(r"^(.*?[&*>\w])\s+(\w+)$", p)   # "<type> <name>"
    typ = m.group(1) if m and not p.endswith("*") else p
    return typ.replace(" &", "&").replace(" *", "*").replace("chainer_compiler::runtime::", "")


def runimpl_table(ref_root):
    table = {}
    for fn in FILES:
        text = open(os.path.join(ref_root, "runtime", "ops", fn)).read()
        for m in re.finditer(r"^([\w:<>, ]+?)\s+(\w+)Op::RunImpl\(([^)]*)\)\s*\{", text, flags=re.M | re.S):
            ret, op, params = m.group(1), m.group(2), m.group(3)
            if op in OPS:
                table[op] = {"returns": " ".join(ret.split()), "params": [param_type(p) for p in split_params(params)]}
    missing = [o for o in OPS if o not in table]
    assert not missing, missing
    return table


def proto_schema(ref_root):
    text = open(os.path.join(ref_root, "runtime", "chxvm.proto.tmpl")).read()
    text = re.sub(r"//[^\n]*", "", text)
    messages = {}
    for m in re.finditer(r"message (\w+) \{(.*?)\n\}", text, flags=re.S):
        name, body = m.group(1), m.group(2)
        body_no_enum = re.sub(r"enum \w+ \{.*?\}", "", body, flags=re.S)
        fields = [[f.group(3), int(f.group(4)), f.group(1), f.group(2)]
                  for f in re.finditer(r"(required|optional|repeated)\s+(\w+)\s+(\w+)\s*=\s*(\d+)\s*;", body_no_enum)]
        messages[name] = fields
    enum = re.search(r"enum Type \{(.*?)\}", text, flags=re.S).group(1)
    value_types = {k: int(v) for k, v in re.findall(r"(\w+)\s*=\s*(\d+)\s*;", enum)}
    assert re.search(r"^syntax = \"proto2\";", text, flags=re.M)
    package = re.search(r"^package ([\w.]+);", text, flags=re.M).group(1)
    return {"syntax": "proto2", "package": package, "messages": messages, "value_types": value_types}


def main(ref_root):
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "chxvm_boundary.json")
    data = {"runimpl": runimpl_table(ref_root), "proto": proto_schema(ref_root)}
    with open(out, "w") as f:
        json.dump(data, f, indent=1, sort_keys=True)
    print("wrote", out)
    for op, sig in data["runimpl"].items():
        print(" ", sig["returns"], op, sig["params"])


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
