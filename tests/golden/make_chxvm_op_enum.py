"""Writes tests/golden/chxvm_op_enum.json: the ChxVM op names in the order of the
reference's op table, with the number each gets in chxvm.proto.

The enum is positional: `gen_chxvm_proto` (runtime/gen_chxvm.py:37-47 in the
chainer-compiler tree) numbers the ops 1, 2, 3, ... in the order of CHX_ALL_OPS,
which is the concatenation CHX_OPS, CHX_CUSTOM_FIELD_OPS, CHX_SEQ_OPS,
CHX_SEQ_OPS_UNTYPED, CHX_GENERIC_OPS (runtime/chxvm_defs.py:589-593).  This script
READS runtime/chxvm_defs.py as text (it is neither imported nor executed) and picks the
first string of every tuple that opens an entry of those five lists.

Run in the build container only:  python tests/golden/make_chxvm_op_enum.py /root/reference
"""
import json
import os
import re
import sys

LISTS = ["CHX_OPS", "CHX_CUSTOM_FIELD_OPS", "CHX_SEQ_OPS", "CHX_SEQ_OPS_UNTYPED", "CHX_GENERIC_OPS"]


def list_body(text, name):
    m = re.search(r"^%s = \[\n" % name, text, flags=re.M)
    assert m, name
    end = text.index("\n]\n", m.end())
    return text[m.end():end]


def main(ref_root):
    text = open(os.path.join(ref_root, "runtime", "chxvm_defs.py")).read()
    names = []
    for lst in LISTS:
        body = list_body(text, lst)
        # an entry starts with "    ('Name'," at list indentation
        names += re.findall(r"^    \('([A-Za-z0-9_]+)',", body, flags=re.M)
    assert len(names) == len(set(names)), "duplicate op name"
    table = {n: i + 1 for i, n in enumerate(names)}
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "chxvm_op_enum.json")
    with open(out, "w") as f:
        json.dump({"order": names, "number": table}, f, indent=0)
    print("wrote %s: %d ops; QuantizeLinear=%d ElementWiseNvrtc=%d In=%d" % (
        out, len(names), table["QuantizeLinear"], table["ElementWiseNvrtc"], table["In"]))


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
