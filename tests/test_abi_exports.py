"""The C-ABI library loads and exports every symbol include/chx_hip.h declares.
No compute call is made (there is no GPU in the CPU test run)."""
import os
import re

import pytest

import __graft_entry__ as entry

ROOT = entry.ROOT


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "chx_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(chx_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    pkg = entry.load_package()
    if not os.path.exists(pkg.capi.LIB_PATH):
        entry.build()
    lib = pkg.capi.lib()
    syms = declared_symbols()
    assert len(syms) >= 20
    for s in syms:
        assert hasattr(lib, s), "missing export: " + s
    assert sorted(pkg.capi.EXPORTS) == syms


def test_errors_are_reported_not_aborted():
    pkg = entry.load_package()
    lib = pkg.capi.lib()
    # null descriptor: validation happens before any device call
    rc = lib.chx_hip_quantize_linear(None, pkg.capi.ctypes.c_float(1.0), 0, 0, None, None)
    assert rc == 1
    assert b"null tensor descriptor" in lib.chx_hip_last_error()
    with pytest.raises(pkg.capi.ChxHipError):
        pkg.capi.check(rc)
