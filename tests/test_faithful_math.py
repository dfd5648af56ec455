"""Host build of chainer-compiler_amd/csrc/faithful_math.h against the C library's
expf / expm1f / tanhf, and 1/(1+expf(-x)), over fp32 bit patterns: all 2^32 of them
when 8 or more cores are available (about 20 s), every 16th otherwise.
The device build of the same header is compared with the C library in
tests/test_gpu_elementwise.py."""
import os
import subprocess

import __graft_entry__ as entry


def test_faithful_math_matches_libm(tmp_path):
    exe = str(tmp_path / "fm_check")
    src = os.path.join(entry.ROOT, "tests", "cpu_checks", "faithful_math_check.cc")
    inc = os.path.join(entry.PKG_DIR, "csrc")
    subprocess.check_call(["g++", "-O2", "-fopenmp", "-ffp-contract=off", "-mfma", "-I", inc, src, "-o", exe])
    stride = os.environ.get("CHX_FM_STRIDE") or ("1" if (os.cpu_count() or 1) >= 8 else "16")
    r = subprocess.run([exe, stride], capture_output=True, text=True)
    print(r.stdout)
    assert r.returncode == 0, r.stdout
    lines = dict(l.split(" mismatches: ") for l in r.stdout.splitlines() if " mismatches: " in l)
    assert lines["tanhf "].startswith("0 ")
    assert lines["expm1f"].strip() == "0"
    # exactly one of the two expf operation groupings is the host's; the library probes which
    fma, plain = int(lines["expf   fma-variant"].split()[0]), int(lines["expf   plain-variant"])
    assert min(fma, plain) == 0
