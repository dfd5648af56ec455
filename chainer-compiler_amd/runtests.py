"""Test driver in the manner of scripts/runtests.py of the chainer-compiler tree: one run_onnx
subprocess per test directory, a summary, and for every failure the captured output with the
command line that reproduces it.  Every case here needs the GPU, so the cases run one after the
other (the reference runs its CPU cases in parallel first and the GPU cases serially).

  python chainer-compiler_amd/runtests.py DIR_OF_TEST_DIRS [-k REGEX] [--rtol R] [--atol A] [--no_fuse_operations]
         [--show_log] [--verbose] [--failure_log FILE] [--failed]

--failure_log (default DIR_OF_TEST_DIRS/failed_tests.log) receives, per failed case, "=== name ===", the
reproducing command line and the captured output, as scripts/runtests.py:1117-1126 writes it; --failed
runs only the cases that file names (scripts/runtests.py:47-48,1010-1022).
"""
import argparse
import os
import re
import subprocess
import sys
import time

# the quantized-path cases of the reference's node-test list (scripts/runtests.py:556-564,577-582)
NODE_TESTS = ["test_quantizelinear", "test_dequantizelinear", "test_qlinearmatmul_2D", "test_qlinearmatmul_3D",
              "test_qlinearconv", "test_convinteger_with_padding", "test_basic_convinteger", "test_matmulinteger",
              "test_round", "test_dynamicquantizelinear", "test_dynamicquantizelinear_max_adjusted", "test_dynamicquantizelinear_min_adjusted",
              "test_dynamicquantizelinear_expanded", "test_dynamicquantizelinear_max_adjusted_expanded",
              "test_dynamicquantizelinear_min_adjusted_expanded"]


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("root", help="directory holding one sub-directory per test case")
    ap.add_argument("-k", "--filter", default="", help="regular expression searched in the case names")
    ap.add_argument("--rtol", type=float, default=None)
    ap.add_argument("--atol", type=float, default=None)
    ap.add_argument("--timeout", type=float, default=120.0)
    ap.add_argument("--no_fuse_operations", action="store_true", help="passed on to run_onnx")
    ap.add_argument("--show_log", action="store_true", help="print the output of every case, not only of the failed ones")
    ap.add_argument("--verbose", action="store_true", help="passed on to run_onnx")
    ap.add_argument("--failure_log", default=None, help="file that receives the failed cases with their logs")
    ap.add_argument("--failed", action="store_true", help="run only the cases listed in the failure log of the last run")
    args = ap.parse_args(argv)
    here = os.path.dirname(os.path.abspath(__file__))
    failure_log = args.failure_log or os.path.join(args.root, "failed_tests.log")
    pattern = re.compile(args.filter)
    cases = sorted(d for d in os.listdir(args.root)
                   if os.path.exists(os.path.join(args.root, d, "model.onnx")) and pattern.search(d))
    if args.failed:
        if not os.path.exists(failure_log):
            print("%s does not exist" % failure_log, file=sys.stderr)
            return 2
        last = set(m.group(1) for m in re.finditer(r"^=== (\S+) ===$", open(failure_log, encoding="utf-8", errors="replace").read(), flags=re.M))
        cases = [c for c in cases if c in last]
    if not cases:
        print("no test cases under %s" % args.root, file=sys.stderr)
        return 2
    failures = []
    t0 = time.time()
    for i, case in enumerate(cases):
        cmd = [sys.executable, os.path.join(here, "run_onnx.py"), "--test", os.path.join(args.root, case)]
        if args.rtol is not None:
            cmd += ["--rtol", str(args.rtol)]
        if args.atol is not None:
            cmd += ["--atol", str(args.atol)]
        if args.no_fuse_operations:
            cmd.append("--no_fuse_operations")
        if args.verbose:
            cmd.append("--verbose")
        try:
            p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=args.timeout)
            ok, log = p.returncode == 0, p.stdout.decode("utf-8", "replace")
        except subprocess.TimeoutExpired as e:
            ok, log = False, (e.stdout or b"").decode("utf-8", "replace") + "\ntimed out"
        print("[%d/%d] %s %s" % (i + 1, len(cases), "OK  " if ok else "FAIL", case))
        if args.show_log and ok:
            print(log)
        sys.stdout.flush()
        if not ok:
            failures.append((case, cmd, log))
    for case, cmd, log in failures:
        print("=== %s ===\n%s\n$ %s" % (case, log, " ".join(cmd)))
    if failures:
        with open(failure_log, "w", encoding="utf-8") as f:
            for case, cmd, log in failures:
                f.write("=== %s ===\n$ %s\n%s\n" % (case, " ".join(cmd), log))
        print("%d/%d tests failed! (see %s)" % (len(failures), len(cases), failure_log))
    elif os.path.exists(failure_log) and not args.failed:
        os.remove(failure_log)   # a clean run leaves no stale list behind
    print("%d/%d tests passed in %.1f s" % (len(cases) - len(failures), len(cases), time.time() - t0))
    return 1 if failures else 0


if __name__ == "__main__":
    sys.exit(main())
