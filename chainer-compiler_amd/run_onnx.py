"""run_onnx for the hip backend: runs the test case of one directory through the C++ ChxVM and
checks the outputs the way tools/run_onnx.cc does.

  python -m chainer_compiler_amd.run_onnx --test DIR [--rtol 1e-4] [--atol 1e-6] [--iterations N]
         [--trace] [--backend hip] [--quantize] [--no_fuse_operations] [--out_onnx FILE] [--out_chxvm FILE]
         [--dump_chxvm] [--compile_only] [--skip_runtime_type_check] [--no_check_values] [--equal_nan]
         [--check_nans] [--check_infs] [--chrome_tracing FILE] [--dump_outputs_dir DIR] [--report_json FILE]

DIR/model.onnx goes through the compiler side of the runtime library (quantizer when --quantize is
given, fusion-group formation, ChxVM emitter: chxvm.compile_onnx); every DIR/test_data_set_N
supplies input_i.pb and output_i.pb in graph order.  An output passes when dtype and shape are equal and every element
has |a - b| <= atol + rtol * |b| (tools/util.cc:89-121; the defaults are run_onnx.cc:299-300).
Exit status 0 when every data set passes.  (From a checkout, where the package directory is
not importable by name, use `python chainer-compiler_amd/run_onnx.py ...`.)
"""
import argparse
import glob
import os
import sys
import time

import numpy as np


def _package():
    here = os.path.dirname(os.path.abspath(__file__))
    root = os.path.dirname(here)
    if root not in sys.path:
        sys.path.insert(0, root)
    import __graft_entry__ as entry
    return entry.load_package()


def load_test_case(test_dir, onnx_lite):
    graph = onnx_lite.parse_model(open(os.path.join(test_dir, "model.onnx"), "rb").read())
    data_sets = []
    for d in sorted(glob.glob(os.path.join(test_dir, "test_data_set_*"))):
        def read(prefix):
            out = []
            i = 0
            while os.path.exists(os.path.join(d, "%s_%d.pb" % (prefix, i))):
                out.append(onnx_lite.parse_tensor(open(os.path.join(d, "%s_%d.pb" % (prefix, i)), "rb").read())[1])
                i += 1
            return out
        data_sets.append((os.path.basename(d), read("input"), read("output")))
    return graph, data_sets


def mismatches(got, want, rtol, atol, equal_nan=False):
    """Number of elements outside the tolerance; raises on a dtype or shape difference.  A NaN
    never matches, unless equal_nan and both sides hold one (--equal_nan of tools/run_onnx.cc)."""
    if got.shape != want.shape:
        raise ValueError("Cannot compare Arrays of different shapes: %s, %s" % (got.shape, want.shape))
    if got.dtype != want.dtype:
        raise ValueError("Cannot compare Arrays of different Dtypes: %s, %s" % (got.dtype, want.dtype))
    a, b = got.astype(np.float64), want.astype(np.float64)
    with np.errstate(invalid="ignore"):
        bad = np.isnan(a) | np.isnan(b) | (np.abs(a - b) > atol + rtol * np.abs(b))
    if equal_nan:
        bad &= ~(np.isnan(a) & np.isnan(b))
    return int(bad.sum())


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--test", required=True, help="test directory")
    ap.add_argument("--backend", default="hip", choices=["hip"])
    ap.add_argument("--rtol", type=float, default=1e-4)
    ap.add_argument("--atol", type=float, default=1e-6)
    ap.add_argument("--iterations", type=int, default=1)
    ap.add_argument("--trace", action="store_true")
    ap.add_argument("--quantize", action="store_true",
                    help="run the quantizer pass in its default mode (dynamic parameters, integer ops), as the reference's flag does")
    ap.add_argument("--no_fuse_operations", action="store_true", help="no fusion groups: every node an instruction of its own")
    ap.add_argument("--out_onnx", "--dump_onnx", dest="dump_onnx", default="", help="write the graph after the passes to this file")
    ap.add_argument("--out_chxvm", default="", help="write the serialized ChxVM program to this file")
    ap.add_argument("--dump_chxvm", action="store_true", help="print the program, one instruction per line")
    ap.add_argument("--compile_only", action="store_true", help="exit after compilation")
    ap.add_argument("--no_check_values", action="store_true", help="run, but do not compare the outputs")
    ap.add_argument("--equal_nan", action="store_true", help="treat NaN as equal to NaN")
    ap.add_argument("--chrome_tracing", default="", help="write a per-instruction timeline (Chrome tracing format) of the last run")
    ap.add_argument("--dump_outputs_dir", default="", help="write every named array output of every instruction there as .npy")
    ap.add_argument("--skip_runtime_type_check", action="store_true",
                    help="do not check dtype and shape of the inputs and of every typed result (checked by default, as in the reference)")
    ap.add_argument("--dump_memory_usage", type=int, default=0, choices=[0, 1, 2], help="1: peak memory held by the variables, 2: after every instruction too")
    ap.add_argument("--check_nans", action="store_true", help="check for NaNs after each operation")
    ap.add_argument("--check_infs", action="store_true", help="check for infinities after each operation")
    ap.add_argument("--report_json", default="", help="write {\"elapsed_times\": [msec, ...]} (the first of several runs dropped)")
    ap.add_argument("--verbose", action="store_true")
    args = ap.parse_args(argv)

    pkg = _package()
    import importlib
    import torch
    onnx_lite = importlib.import_module(pkg.__name__ + ".onnx_lite")
    vm = importlib.import_module(pkg.__name__ + ".chxvm")
    pkg.capi.init(0)

    graph, data_sets = load_test_case(args.test, onnx_lite)
    if not data_sets:
        print("%s: no test_data_set_* directories" % args.test, file=sys.stderr)
        return 2
    model_bytes = open(os.path.join(args.test, "model.onnx"), "rb").read()
    options = {"fuse": "none" if args.no_fuse_operations else "hip"}
    if args.quantize:
        options["quantize"] = {}
    if args.dump_onnx:
        open(args.dump_onnx, "wb").write(vm.transform_onnx(model_bytes, options)[0])
    input_names = [name for name, _, _ in graph.inputs if name not in graph.initializers]
    output_names = [name for name, _, _ in graph.outputs]
    serialized = vm.compile_onnx(model_bytes, options)
    if args.out_chxvm:
        open(args.out_chxvm, "wb").write(serialized)
    if args.dump_chxvm:
        for i, (op, operands, outputs) in enumerate(vm.decode_program(serialized)):
            print("%4d: %s(%s)%s" % (i, op, ", ".join(str(o) for o in operands),
                                    " -> " + ", ".join("$%d" % o for o in outputs) if outputs else ""))
    if args.compile_only:
        return 0
    program = vm.Program(serialized)
    if args.dump_outputs_dir:
        os.makedirs(args.dump_outputs_dir, exist_ok=True)
    vm.set_option("chrome_tracing", args.chrome_tracing)
    vm.set_option("dump_outputs_dir", args.dump_outputs_dir)
    vm.set_option("check_nans", "on" if args.check_nans else "off")
    vm.set_option("check_types", "off" if args.skip_runtime_type_check else "on")
    vm.set_option("dump_memory_usage", str(args.dump_memory_usage))
    vm.set_option("check_infs", "on" if args.check_infs else "off")
    failed = 0
    elapsed_times = []
    for name, inputs, wants in data_sets:
        if len(inputs) != len(input_names) or len(wants) != len(output_names):
            print("%s: %d inputs / %d outputs on disk, the graph has %d / %d" % (
                name, len(inputs), len(wants), len(input_names), len(output_names)), file=sys.stderr)
            return 2
        feed = {n: torch.from_numpy(np.array(a, order="C")).cuda() for n, a in zip(input_names, inputs)}
        elapsed = []
        for _ in range(max(1, args.iterations)):
            t0 = time.perf_counter()
            outs = program.run(feed, trace_level=1 if args.trace else 0)
            elapsed.append(time.perf_counter() - t0)
        for n, want in zip(output_names, wants):
            if args.no_check_values:
                continue
            bad = mismatches(outs[n], want, args.rtol, args.atol, args.equal_nan)
            if bad:
                failed += 1
                print("FAIL %s/%s: %d of %d elements differ (rtol %g atol %g)" % (name, n, bad, want.size, args.rtol,
                                                                                args.atol), file=sys.stderr)
            elif args.verbose:
                print("OK   %s/%s %s %s" % (name, n, want.dtype, want.shape))
        elapsed_times += [1e3 * t for t in (elapsed[1:] if len(elapsed) > 1 else elapsed)]
        if args.iterations > 1:
            rest = elapsed[1:]   # the first run is discarded, as run_onnx.cc does
            print("%s: average %.3f ms, best %.3f ms over %d runs" % (name, 1e3 * sum(rest) / len(rest), 1e3 * min(rest),
                                                                    len(rest)))
    program.close()
    vm.set_option("chrome_tracing", "")
    vm.set_option("dump_outputs_dir", "")
    vm.set_option("check_nans", "off")
    vm.set_option("check_infs", "off")
    vm.set_option("check_types", "off")
    vm.set_option("dump_memory_usage", "0")
    if args.report_json:
        import json
        with open(args.report_json, "w") as f:   # tools/run_onnx.cc:493-498
            json.dump({"elapsed_times": elapsed_times}, f)
    print("%s: %s" % (args.test, "FAILED" if failed else "OK"))
    return 1 if failed else 0


if __name__ == "__main__":
    sys.exit(main())
