"""The reference's quantized-path node tests as ONNX test directories, run by the test driver
(one run_onnx subprocess per directory) through the emitter and the C++ ChxVM on the MI355X."""
import importlib
import os
import subprocess
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_runtests_over_the_node_tests(onnx_vectors, tmp_path):
    import gpu_util
    import onnx_cases
    ol = importlib.import_module(gpu_util.pkg.__name__ + ".onnx_lite")
    driver = importlib.import_module(gpu_util.pkg.__name__ + ".runtests")
    cases = onnx_cases.build_cases(ol, onnx_vectors)
    assert sorted(cases) == sorted(driver.NODE_TESTS)
    for name, case in cases.items():
        onnx_cases.write_case(ol, str(tmp_path), name, case)
    # one more directory whose expected output is wrong by one code: the driver must report it
    g, ins, outs = cases["test_quantizelinear"]
    wrong = outs[0].copy()
    wrong[2] += 1
    onnx_cases.write_case(ol, str(tmp_path), "zz_expected_failure", (g, ins, [wrong]))
    p = subprocess.run([sys.executable, os.path.join(ROOT, "chainer-compiler_amd", "runtests.py"), str(tmp_path)],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=600)
    log = p.stdout.decode()
    print(log)
    assert p.returncode == 1
    for name in cases:
        assert "OK   %s" % name in log
    assert "FAIL zz_expected_failure" in log and "%d/%d tests passed" % (len(cases), len(cases) + 1) in log
    assert "1 of 6 elements differ" in log and "run_onnx.py --test" in log      # failure log + reproducing command
    # the failure log names the failed case with its command and output; --failed reruns only what it lists
    flog = open(os.path.join(str(tmp_path), "failed_tests.log")).read()
    assert flog.startswith("=== zz_expected_failure ===\n$ ") and "1 of 6 elements differ" in flog and "see %s" % os.path.join(str(tmp_path), "failed_tests.log") in log
    again = subprocess.run([sys.executable, os.path.join(ROOT, "chainer-compiler_amd", "runtests.py"), str(tmp_path), "--failed"],
                           stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=300)
    assert again.returncode == 1 and "[1/1] FAIL zz_expected_failure" in again.stdout.decode()
    ok = subprocess.run([sys.executable, os.path.join(ROOT, "chainer-compiler_amd", "runtests.py"), str(tmp_path), "-k", "^test_(round|matmul)",
                         "--show_log", "--verbose", "--no_fuse_operations"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, timeout=300)
    text = ok.stdout.decode()
    assert ok.returncode == 0 and "2/2 tests passed" in text and "OK   test_data_set_0/" in text
    assert not os.path.exists(os.path.join(str(tmp_path), "failed_tests.log"))          # a clean run removes the stale list


def test_run_onnx_in_process_with_iterations(onnx_vectors, tmp_path, capsys):
    import gpu_util
    import onnx_cases
    ol = importlib.import_module(gpu_util.pkg.__name__ + ".onnx_lite")
    run_onnx = importlib.import_module(gpu_util.pkg.__name__ + ".run_onnx")
    cases = onnx_cases.build_cases(ol, onnx_vectors)
    d = onnx_cases.write_case(ol, str(tmp_path), "test_qlinearmatmul_3D", cases["test_qlinearmatmul_3D"])
    assert run_onnx.main(["--test", d, "--iterations", "3", "--verbose"]) == 0
    out = capsys.readouterr().out
    assert "average" in out and "OK   test_data_set_0/y uint8 (2, 2, 3)" in out


def test_run_onnx_parity_tooling(onnx_vectors, tmp_path):
    """--chrome_tracing, --dump_outputs_dir and --report_json of the reference's run_onnx
    (tools/run_onnx.cc:147-149,208-209,493-498): one trace event per executed instruction, every
    named array output as a .npy that numpy reads back, the elapsed times with the warm-up run dropped."""
    import json
    import gpu_util
    import onnx_cases
    ol = importlib.import_module(gpu_util.pkg.__name__ + ".onnx_lite")
    run_onnx = importlib.import_module(gpu_util.pkg.__name__ + ".run_onnx")
    vm = importlib.import_module(gpu_util.pkg.__name__ + ".chxvm")
    cases = onnx_cases.build_cases(ol, onnx_vectors)
    name = "test_dynamicquantizelinear_min_adjusted_expanded"
    d = onnx_cases.write_case(ol, str(tmp_path), name, cases[name])
    trace, dumps, report = str(tmp_path / "trace.json"), str(tmp_path / "dumps"), str(tmp_path / "report.json")
    assert run_onnx.main(["--test", d, "--no_fuse_operations", "--iterations", "3", "--chrome_tracing", trace,
                          "--dump_outputs_dir", dumps, "--report_json", report]) == 0
    events = json.load(open(trace))
    program = vm.compile_onnx(open(os.path.join(d, "model.onnx"), "rb").read(), {"fuse": "none"})
    loaded = vm.Program(program)
    assert len(events) == loaded.num_instructions
    loaded.close()
    names = [e["name"] for e in events]
    assert all(e["ph"] == "X" and e["cat"] == "ChxVM" and e["dur"] >= 0 for e in events)
    assert [e["args"]["pc"] for e in events] == list(range(len(events)))
    for op in ("ReduceMin", "ReduceMax", "Clip", "Round", "Cast", "QuantizeLinear", "In", "Out", "Free"):
        assert op in names
    files = sorted(os.listdir(dumps))
    by_name = {f.split("_", 1)[1][:-4]: np.load(os.path.join(dumps, f)) for f in files}
    graph, inputs, outs = cases[name]
    np.testing.assert_array_equal(by_name["y"], outs[0])
    assert by_name["y"].shape == (3, 4) and by_name["y"].dtype == np.uint8
    assert by_name["Scale"].shape == () and by_name["Scale"] == outs[1]
    assert by_name["Zeropoint"] == outs[2] and by_name["Rounded_ZeroPoint_FP"] == np.float32(0)
    assert all(f[:5].isdigit() for f in files)
    times = json.load(open(report))["elapsed_times"]
    assert len(times) == 2 and all(t > 0 for t in times)


def test_type_checks_and_memory_report(onnx_vectors, tmp_path, capfd):
    """--check_types (runtime/chxvm.cc:38-64,140-158) and --dump_memory_usage (:208-237): every node
    test passes with the checks on (the emitter declares each result's dtype and shape where the
    graph knows them); an input of another shape, or a result that contradicts its declaration, fails."""
    import gpu_util
    import onnx_cases
    ol = importlib.import_module(gpu_util.pkg.__name__ + ".onnx_lite")
    run_onnx = importlib.import_module(gpu_util.pkg.__name__ + ".run_onnx")
    vm = importlib.import_module(gpu_util.pkg.__name__ + ".chxvm")
    cases = onnx_cases.build_cases(ol, onnx_vectors)
    for name in ("test_qlinearconv", "test_dynamicquantizelinear_expanded", "test_qlinearmatmul_3D", "test_convinteger_with_padding"):
        d = onnx_cases.write_case(ol, str(tmp_path), name, cases[name])
        capfd.readouterr()
        assert run_onnx.main(["--test", d, "--check_nans", "--check_infs", "--dump_memory_usage", "2"]) == 0, name   # types: checked by default
        err = capfd.readouterr().err
        import re
        assert "Peak memory usage=" in err and " Memory usage=" in err and re.search(r"^\$\d+: \d+$", err, flags=re.M)   # slots alive at the end
    # a program whose declarations are wrong
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", (3, 5))
    q = b.QuantizeLinear(x, b.scalar(0.5, "float32"), b.scalar(3, "uint8"), output_types=[(vm.DTYPE["uint8"], [3, 5])], output_names=["q"])
    d = b.DequantizeLinear(q, b.scalar(0.5, "float32"), b.scalar(3, "uint8"), output_types=[(vm.DTYPE["float32"], [5, 3])],
                           output_names=["d"], debug_info="the badly declared one")
    b.output("q", q)
    prog = vm.Program(b.serialize())
    xv = np.zeros((3, 5), np.float32)
    try:
        vm.set_option("check_types", "on")
        with pytest.raises(vm.ChxVMError, match="Shape check failed in output #0: the badly declared one"):
            prog.run({"x": gpu_util.dev(xv)})
        with pytest.raises(vm.ChxVMError, match="Input 'x' has an unexpected shape"):
            prog.run({"x": gpu_util.dev(np.zeros((5, 3), np.float32))})
        with pytest.raises(vm.ChxVMError, match="Input 'x' has an unexpected dtype"):
            prog.run({"x": gpu_util.dev(np.zeros((3, 5), np.uint8))})
    finally:
        vm.set_option("check_types", "off")
    assert prog.run({"x": gpu_util.dev(np.zeros((5, 3), np.float32))})["q"].shape == (5, 3)   # unchecked by default, as in the reference
    prog.close()


def test_run_onnx_compile_flags(onnx_vectors, tmp_path, capsys):
    """--compile_only, --out_chxvm, --dump_chxvm, --out_onnx, --no_check_values, --skip_runtime_type_check
    (tools/run_onnx.cc:294-310)."""
    import gpu_util
    import onnx_cases
    ol = importlib.import_module(gpu_util.pkg.__name__ + ".onnx_lite")
    run_onnx = importlib.import_module(gpu_util.pkg.__name__ + ".run_onnx")
    vm = importlib.import_module(gpu_util.pkg.__name__ + ".chxvm")
    cases = onnx_cases.build_cases(ol, onnx_vectors)
    graph, inputs, outputs = cases["test_quantizelinear"]
    d = onnx_cases.write_case(ol, str(tmp_path), "test_quantizelinear", cases["test_quantizelinear"])
    prog_file, onnx_file = str(tmp_path / "p.chxvm"), str(tmp_path / "o.onnx")
    capsys.readouterr()
    assert run_onnx.main(["--test", d, "--compile_only", "--out_chxvm", prog_file, "--dump_chxvm", "--out_onnx", onnx_file]) == 0
    listing = capsys.readouterr().out
    assert "QuantizeLinear(" in listing and "-> $" in listing and "Out(" in listing
    loaded = vm.Program(open(prog_file, "rb").read())            # the file is the program
    out = loaded.run({n: gpu_util.dev(np.array(a, order="C")) for (n, _, _), a in zip(graph.inputs, inputs)})
    np.testing.assert_array_equal(out[graph.outputs[0][0]], outputs[0])
    loaded.close()
    assert [n.op_type for n in ol.parse_model(open(onnx_file, "rb").read()).nodes] == ["QuantizeLinear"]
    # wrong expectations on disk: fails, passes with --no_check_values
    bad = (graph, inputs, [np.array(outputs[0]) ^ 1])
    d2 = onnx_cases.write_case(ol, str(tmp_path / "bad"), "test_quantizelinear", bad)
    assert run_onnx.main(["--test", d2]) == 1
    assert run_onnx.main(["--test", d2, "--no_check_values", "--skip_runtime_type_check"]) == 0
    assert run_onnx.mismatches(np.array([np.nan, 1.0], np.float32), np.array([np.nan, 1.0], np.float32), 1e-4, 1e-6, equal_nan=True) == 0
    assert run_onnx.mismatches(np.array([np.nan, 1.0], np.float32), np.array([2.0, 1.0], np.float32), 1e-4, 1e-6, equal_nan=True) == 1
