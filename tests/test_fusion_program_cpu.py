"""Host logic of the fused element-wise path, exercised without a GPU: program
parsing, operand-layout planning, source generation and hiprtc compilation for
gfx950 (hiprtc cross-compiles without a device)."""
import pytest
import torch

import __graft_entry__ as entry

pkg = entry.load_package()
capi, ops = pkg.capi, pkg.ops

F32 = torch.float32
CHAIN = ops.fusion_program(
    [("x", F32), ("a", F32), ("b", F32), ("c", F32)],
    [("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"), ("t3", "Sigmoid", "c"),
     ("t4", "Mul", "t2", "t3"), ("t5", "Add", "t4", "x"), ("y", "Relu", "t5")],
    [("y", F32)])


def fake(shape, dtype=capi.FLOAT32, es=4, addr=0x10000000, strides=None):
    if strides is None:
        strides, acc = [], es
        for n in reversed(shape):
            strides.insert(0, acc)
            acc *= n
    return capi.make_desc(addr, dtype, shape, strides)


def test_chain_plans_vector_kernel_with_periodic_broadcast():
    full = (64, 1024, 1024)
    src = capi.elementwise_source(CHAIN, 7, [fake(full), fake((1024,)), fake((1024,)), fake(full)], [fake(full)],
                                  compile=True)
    head = src.splitlines()[0]
    assert "modes=FPPF vector" in head
    assert "fusion7_vec" in src and "fusion7_gen" in src
    assert "base % 1024u" in src                 # the [1024] operands are read in place, not materialised
    assert "tanhf_faithful" in src and "sigmoid_faithful" in src
    assert "#pragma clang fp contract(off)" in src


def test_scalar_and_general_modes():
    full = (8, 30)
    src = capi.elementwise_source(CHAIN, 1, [fake(full), fake(()), fake((1,)), fake(full)], [fake(full)])
    assert "modes=FSSF vector" in src.splitlines()[0]
    # a column operand [8,1] is neither full, scalar nor periodic -> general kernel
    src = capi.elementwise_source(CHAIN, 1, [fake(full), fake((8, 1)), fake((30,)), fake(full)], [fake(full)])
    assert "general" in src.splitlines()[0]
    # misaligned full operand -> general kernel
    src = capi.elementwise_source(CHAIN, 1, [fake(full, addr=0x10000004), fake(()), fake(()), fake(full)], [fake(full)])
    assert "general" in src.splitlines()[0]


def test_quantized_chain_uses_16_wide_vectors():
    prog = ops.fusion_program(
        [("qa", torch.uint8), ("qb", torch.uint8)],
        [("a", "DequantizeLinear", "qa", 0.05, 128), ("b", "DequantizeLinear", "qb", 0.02, 120),
         ("s", "Add", "a", "b"), ("r", "Relu", "s"), ("q", "QuantizeLinear", "r", 0.06, 0, "uint8")],
        [("q", torch.uint8)])
    shp = (4, 64, 14, 14)
    u8 = dict(dtype=capi.UINT8, es=1)
    src = capi.elementwise_source(prog, 2, [fake(shp, **u8), fake(shp, **u8)], [fake(shp, **u8)], compile=True)
    assert "modes=FF vector" in src.splitlines()[0]
    assert "int x0[16]" in src


@pytest.mark.parametrize("prog,msg", [
    ("extern \"C\" __global__ void fusion0() {}", "header"),
    ("chxhip-fusion 1\nin x:float32\ny = Cosh x\nout y:float32\n", "not in the fusable set"),
    ("chxhip-fusion 1\nin x:float32\ny = Add x z\nout y:float32\n", "before definition"),
    ("chxhip-fusion 1\nin x:float32\ny = Add x\nout y:float32\n", "takes 2 operands"),
    ("chxhip-fusion 1\nin x:float32\ny = Tanh x\nout y:uint8\n", "declared uint8"),
    ("chxhip-fusion 1\nin x:int32\ny = Tanh x\nout y:float32\n", "unsupported dtype"),
    ("chxhip-fusion 1\nin x:float64\ny = Tanh x\nout y:float32\n", "two floating-point types"),
    ("chxhip-fusion 1\nin x:uint8\ny = Tanh x\nout y:float32\n", "wrong kind"),
    ("chxhip-fusion 1\nin x:float32\ny = QuantizeLinear x 0.1 300 uint8\nout y:uint8\n", "out of range"),
])
def test_program_errors(prog, msg):
    with pytest.raises(capi.ChxHipError, match=msg):
        u8 = dict(dtype=capi.UINT8, es=1)
        capi.elementwise_source(prog, 0, [fake((16,), **(u8 if "x:uint8" in prog else {}))],
                                [fake((16,), **(u8 if "y:uint8" in prog else {}))])


def test_operand_errors():
    with pytest.raises(capi.ChxHipError, match="does not broadcast"):
        capi.elementwise_source(CHAIN, 0, [fake((4, 5)), fake((3,)), fake(()), fake((4, 5))], [fake((4, 5))])
    with pytest.raises(capi.ChxHipError, match="extent"):
        capi.elementwise_source(CHAIN, 0, [fake((4, 5)), fake(()), fake(()), fake((4, 5))], [fake((4, 6))])
    with pytest.raises(capi.ChxHipError, match="program declares 4 inputs"):
        capi.elementwise_source(CHAIN, 0, [fake((4, 5))], [fake((4, 5))])
    with pytest.raises(capi.ChxHipError, match="is uint8, program says float32"):
        capi.elementwise_source(CHAIN, 0, [fake((4, 5), dtype=capi.UINT8), fake(()), fake(()), fake((4, 5))],
                                [fake((4, 5))])


def test_residual_sum_groups_are_recognised():
    """The one group shape a convolution can absorb: Q(act(DQ(in0) + DQ(in1))), operands of the Add in
    either order, Relu optional; anything else is left to the element-wise kernel."""
    import numpy as np
    u8, i8 = torch.uint8, torch.int8

    def group(relu=True, swap=False, tail=(), out_dtype="uint8", rne=False, second="b"):
        st = [("fa", "DequantizeLinear", "a", 0.05, 128), ("fb", "DequantizeLinear", second, "0x3ca3d70a", -3)]
        st.append(("s", "Add", "fb", "fa") if swap else ("s", "Add", "fa", "fb"))
        last = "s"
        if relu:
            st.append(("r", "Relu", "s"))
            last = "r"
        st.extend(tail)
        q = ("q", "QuantizeLinear", tail[-1][0] if tail else last, 0.06, 7, out_dtype) + (("rne",) if rne else ())
        return ops.fusion_program([("a", u8), ("b", i8)], st + [q], [("q", u8 if out_dtype == "uint8" else i8)])
    for relu in (True, False):
        for swap in (True, False):
            m = capi.match_residual_add(group(relu, swap))
            assert m is not None and m["relu"] == relu
            assert m["in_scale"] == [np.float32(0.05), np.float32(0.02)] and m["in_zero_point"] == [128, -3]
            assert m["in_dtype"] == [capi.UINT8, capi.INT8]
            assert (m["out_scale"], m["out_zero_point"], m["out_dtype"]) == (np.float32(0.06), 7, capi.UINT8)
    assert capi.match_residual_add(group(out_dtype="int8"))["out_dtype"] == capi.INT8
    assert capi.match_residual_add(group(rne=True)) is None                       # another rounding
    assert capi.match_residual_add(group(tail=(("t", "Tanh", "r"),))) is None     # another activation
    assert capi.match_residual_add(group(second="a")) is None                     # the same operand twice
    assert capi.match_residual_add(CHAIN) is None                                 # float chain
    with pytest.raises(capi.ChxHipError):
        capi.match_residual_add("not a program")


# ---- the CUDA C text of the reference's BuildNvrtcProgram as program text ----------------------------------

def _nvrtc_sources():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "nvrtc_fusion_sources.json")) as f:
        return json.load(f)


def test_reference_kernel_text_is_accepted():
    src = _nvrtc_sources()
    assert capi.elementwise_output_dtypes(src["tanh_sigmoid_float"]) == [capi.FLOAT32]
    text = capi.elementwise_source(src["tanh_sigmoid_float"], 1, [fake((4, 8))], [fake((4, 8))], compile=True)
    # tanh through the C library's arithmetic; the sigmoid is that text's helper, operation by operation
    assert text.count("tanhf_faithful") >= 2 and "sigmoid_faithful<" not in text.split("namespace {")[-1]
    full = (16, 64)
    chain = src["chain_T"].replace("@T@", "float")
    text = capi.elementwise_source(chain, 3, [fake(full), fake((64,)), fake((64,)), fake(full)], [fake(full)], compile=True)
    assert "modes=FPPF vector" in text.splitlines()[0]
    two = src["const_sub_div_exp_identity_float"]
    assert capi.elementwise_output_dtypes(two) == [capi.FLOAT32, capi.FLOAT32]
    capi.elementwise_source(two, 12, [fake((5,)), fake((5,))], [fake((5,)), fake((5,))], compile=True)


@pytest.mark.parametrize("ctype,code,es", [("half", capi.FLOAT16, 2), ("double", capi.FLOAT64, 8)])
def test_half_and_double_programs_compile_for_the_general_kernel(ctype, code, es):
    chain = _nvrtc_sources()["chain_T"].replace("@T@", ctype)
    assert capi.elementwise_output_dtypes(chain) == [code]
    full = (16, 64)
    t = dict(dtype=code, es=es)
    text = capi.elementwise_source(chain, 3, [fake(full, **t), fake((64,), **t), fake((64,), **t), fake(full, **t)], [fake(full, **t)],
                                   compile=True)
    assert "general" in text.splitlines()[0]
    assert ("chx_round_f16(" in text.split("namespace {")[-1]) == (ctype == "half")
    # this library's own program text in the same types
    dt = {"half": torch.float16, "double": torch.float64}[ctype]
    own = ops.fusion_program([("x", dt), ("y", dt)], [("s", "Add", "x", "y"), ("r", "Relu", "s"), ("c", "Clip", "r", 0.25, 6.0)], [("c", dt)])
    capi.elementwise_source(own, 4, [fake(full, **t), fake(full, **t)], [fake(full, **t)], compile=True)


@pytest.mark.parametrize("bad,msg", [
    ("typedef int T;\nextern \"C\" __global__\nvoid fusion1(size_t n, T* i_a, T* o_b) {\nconst T v_a = i_a[tid];\no_b[tid] = v_a;\n}\n", "half, float or double"),
    ("typedef float T;\nextern \"C\" __global__\nvoid fusion1(size_t n, T* i_a, T* o_b) {\nconst T v_a = i_a[tid];\nconst T v_b = erf(v_a);\no_b[tid] = v_b;\n}\n", "not one the reference"),
    ("typedef float T;\nextern \"C\" __global__\nvoid fusion1(size_t n, T* i_a, T* o_b) {\nconst T v_a = i_a[tid];\n}\n", "never stored"),
])
def test_reference_kernel_text_errors(bad, msg):
    with pytest.raises(capi.ChxHipError) as e:
        capi.elementwise_source(bad, 1, [fake((4,))], [fake((4,))])
    assert msg in str(e.value)


def test_mixed_float_types_and_quantization_outside_float32_are_refused():
    with pytest.raises(capi.ChxHipError) as e:
        capi.elementwise_output_dtypes(ops.fusion_program([("x", torch.float16), ("y", torch.float32)], [("s", "Add", "x", "y")], [("s", torch.float32)]))
    assert "two floating-point types" in str(e.value)
    prog = ops.fusion_program([("x", torch.float64)], [("q", "QuantizeLinear", "x", 0.05, 0, "int8")], [("q", torch.int8)])
    with pytest.raises(capi.ChxHipError) as e:
        capi.elementwise_source(prog, 1, [fake((4,), dtype=capi.FLOAT64, es=8)], [fake((4,), dtype=capi.INT8, es=1)])
    assert "8-bit ports go with float32" in str(e.value)
