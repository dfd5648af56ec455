"""ctypes binding of include/chx_hip.h.  Torch is used for device memory and the
current stream only; every computation goes through libchx_hip.so, and a missing
library is an error (there is no fallback path)."""
import ctypes
import os

import torch

MAX_NDIM = 10
_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libchx_hip.so")

# ChainerX dtype codes (compiler/dtype.h:14-25 of the reference tree)
BOOL, INT8, INT16, INT32, INT64, UINT8, FLOAT16, FLOAT32, FLOAT64 = 1, 2, 3, 4, 5, 6, 7, 8, 9
_TORCH_TO_CHX = {
    torch.bool: BOOL, torch.int8: INT8, torch.int16: INT16, torch.int32: INT32, torch.int64: INT64,
    torch.uint8: UINT8, torch.float16: FLOAT16, torch.float32: FLOAT32, torch.float64: FLOAT64,
}

ROUND_REFERENCE = 0
ROUND_ONNX_RNE = 1
BIAS_REFERENCE_FLOAT = 0
BIAS_ONNX_INT32 = 2
FUSE_RELU = 4
STORE_MINUS_128 = 8
EINVAL, EUNSUPPORTED, ERUNTIME = 1, 2, 3

EXPORTS = [
    "chx_hip_init", "chx_hip_last_error", "chx_hip_version", "chx_hip_get_device_props", "chx_hip_malloc",
    "chx_hip_free", "chx_hip_memcpy_h2d", "chx_hip_memcpy_d2h", "chx_hip_memset", "chx_hip_stream_synchronize",
    "chx_hip_quantize_linear", "chx_hip_dequantize_linear", "chx_hip_qlinear_conv", "chx_hip_qlinear_conv_nd", "chx_hip_conv_integer_nd", "chx_hip_qconv_plan_create",
    "chx_hip_qconv_plan_run", "chx_hip_qconv_plan_run_add", "chx_hip_qconv_plan_run_pair", "chx_hip_qconv_plan_describe", "chx_hip_qconv_plan_pin", "chx_hip_qconv_plan_destroy", "chx_hip_conv_integer", "chx_hip_matmul_integer",
    "chx_hip_qlinear_matmul", "chx_hip_elementwise", "chx_hip_elementwise_source", "chx_hip_elementwise_output_dtypes", "chx_hip_elementwise_match_residual_add",
    "chx_hip_max_pool_q8", "chx_hip_average_pool_q8", "chx_hip_reduce_min_max", "chx_hip_reduce_min_max_noalloc", "chx_hip_cast", "chx_hip_codes_minus_128", "chx_hip_bit_shift", "chx_hip_count_nonfinite",
    "chx_hip_stream_create", "chx_hip_stream_destroy", "chx_hip_capture_begin", "chx_hip_capture_end", "chx_hip_stream_is_capturing",
    "chx_hip_graph_launch", "chx_hip_graph_destroy", "chx_hip_gemm_f32", "chx_hip_linear_f32", "chx_hip_max_pool_f32", "chx_hip_average_pool_f32", "chx_hip_fixed_batch_norm_f32", "chx_hip_conv_f32", "chx_hip_softmax_f32",
]


class Tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("shape", ctypes.c_int64 * MAX_NDIM), ("strides", ctypes.c_int64 * MAX_NDIM)]


class ConvParams(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "stride_h", "stride_w", "pad_h_begin", "pad_w_begin", "pad_h_end", "pad_w_end", "group")]


class ConvNdParams(ctypes.Structure):
    _fields_ = [("n_spatial", ctypes.c_int32), ("stride", ctypes.c_int32 * 3), ("pad_begin", ctypes.c_int32 * 3),
                ("pad_end", ctypes.c_int32 * 3), ("group", ctypes.c_int32)]


def conv_nd_params(strides, begin, end, group):
    p = ConvNdParams()
    p.n_spatial = len(strides)
    for i in range(3):
        p.stride[i], p.pad_begin[i], p.pad_end[i] = 1, 0, 0
    for i, (s, b, e) in enumerate(list(zip(strides, begin, end))[:3]):   # more than three axes: the library refuses n_spatial
        p.stride[i], p.pad_begin[i], p.pad_end[i] = int(s), int(b), int(e)
    p.group = int(group)
    return p


class DeviceProps(ctypes.Structure):
    _fields_ = [("compute_units", ctypes.c_int32), ("clock_khz", ctypes.c_int32),
                ("memory_clock_khz", ctypes.c_int32), ("memory_bus_bits", ctypes.c_int32),
                ("total_memory", ctypes.c_int64), ("arch", ctypes.c_char * 64), ("name", ctypes.c_char * 128)]


class ChxHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("chx_hip error %d: %s" % (code, message))
        self.code = code


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no CPU fallback for the device ops)" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.chx_hip_last_error.restype = ctypes.c_char_p
        _lib.chx_hip_version.restype = ctypes.c_char_p
        _lib.chx_hip_qconv_plan_destroy.restype = None
    return _lib


def check(rc):
    if rc != 0:
        raise ChxHipError(rc, lib().chx_hip_last_error().decode("utf-8", "replace"))


def desc(t):
    """chx_hip_tensor for a torch device tensor (byte strides, like ChainerX)."""
    d = Tensor()
    d.data = t.data_ptr()
    d.dtype = _TORCH_TO_CHX[t.dtype]
    d.ndim = t.dim()
    es = t.element_size()
    for i in range(t.dim()):
        d.shape[i] = t.shape[i]
        d.strides[i] = t.stride(i) * es
    return d


def ref(t):
    return None if t is None else ctypes.byref(desc(t))


def stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def init(device=0):
    check(lib().chx_hip_init(ctypes.c_int(device)))


def device_props():
    p = DeviceProps()
    check(lib().chx_hip_get_device_props(ctypes.byref(p)))
    return dict(compute_units=p.compute_units, clock_khz=p.clock_khz, memory_clock_khz=p.memory_clock_khz,
                memory_bus_bits=p.memory_bus_bits, total_memory=p.total_memory, arch=p.arch.decode(),
                name=p.name.decode())


def conv_params(strides, pads_begin, pads_end, group):
    return ConvParams(strides[0], strides[1], pads_begin[0], pads_begin[1], pads_end[0], pads_end[1], group)


def tensor_array(descs):
    """Array of pointers to chx_hip_tensor (keeps the descriptors alive on the result)."""
    arr = (ctypes.POINTER(Tensor) * len(descs))(*[ctypes.pointer(d) for d in descs])
    arr._keep = descs
    return arr


def make_desc(data_ptr, dtype, shape, strides_bytes):
    d = Tensor()
    d.data = data_ptr
    d.dtype = dtype
    d.ndim = len(shape)
    for i, (n, st) in enumerate(zip(shape, strides_bytes)):
        d.shape[i] = n
        d.strides[i] = st
    return d


def elementwise_output_dtypes(code):
    """chx_hip_elementwise_output_dtypes: the dtype codes of a fusion program's outputs, in order."""
    codes = (ctypes.c_int32 * 64)()
    count = ctypes.c_int32(0)
    check(lib().chx_hip_elementwise_output_dtypes(code.encode(), codes, ctypes.c_int32(64), ctypes.byref(count)))
    return [int(codes[i]) for i in range(count.value)]


def elementwise_source(code, fusion_id, in_descs, out_descs, compile=False):
    """Generated HIP source for a fusion program and operand layouts (no GPU needed)."""
    ins, outs = tensor_array(in_descs), tensor_array(out_descs)
    needed = ctypes.c_size_t(0)
    args = (code.encode(), ctypes.c_int32(fusion_id), ins, ctypes.c_int32(len(in_descs)), outs,
            ctypes.c_int32(len(out_descs)), ctypes.c_int32(1 if compile else 0))
    check(lib().chx_hip_elementwise_source(*args, None, ctypes.c_size_t(0), ctypes.byref(needed)))
    buf = ctypes.create_string_buffer(needed.value)
    check(lib().chx_hip_elementwise_source(*args, buf, ctypes.c_size_t(needed.value), None))
    return buf.value.decode()


class ResidualGroup(ctypes.Structure):
    _fields_ = [("in_scale", ctypes.c_float * 2), ("in_zero_point", ctypes.c_int32 * 2), ("in_dtype", ctypes.c_int32 * 2),
                ("relu", ctypes.c_int32), ("out_scale", ctypes.c_float), ("out_zero_point", ctypes.c_int32),
                ("out_dtype", ctypes.c_int32)]


def match_residual_add(code):
    """chx_hip_elementwise_match_residual_add: None, or a dict of the group's constants."""
    matches = ctypes.c_int32()
    grp = ResidualGroup()
    check(lib().chx_hip_elementwise_match_residual_add(code.encode(), ctypes.byref(matches), ctypes.byref(grp)))
    if not matches.value:
        return None
    return dict(in_scale=list(grp.in_scale), in_zero_point=list(grp.in_zero_point), in_dtype=list(grp.in_dtype), relu=bool(grp.relu),
                out_scale=grp.out_scale, out_zero_point=grp.out_zero_point, out_dtype=grp.out_dtype)
