"""The entry point that allocates nothing (chx_hip_reduce_min_max_noalloc) against the one it is a variant of,
through the C ABI: two calls in a row, the second on a smaller input, bit for bit; and the size limit."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.capi.init(0)
    return gpu_util


def _reduce(g, entry, x, is_max):
    y = torch.full((), float("nan"), dtype=torch.float32, device="cuda")
    g.capi.check(getattr(g.capi.lib(), entry)(g.capi.ref(x), ctypes.c_int32(1 if is_max else 0), g.capi.ref(y), g.capi.stream_ptr()))
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_two_calls_in_a_row_match_the_allocating_entry_point(g):
    rng = np.random.default_rng(41)
    big = torch.from_numpy(rng.standard_normal((64, 3, 224, 224)).astype(np.float32)).cuda()     # 1024 work-groups: the whole array
    small = torch.from_numpy(rng.standard_normal((5, 7, 11)).astype(np.float32) * 3).cuda()     # one work-group
    strided = big[:, :, ::3, 5:200:7]                                                             # any strides
    for is_max in (True, False):
        for x in (big, small, strided, small):     # a smaller input right after a larger one, twice
            want = _reduce(g, "chx_hip_reduce_min_max", x, is_max)
            got = _reduce(g, "chx_hip_reduce_min_max_noalloc", x, is_max)
            assert got.tobytes() == want.tobytes()
            ref = x.max() if is_max else x.min()
            assert got == ref.cpu().numpy()


def test_sizes_beyond_the_limit_are_refused(g):
    one = torch.zeros(1, dtype=torch.float32, device="cuda")
    huge = one.expand((1 << 30) + 1)               # a broadcast view: no memory behind the extra elements is needed to be refused
    y = torch.zeros((), dtype=torch.float32, device="cuda")
    rc = g.capi.lib().chx_hip_reduce_min_max_noalloc(g.capi.ref(huge), ctypes.c_int32(1), g.capi.ref(y), g.capi.stream_ptr())
    assert rc == g.capi.EINVAL
    assert b"at most" in g.capi.lib().chx_hip_last_error()
    # the limit itself passes (the one element is read 2^30 times)
    ok = one.expand(1 << 30)
    assert _reduce(g, "chx_hip_reduce_min_max_noalloc", ok, True) == 0.0


def test_inside_a_recording(g):
    """What the entry point is for: between capture_begin and capture_end on a created stream it is recorded (it
    allocates nothing), and every replay reduces what the input holds then; the allocating entry point is refused
    there."""
    lib = g.capi.lib()
    stream = ctypes.c_void_p()
    g.capi.check(lib.chx_hip_stream_create(ctypes.byref(stream)))
    rng = np.random.default_rng(43)
    x = torch.from_numpy(rng.standard_normal((300, 1000)).astype(np.float32)).cuda()
    y = torch.full((), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    g.capi.check(lib.chx_hip_capture_begin(stream))
    rc_alloc = lib.chx_hip_reduce_min_max(g.capi.ref(x), ctypes.c_int32(1), g.capi.ref(y), stream)
    rc = lib.chx_hip_reduce_min_max_noalloc(g.capi.ref(x), ctypes.c_int32(1), g.capi.ref(y), stream)
    graph = ctypes.c_void_p()
    g.capi.check(lib.chx_hip_capture_end(stream, ctypes.byref(graph)))
    assert rc_alloc == g.capi.EUNSUPPORTED and rc == 0
    try:
        for i in range(3):
            x.copy_(torch.from_numpy(rng.standard_normal((300, 1000)).astype(np.float32) * (i + 1)))
            torch.cuda.synchronize()
            g.capi.check(lib.chx_hip_graph_launch(graph, stream))
            g.capi.check(lib.chx_hip_stream_synchronize(stream))
            assert float(y) == float(x.max())
            # eager work of the same entry point between the replays (it shares the scratch array, one call at a time)
            assert _reduce(g, "chx_hip_reduce_min_max_noalloc", x[:7], False) == x[:7].min().cpu().numpy()
    finally:
        lib.chx_hip_graph_destroy(graph)
        g.capi.check(lib.chx_hip_stream_destroy(stream))
