"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

import __graft_entry__ as entry

pkg = entry.load_package()
capi = pkg.capi
ops = pkg.ops
workloads = pkg.workloads


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def ulp_diff(a, b):
    a = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7FFFFFFF), a)
    b = np.where(b < 0, -(b & 0x7FFFFFFF), b)
    return np.abs(a - b)


def to_channels_last(t):
    """NCHW-shaped view of channels-last memory holding the same values."""
    return t.permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)
