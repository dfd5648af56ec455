"""MI355X-native quantized-inference ops behind chainer-compiler's ChxVM op API.

The directory name carries a hyphen, so the package is imported under the name
``chainer_compiler_amd`` through ``__graft_entry__.load_package()``.

  capi   ctypes binding of the C ABI declared in include/chx_hip.h
  ops    Python mirror of the ChxVM ops on this path (same names and argument
         order as the RunImpl signatures), on torch device tensors
  workloads  the quantized networks of the benchmark configurations as hand-built
         op programs, and the runner that executes them on the device
"""
from . import capi  # noqa: F401
from . import ops  # noqa: F401
from . import workloads  # noqa: F401
