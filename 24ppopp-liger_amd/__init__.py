"""MI355X-native (gfx950) implementation of Liger's per-GPU hot path.

The product is native code: `lib/libliger_hip.so` (hand-written HIP kernels behind the C ABI declared in
`include/liger_hip.h`) and `lib/libliger_host.so` (the C++ launch-vector runtime: FuncWrap, layer
assembly, Sample, Scheduler).  This Python package only binds those two libraries with ctypes so that
tests and the benchmark can drive them; it contains no compute and no fallback path: importing `capi`
or `host` raises if the native libraries have not been built.
"""
from . import capi  # noqa: F401
