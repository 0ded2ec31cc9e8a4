"""MI355X-native kernels for the inference path SOFIE emits (Gemm, Conv, quantized and FP8
GEMM/conv), reached through the C ABI declared in include/sofie_hip.h.

`sofie_amd.lib`      ctypes binding of libsofie_hip.so
`sofie_amd.ops`      array-in / array-out operator front end used by tests and the benchmark
`sofie_amd/host`     C++ RModel / ROperator emitters that generate Session code calling the C ABI
"""
from . import lib  # noqa: F401
