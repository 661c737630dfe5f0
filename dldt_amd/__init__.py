"""dldt_amd — MI355X-native INT8 execution engine behind the OpenVINO 2021.4 plugin API.

The product is the C-ABI library ``libhipie.so`` (``include/hipie.h``); this package is the thin
Python binding used by the tests and the benchmark.  There is no CPU fallback: every operator
object raises if the library is missing.
"""
from ._lib import HipieError, lib  # noqa: F401
from .ops import BatchedMatMul, Convolution, FakeQuantize, attention, gelu, make_epilogue, mvn, softmax  # noqa: F401
from .tensor import DeviceTensor  # noqa: F401
