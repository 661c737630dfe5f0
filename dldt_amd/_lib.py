"""ctypes loader for libhipie.so (the C-ABI library).  Fails loudly when it is not built."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhipie.so")

_lib = None


class HipieError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("hipie status %d: %s" % (status, message))
        self.status = status


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m dldt_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        # One HIP runtime per process: PyTorch bundles its own libamdhip64.so.7; importing torch first
        # makes the dynamic loader bind libhipie.so to that copy (same SONAME) instead of mapping a
        # second runtime from /opt/rocm, which leaves whichever initialises second without a GPU.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.hipie_last_error.restype = ctypes.c_char_p
        _lib.hipie_version.restype = ctypes.c_char_p
        _lib.hipie_fq_host_eval.restype = ctypes.c_float
    return _lib


def check(status):
    if status != 0:
        raise HipieError(status, lib().hipie_last_error().decode(errors="replace"))
