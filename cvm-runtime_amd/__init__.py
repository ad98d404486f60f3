"""MI355X (gfx950) backend for the CVM deterministic integer inference path.

The product is the shared library `libcvm_runtime_hip.so` built from csrc/:
hand-written HIP kernels behind the operator-level C ABI
(include/cvm_hip_ops.h) and a C++ graph runtime behind the reference's model
C API (include/cvm_c_api.h).  This Python package is only a loader plus thin
ctypes wrappers; torch is used for device memory and streams, nothing else.

There is no CPU fallback: if the library is missing or no GPU is present the
wrappers raise.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcvm_runtime_hip.so")
_lib = None


class CvmHipError(RuntimeError):
    pass


def lib():
    """The loaded shared library (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CvmHipError(
                "%s is missing: build it with `python cvm-runtime_amd/build.py` "
                "(there is no CPU fallback)" % LIB_PATH)
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.cvmhip_last_error.restype = ctypes.c_char_p
        for name in ("cvmhip_conv2d_workspace_bytes", "cvmhip_dense_workspace_bytes",
                     "cvmhip_get_valid_counts_workspace_bytes", "cvmhip_nms_workspace_bytes",
                     "cvmhip_nms_static_capacity_bytes",
                     "cvmhip_packed_weight_bytes", "cvmhip_packed_act_bytes", "cvmhip_packed_depthwise_bytes"):
            getattr(_lib, name).restype = ctypes.c_size_t
    return _lib


def check(rc):
    if rc != 0:
        raise CvmHipError("cvmhip error %d: %s" % (rc, lib().cvmhip_last_error().decode()))
