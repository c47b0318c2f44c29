"""ctypes binding of libqmm_hip.so (the C ABI declared in include/qmm_hip.h).

The library is loaded from the in-tree build (metaljax_amd/lib).  There is no
CPU fallback: if the shared library is missing or fails to load, every entry
point raises QmmLibraryError.
"""

from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libqmm_hip.so")

QMM_OK = 0
ABI_VERSION = 2
ERR_NAMES = {1: "BAD_ARGUMENT", 2: "BAD_SHAPE", 3: "UNSUPPORTED", 4: "WORKSPACE", 5: "HIP"}
F32, BF16, F16 = 0, 1, 2
STATIC_SCRATCH_BYTES = 16 << 20      # QMM_STATIC_SCRATCH_BYTES of include/qmm_hip.h
MODE_AFFINE, MODE_MXFP4 = 0, 1
KERNEL_GEMV, KERNEL_GEMM, KERNEL_MXFP4_MFMA = 1, 2, 3

# every symbol include/qmm_hip.h declares
SYMBOLS = (
    "qmm_abi_version", "qmm_last_error", "qmm_quantized_matmul", "qmm_workspace_bytes",
    "qmm_gather_workspace_bytes", "qmm_plan", "qmm_gather_qmm", "qmm_grouped_qmm",
    "qmm_gather_qmm_static", "qmm_dequantize", "qmm_unpack_codes", "qmm_pack_codes", "qmm_take_k",
)


class QmmLibraryError(RuntimeError):
    """libqmm_hip.so is missing or unusable."""


class QmmError(RuntimeError):
    """A library call returned a non-zero status; `.code` holds it."""

    def __init__(self, code: int, message: str):
        super().__init__(f"qmm_hip {ERR_NAMES.get(code, code)}: {message}")
        self.code = code


class UnsupportedQmm(QmmError):
    """Status UNSUPPORTED / BAD_SHAPE: the caller should run the chain literally."""


_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise QmmLibraryError(
            f"{LIB_PATH} not found: build it with `python -m metaljax_amd.build`")
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:
        raise QmmLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    vp, i64, ci, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
    ip = ctypes.POINTER(ctypes.c_int)
    lib.qmm_abi_version.restype = ci
    lib.qmm_last_error.restype = ctypes.c_char_p
    lib.qmm_quantized_matmul.argtypes = [vp, ci, vp, vp, vp, ci, vp, ci, i64, i64, i64, i64,
                                         ci, ci, ci, vp, sz, vp]
    lib.qmm_workspace_bytes.argtypes = [i64, i64, i64, i64, ci, ci, ci, ci]
    lib.qmm_workspace_bytes.restype = sz
    lib.qmm_gather_workspace_bytes.argtypes = [i64, i64, i64, i64, ci]
    lib.qmm_gather_workspace_bytes.restype = sz
    lib.qmm_plan.argtypes = [i64, i64, i64, ci, ci, ci, ip, ip, ip]
    lib.qmm_gather_qmm.argtypes = [vp, ci, vp, vp, vp, ci, vp, ci, vp, vp, i64, i64, i64, i64,
                                   i64, ci, ci, ci, vp, sz, vp]
    lib.qmm_gather_qmm_static.argtypes = [vp, ci, vp, vp, vp, ci, vp, ci, vp, vp, i64, i64, i64,
                                          i64, i64, ci, ci, ci, vp]
    lib.qmm_grouped_qmm.argtypes = [vp, ci, vp, vp, vp, ci, vp, ci, vp, i64, i64, i64, i64, ci,
                                    ci, ci, vp, sz, vp]
    lib.qmm_dequantize.argtypes = [vp, vp, vp, ci, vp, ci, i64, i64, ci, ci, ci, vp]
    lib.qmm_unpack_codes.argtypes = [vp, vp, i64, i64, ci, vp]
    lib.qmm_pack_codes.argtypes = [vp, vp, i64, i64, ci, vp]
    lib.qmm_take_k.argtypes = [vp, ci, vp, vp, i64, i64, vp]
    for name in SYMBOLS:
        getattr(lib, name)
    if lib.qmm_abi_version() != ABI_VERSION:
        raise QmmLibraryError(f"{LIB_PATH} has ABI version {lib.qmm_abi_version()}, this binding "
                              f"speaks {ABI_VERSION}: rebuild it with `python -m metaljax_amd.build`")
    _lib = lib
    return lib


def check(rc: int):
    if rc == QMM_OK:
        return
    msg = load().qmm_last_error().decode("utf-8", "replace")
    if rc in (2, 3):
        raise UnsupportedQmm(rc, msg)
    raise QmmError(rc, msg)
