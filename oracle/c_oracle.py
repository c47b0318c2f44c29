"""ctypes loader for the C oracle (oracle/qmm_oracle.c).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libqmm_oracle.so")
_LIB = None

MODE = {"affine": 0, "mxfp4": 1}


def build(force: bool = False) -> str:
    """Compile oracle/qmm_oracle.c with gcc (make)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libqmm_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.oracle_num_threads.restype = ctypes.c_int
        L.oracle_unpack_codes.argtypes = [vp, i64, i64, i32, vp]
        L.oracle_dequant.argtypes = [vp, vp, vp, i64, i64, i32, i32, i32, i32, i32, vp]
        L.oracle_qmm.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32, i32, i32, i32, vp]
        L.oracle_grouped_qmm.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i32, i32, i32,
                                         i32, i32, vp]
        _LIB = L
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _tables(scales, biases, mode):
    """Tables as contiguous arrays + the bf16 flag.  bf16 tables are passed as
    uint16 bit patterns, f32 tables as float32, E8M0 as uint8."""
    if mode == "mxfp4":
        return np.ascontiguousarray(scales, np.uint8), None, 0
    if scales.dtype == np.uint16:
        return np.ascontiguousarray(scales), np.ascontiguousarray(biases), 1
    return (np.ascontiguousarray(scales, np.float32),
            np.ascontiguousarray(biases, np.float32), 0)


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def unpack_codes(words, bits):
    words = np.ascontiguousarray(words, np.uint32)
    rows = int(np.prod(words.shape[:-1]))
    k = words.shape[-1] * (32 // bits)
    out = np.empty(words.shape[:-1] + (k,), np.uint8)
    lib().oracle_unpack_codes(_p(words), rows, k, bits, _p(out))
    return out


def dequant(words, scales, biases, gs, bits, mode, round_tile_bf16=False):
    """words u32 [N, W]; returns f32 [N, K]."""
    words = np.ascontiguousarray(words).view(np.uint32)
    n = words.shape[0]
    k = words.shape[1] * (8 if mode == "mxfp4" else 32 // bits)
    s, b, isbf = _tables(scales, biases, mode)
    out = np.empty((n, k), np.float32)
    lib().oracle_dequant(_p(words), _p(s), _p(b), n, k, gs, bits, MODE[mode], isbf,
                         int(round_tile_bf16), _p(out))
    return out


def qmm(x_bf16_bits, words, scales, biases, gs, bits, mode, round_tile_bf16=False):
    """x: uint16 bf16 bit patterns [M, K]; returns f32 [M, N] (f32 accumulate)."""
    x = np.ascontiguousarray(x_bf16_bits, np.uint16)
    words = np.ascontiguousarray(words).view(np.uint32)
    m, k = x.shape
    n = words.shape[0]
    s, b, isbf = _tables(scales, biases, mode)
    y = np.empty((m, n), np.float32)
    lib().oracle_qmm(_p(x), _p(words), _p(s), _p(b), m, n, k, gs, bits, MODE[mode], isbf,
                     int(round_tile_bf16), _p(y))
    return y


def grouped_qmm(x_bf16_bits, words, scales, biases, row_offsets, gs, bits, mode,
                round_tile_bf16=False):
    """words [E, N, W]; rows of x sorted by expert; returns f32 [R, N]."""
    x = np.ascontiguousarray(x_bf16_bits, np.uint16)
    words = np.ascontiguousarray(words).view(np.uint32)
    e, n = words.shape[0], words.shape[1]
    r, k = x.shape
    s, b, isbf = _tables(scales, biases, mode)
    ro = np.ascontiguousarray(row_offsets, np.int32)
    y = np.zeros((r, n), np.float32)
    lib().oracle_grouped_qmm(_p(x), _p(words), _p(s), _p(b), _p(ro), e, n, k, gs, bits,
                             MODE[mode], isbf, int(round_tile_bf16), _p(y))
    return y
