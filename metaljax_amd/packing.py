"""Host-side pack primitives of the quantized-matmul recognizer.

One-time work done at the first execute of a recognized dot: verify the
materialized codes / scale / zero maps and repack them into the layout the
kernels read.  Same names, argument meaning and error behaviour as the
reference's primitives (reference src/metaljax/qmm.py:206-457, :1204-1247),
computed with numpy on the host (the maps are evaluated there by the
recognizer); `kernels.pack_codes` is the device-side twin of `pack_codes` for
weights that are already resident.

bf16 arrays are carried as uint16 bit patterns wrapped in `BF16Array`, since
numpy has no bfloat16.
"""

from __future__ import annotations

import math
import os

import numpy as np

GROUP_SIZES = (128, 64, 32)                     # largest first (reference qmm.py:147)
E2M1_MAGS = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
MXFP4_GROUP = 32
# Width policy of the scale / bias tables: auto | source | f32 (reference qmm.py:154-161).
SCALE_WIDTH = os.environ.get("METALJAX_QMM_SCALES", "auto")


class Reject(Exception):
    """A candidate does not match (or cannot be trusted): run it literally."""


# ---------------------------------------------------------------- bf16 ----

class BF16Array:
    """A bfloat16 array held as uint16 bit patterns."""

    __slots__ = ("bits",)

    def __init__(self, bits):
        self.bits = np.ascontiguousarray(bits, dtype=np.uint16)

    @property
    def shape(self):
        return self.bits.shape

    @classmethod
    def from_f32(cls, x):
        return cls(f32_to_bf16_bits(x))

    def to_f32(self) -> np.ndarray:
        return (self.bits.astype(np.uint32) << 16).view(np.float32)

    def __getitem__(self, idx):
        return BF16Array(self.bits[idx])

    def reshape(self, *shape):
        return BF16Array(self.bits.reshape(*shape))


def f32_to_bf16_bits(x) -> np.ndarray:
    """float32 -> bf16 bit patterns, round to nearest even; NaN stays NaN."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    bias = ((u >> 16) & 1) + np.uint32(0x7FFF)
    out = ((u.astype(np.uint64) + bias) >> 16).astype(np.uint16)
    is_nan = (u & 0x7FFFFFFF) > 0x7F800000
    return np.where(is_nan, ((u >> 16) | 0x40).astype(np.uint16), out)


def as_f32(x) -> np.ndarray:
    """Any supported float array (np.float32/16, BF16Array) widened exactly."""
    if isinstance(x, BF16Array):
        return x.to_f32()
    return np.asarray(x).astype(np.float32)


def float_kind(x) -> str:
    if isinstance(x, BF16Array):
        return "bf16"
    dt = np.asarray(x).dtype
    return {np.dtype(np.float32): "f32", np.dtype(np.float16): "f16"}.get(dt, str(dt))


def _narrow(x32: np.ndarray, kind: str):
    """float32 -> `kind` ("bf16" | "f16"), plus the value it round-trips to."""
    if kind == "bf16":
        a = BF16Array.from_f32(x32)
        return a, a.to_f32()
    h = x32.astype(np.float16)
    return h, h.astype(np.float32)


# --------------------------------------------------------- code packing ----

def pack_codes(codes, bits: int) -> np.ndarray:
    """Unsigned codes [..., K] -> uint32 words [..., K*bits/32]; element i at
    bits [i*bits, (i+1)*bits) of the row's little-endian stream; codes masked
    to `bits` (reference qmm.py:206-232)."""
    if 32 % bits:
        raise ValueError(f"pack_codes: bits={bits} does not divide 32")
    per = 32 // bits
    codes = np.asarray(codes)
    k = codes.shape[-1]
    if k % per:
        raise ValueError(f"pack_codes: K={k} not a multiple of {per}")
    if codes.dtype == np.uint8 and bits in (4, 8):
        # byte-wise fast path for the common widths (same stream, fewer passes)
        if bits == 4:
            by = (codes[..., 0::2] & np.uint8(15)) | (codes[..., 1::2] << np.uint8(4))
        else:
            by = codes
        return np.ascontiguousarray(by).view(np.uint32)
    c = codes.astype(np.uint32, copy=False).reshape(codes.shape[:-1] + (k // per, per))
    mask = np.uint32((1 << bits) - 1)
    out = c[..., 0] & mask
    for i in range(1, per):
        out = out | ((c[..., i] & mask) << np.uint32(i * bits))
    return out


def scale_bias(scales, zeros, offset: int, scale_kind: str | None):
    """(scales, biases) tables: biases = -(scale*(zero+offset)) in float32;
    narrowed to the source kind ("bf16"/"f16") iff lossless (auto), always
    (source), never (f32) (reference qmm.py:262-286)."""
    s32 = np.ascontiguousarray(as_f32(scales))
    z32 = as_f32(zeros) if zeros is not None else np.float32(0.0)
    b32 = (-(s32 * (z32 + np.float32(offset)))).astype(np.float32)
    if scale_kind in ("bf16", "f16") and SCALE_WIDTH != "f32":
        s_n, s_back = _narrow(s32, scale_kind)
        b_n, b_back = _narrow(b32, scale_kind)
        if SCALE_WIDTH == "source" or (np.array_equal(s_back, s32) and np.array_equal(b_back, b32)):
            return s_n, b_n
    return s32, b32


def pack_exact(codes, scales, zeros, bits: int, scale_kind=None, offset=None):
    """Signed codes [N,K] + per-group (scale, zero) [N,K/gs] of
    w = scale*(code-zero) -> (packed uint32, scales, biases) with
    q_hat = code+offset, biases = -scale*(offset+zero); offset defaults to
    2^(bits-1) (reference qmm.py:235-259)."""
    off = (1 << (bits - 1)) if offset is None else int(offset)
    q = np.asarray(codes).astype(np.int64) + off
    return (pack_codes(q.astype(np.uint32), bits),) + scale_bias(scales, zeros, off, scale_kind)


# --------------------------------------------------------------- MXFP4 ----

def _bit_view(values):
    if isinstance(values, BF16Array):
        return values.bits, 16, f32_to_bf16_bits(np.array(E2M1_MAGS, np.float32))
    v = np.ascontiguousarray(values)
    if v.dtype == np.float32:
        return v.view(np.uint32), 32, np.array(E2M1_MAGS, np.float32).view(np.uint32)
    if v.dtype == np.float16:
        return v.view(np.uint16), 16, np.array(E2M1_MAGS, np.float16).view(np.uint16)
    raise Reject(f"MXFP4 values in {v.dtype}")


def mxfp4_codes(values) -> np.ndarray:
    """4-bit codes for values lying EXACTLY on the E2M1 grid, matched by bit
    pattern in the values' own dtype (-0.0 is code 8); raises Reject on any
    other value (reference qmm.py:300-332)."""
    bits, width, grid = _bit_view(values)
    if len(set(grid.tolist())) != len(E2M1_MAGS):
        raise Reject("the E2M1 grid is not distinct in this dtype")
    sign = (bits >> (width - 1)).astype(np.uint8)
    mag = bits & bits.dtype.type((1 << (width - 1)) - 1)
    order = np.argsort(grid)
    pos = np.searchsorted(grid[order], mag)
    pos = np.minimum(pos, len(grid) - 1)
    hit = grid[order][pos] == mag
    if not bool(hit.all()):
        raise Reject("weight values are not on the MXFP4 (E2M1) grid")
    return (order[pos].astype(np.uint8) | (sign << 3)).astype(np.uint8)


def mxfp4_scale_bytes(scales) -> np.ndarray:
    """E8M0 bytes of scales that are exact positive normal powers of two: the
    float32 exponent field; anything else raises Reject (reference qmm.py:335-357)."""
    bits = np.ascontiguousarray(as_f32(scales)).view(np.uint32)
    exp = (bits >> 23) & 0xFF
    if bool(((bits & 0x807FFFFF) != 0).any() or (exp == 0).any() or (exp == 0xFF).any()):
        raise Reject("MXFP4 group scales are not exact positive powers of two")
    return exp.astype(np.uint8)


# --------------------------------------------------------- group logic ----

def _values(x):
    return x.to_f32() if isinstance(x, BF16Array) else np.asarray(x)


def group_const(x, gs: int) -> bool:
    """Is `x` [..., K] constant within each contiguous group of `gs`? (qmm.py:1204)"""
    v = _values(x)
    k = v.shape[-1]
    v = v.reshape(-1, k // gs, gs)
    return bool((v == v[:, :, :1]).all())


def group_heads(x, gs: int):
    """First element of each group, [..., K] -> [..., K/gs] (qmm.py:1210)."""
    if isinstance(x, BF16Array):
        return BF16Array(group_heads(x.bits, gs))
    x = np.asarray(x)
    k = x.shape[-1]
    return np.ascontiguousarray(x.reshape(x.shape[:-1] + (k // gs, gs))[..., 0])


def pick_group_heads(k: int, scale_heads, zero_heads):
    """Largest legal group size, read off the per-32 heads (qmm.py:1230-1247)."""
    g0 = GROUP_SIZES[-1]
    for g in GROUP_SIZES:
        if g < g0 or k % g:
            continue
        r = g // g0
        if r == 1 or (group_const(scale_heads, r)
                      and (zero_heads is None or group_const(zero_heads, r))):
            return g
    return None


def pick_group(k: int, scale_map, zero_map):
    """Largest legal group size the maps are constant within (qmm.py:1218-1227)."""
    g0 = GROUP_SIZES[-1]
    if k % g0 or not group_const(scale_map, g0):
        return None
    if zero_map is not None and not group_const(zero_map, g0):
        return None
    return pick_group_heads(k, group_heads(scale_map, g0),
                            None if zero_map is None else group_heads(zero_map, g0))


def _column_words(x, k: int) -> np.ndarray:
    """[..., K] -> uint32 [K, rows]: an injective widening of every column."""
    if isinstance(x, BF16Array):
        v = x.bits.reshape(-1, k).astype(np.uint32)
    else:
        v = np.asarray(x).reshape(-1, k)
        if v.dtype.kind == "f":
            v = np.ascontiguousarray(v.astype(np.float32)).view(np.uint32)
        else:
            v = v.astype(np.int64).astype(np.uint32)
    return np.ascontiguousarray(v.T)


def regroup(k: int, maps):
    """A permutation of the contraction axis that makes interleaved
    quantization groups contiguous, or None when none can help or the columns
    are already grouped (reference qmm.py:418-457).  Columns are clustered by
    their exact (scale, zero) contents, clusters laid out in first-occurrence
    order, members kept in their original order."""
    cols = np.concatenate([_column_words(x, k) for x in maps if x is not None], axis=1)
    _, first, inv = np.unique(cols, axis=0, return_index=True, return_inverse=True)
    inv = np.asarray(inv).reshape(-1)
    rank = np.empty(len(first), np.int64)
    rank[np.argsort(first)] = np.arange(len(first))
    ids = rank[inv]
    g = 0
    for length in np.bincount(ids):
        g = math.gcd(g, int(length))
    if not any(g and g % s == 0 for s in GROUP_SIZES):
        return None
    perm = np.argsort(ids, kind="stable").astype(np.int32)
    if np.array_equal(perm, np.arange(k, dtype=np.int32)):
        return None
    return perm


def take_k(x, perm):
    """`x[..., perm]` for numpy arrays and BF16Array alike."""
    if isinstance(x, BF16Array):
        return BF16Array(x.bits[..., perm])
    return np.ascontiguousarray(np.asarray(x)[..., perm])
