"""CPU oracle for the quantized-matmul path.  TEST INFRASTRUCTURE ONLY.

Nothing under the product package may import this module: only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg use it, and only as the
checker.  It restates the *semantics* of the reference's quantized-matmul path
in plain numpy (pure-Python loops only where marked "tiny inputs"), each
function citing the reference lines it follows (paths relative to the
reference tree).

Pinning status (what independently fixes each function; the checks live in
tests/test_oracle.py):

  pack_codes / unpack_codes   hand-computed nibble words (tests/test_qmm_mxfp4.py:162-174),
                              a per-bit brute-force stream writer, round trips
  bf16 helpers                torch.bfloat16 casts (library routine), tie cases by hand
  fma_f32                     exact rational arithmetic (fractions.Fraction)
  scale_bias / pack_exact     the exactness matrix of tests/test_qmm.py:96-171
  dequant_affine              float32 scale*(code-zp) expectation (tests/test_qmm.py:117-132)
  dequant_mxfp4 (table form)  arithmetic sign/exp/mantissa decoder
                              (scripts/model_bench/check_mxfp4_checkpoint.py:39-77),
                              torch.float4_e2m1fn_x2 / float8_e8m0fnu where present
  mxfp4_codes / scale_bytes   accept/reject vectors of tests/test_qmm_mxfp4.py:116-159
  group_const / pick_group*   invariants and the cases of tests/test_qmm.py:510-571
  regroup                     permutation invariants (same tests)
  qmm / gather_qmm / grouped  torch.matmul in float64 on the dequantized weight,
                              brute-force pair loops on tiny inputs

MLX's own accumulation order inside quantized_matmul and XLA:CPU's bf16 dot
rounding are parity unpinned beyond the stated tolerances (the reference tests
say the same: tests/test_qmm_mxfp4.py:319-328).
"""

from __future__ import annotations

import math

import numpy as np

# OCP MXFP4 element grid, indexed by the low three bits of the code; bit 3 is
# the sign (src/metaljax/qmm.py:167-173; tests/test_qmm_mxfp4.py:59-61).
E2M1_MAGS = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)
E2M1 = np.array(list(E2M1_MAGS) + [-m for m in E2M1_MAGS], np.float32)
MXFP4_GROUP = 32
GROUP_SIZES = (128, 64, 32)          # src/metaljax/qmm.py:147


class Reject(Exception):
    """A value-level check failed: the dot must run literally
    (src/metaljax/qmm.py:197-198)."""


# --------------------------------------------------------------------------
# bf16 bit handling
# --------------------------------------------------------------------------


def f32_to_bf16_bits(x) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even.

    NaNs are quieted; infinities and signed zeros pass through.
    """
    u = np.ascontiguousarray(np.asarray(x, np.float32)).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    r = (u.astype(np.uint64) + np.uint64(0x7FFF) + lsb.astype(np.uint64)) >> np.uint64(16)
    r = r.astype(np.uint32)
    r = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b) -> np.ndarray:
    """bfloat16 bit patterns (uint16) -> float32 (exact)."""
    b = np.ascontiguousarray(np.asarray(b, np.uint16))
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_bf16(x) -> np.ndarray:
    """float32 -> nearest bfloat16 value, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def f32_to_f16(x) -> np.ndarray:
    return np.asarray(x, np.float32).astype(np.float16)


# --------------------------------------------------------------------------
# A1: packed code layout
# --------------------------------------------------------------------------


def pack_codes(codes, bits: int) -> np.ndarray:
    """Unsigned codes [..., K] -> uint32 words [..., K*bits/32].

    Each row is one little-endian bit stream, LSB first: element i occupies
    bits [i*bits, (i+1)*bits); out-of-range codes are masked to `bits`
    (src/metaljax/qmm.py:206-232).  Only widths that divide 32 are legal.
    """
    if 32 % bits:
        raise ValueError(f"pack_codes: bits={bits} does not divide 32")
    per = 32 // bits
    codes = np.asarray(codes)
    k = codes.shape[-1]
    if k % per:
        raise ValueError(f"pack_codes: K={k} not a multiple of {per}")
    c = codes.astype(np.int64).astype(np.uint64) & np.uint64((1 << bits) - 1)
    c = c.reshape(codes.shape[:-1] + (k // per, per))
    sh = (np.arange(per, dtype=np.uint64) * np.uint64(bits))
    return (c << sh).sum(axis=-1, dtype=np.uint64).astype(np.uint32)


def pack_codes_bitstream(codes, bits: int) -> np.ndarray:
    """The same layout written one BIT at a time (tiny inputs).

    An independent formulation: bit j of element i lands at stream position
    i*bits + j; position p lives in word p // 32, bit p % 32.  Handles widths
    that straddle words too (the generic reference of tests/test_qmm.py:60-73).
    """
    codes = np.asarray(codes)
    k = codes.shape[-1]
    words = k * bits // 32
    flat = codes.reshape(-1, k)
    out = np.zeros((flat.shape[0], words), np.uint32)
    for r in range(flat.shape[0]):
        for i in range(k):
            v = int(flat[r, i]) & ((1 << bits) - 1)
            for j in range(bits):
                if (v >> j) & 1:
                    p = i * bits + j
                    out[r, p // 32] |= np.uint32(1 << (p % 32))
    return out.reshape(codes.shape[:-1] + (words,))


def unpack_codes(words, bits: int) -> np.ndarray:
    """uint32 words [..., W] -> unsigned codes [..., W*32/bits] (uint8/uint16).

    Inverse of `pack_codes`.
    """
    per = 32 // bits
    w = np.asarray(words, np.uint32)
    sh = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
    c = (w[..., None] >> sh) & np.uint32((1 << bits) - 1)
    dt = np.uint8 if bits <= 8 else np.uint16
    return c.reshape(w.shape[:-1] + (w.shape[-1] * per,)).astype(dt)


def pack_blocks(codes) -> np.ndarray:
    """4-bit codes [..., K] -> checkpoint-style bytes [..., K/2]: low nibble =
    even element (tests/test_qmm_mxfp4.py:93-97;
    scripts/model_bench/mxfp4_gpt_oss.py:93-96)."""
    codes = np.asarray(codes, np.uint8)
    return (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)


# --------------------------------------------------------------------------
# A2/A3: affine algebra
# --------------------------------------------------------------------------


def fma_f32(a, b, c) -> np.ndarray:
    """Correctly rounded float32 fused multiply-add a*b+c, elementwise.

    Valid when a*b is exact in float64 (|b| an integer below 2^29 times a
    float32 `a`, which is every use here).  The float64 sum is rounded to odd
    before the final narrowing so the result is rounded exactly once.
    """
    a64 = np.asarray(a, np.float32).astype(np.float64)
    b64 = np.asarray(b, np.float32).astype(np.float64)
    c64 = np.asarray(c, np.float32).astype(np.float64)
    p = a64 * b64                                   # exact
    t = p + c64
    bb = t - p
    err = (p - (t - bb)) + (c64 - bb)               # TwoSum: p + c == t + err
    bits = t.view(np.int64) if t.ndim else np.array(t).view(np.int64)
    inexact = (err != 0) & np.isfinite(t)
    even = (bits & 1) == 0
    toward = np.where(err > 0, np.inf, -np.inf)
    t = np.where(inexact & even, np.nextafter(t, toward), t)
    return t.astype(np.float32)


def scale_bias(scales, zeros, offset: int, narrow: str | None, width: str = "auto"):
    """The (scales, biases) tables of an exact repack.

    `w = scale*(code - zero)` becomes `scales*q_hat + biases` with
    `q_hat = code + offset` and `biases = -(scale*(zero + offset))`, computed
    in float32.  `narrow` names the source table dtype ("bf16", "f16" or
    None); the tables keep it iff both round-trip losslessly ("auto"), always
    ("source") or never ("f32") (src/metaljax/qmm.py:262-286).

    Returns (scales_f32_values, biases_f32_values, kept_dtype) where
    kept_dtype is "f32", "bf16" or "f16" and the values are already rounded
    to that dtype.
    """
    s32 = np.asarray(scales, np.float32)
    z32 = (np.asarray(zeros).astype(np.float32) if zeros is not None
           else np.float32(0.0))
    b32 = -(s32 * (z32 + np.float32(offset))).astype(np.float32)
    if narrow in ("bf16", "f16") and width != "f32":
        rnd = round_bf16 if narrow == "bf16" else (
            lambda v: f32_to_f16(v).astype(np.float32))
        s_n, b_n = rnd(s32), rnd(b32)
        lossless = bool(np.all(s_n == s32)) and bool(np.all(b_n == b32))
        if width == "source" or lossless:
            return s_n, b_n, narrow
    return s32, b32, "f32"


def pack_exact(codes, scales, zeros, bits: int, narrow=None, offset=None,
               width: str = "auto"):
    """Signed codes + per-group (scale, zero) -> (packed u32, scales, biases,
    table dtype) (src/metaljax/qmm.py:235-259)."""
    off = (1 << (bits - 1)) if offset is None else int(offset)
    packed = pack_codes(np.asarray(codes).astype(np.int64) + off, bits)
    s, b, dt = scale_bias(scales, zeros, off, narrow, width)
    return packed, s, b, dt


def dequant_affine(words, scales, biases, group_size: int, bits: int) -> np.ndarray:
    """Packed affine weight -> float32 [..., K]: one fused multiply-add
    `fma(scale, q_hat, bias)` per element (src/metaljax/qmm.py:71-79;
    tests/test_qmm.py:124-132)."""
    q = unpack_codes(words, bits).astype(np.float32)
    s = np.repeat(np.asarray(scales, np.float32), group_size, axis=-1)
    b = np.repeat(np.asarray(biases, np.float32), group_size, axis=-1)
    return fma_f32(s, q, b)


def dequant_affine_bf16(words, scales, biases, group_size: int, bits: int) -> np.ndarray:
    """The bf16 weight tile: a single round-to-nearest-even of the exact
    float32 FMA (returned as float32 values)."""
    return round_bf16(dequant_affine(words, scales, biases, group_size, bits))


# --------------------------------------------------------------------------
# A4-A6: MXFP4
# --------------------------------------------------------------------------


def e8m0_to_f32(scale_bytes) -> np.ndarray:
    """E8M0 byte -> 2**(byte-127) as float32 (byte 0 is the subnormal 2^-127,
    byte 255 is NaN)."""
    e = np.asarray(scale_bytes, np.uint8).astype(np.int32)
    out = np.ldexp(np.float64(1.0), e - 127).astype(np.float32)
    return np.where(e == 255, np.float32(np.nan), out).astype(np.float32)


def dequant_mxfp4(blocks, scale_bytes) -> np.ndarray:
    """blocks [..., K/2] uint8 + E8M0 bytes [..., K/32] -> float32 [..., K],
    table form: E2M1[code] * 2**(byte-127); low nibble of byte j is element
    2j (tests/test_qmm_mxfp4.py:77-90)."""
    blocks = np.asarray(blocks, np.uint8)
    lo = blocks & 0x0F
    hi = blocks >> 4
    nib = np.stack([lo, hi], axis=-1).reshape(blocks.shape[:-1] + (-1,))
    vals = E2M1[nib]
    k = vals.shape[-1]
    g = vals.reshape(vals.shape[:-1] + (k // MXFP4_GROUP, MXFP4_GROUP))
    return (g * e8m0_to_f32(scale_bytes)[..., None]).reshape(vals.shape).astype(np.float32)


def dequant_mxfp4_arith(blocks, scale_bytes) -> np.ndarray:
    """The same decode by sign/exponent/mantissa arithmetic, an independent
    formulation (scripts/model_bench/check_mxfp4_checkpoint.py:39-77):
    normal (e != 0): (-1)^s * 2^(e-1) * (1 + m/2); subnormal: (-1)^s * m/2."""
    blocks = np.asarray(blocks, np.uint8)
    nib = np.stack([blocks & 0xF, (blocks >> 4) & 0xF], axis=-1)
    nib = nib.reshape(blocks.shape[:-1] + (-1,))
    s = ((nib >> 3) & 1).astype(np.float32)
    e = ((nib >> 1) & 3).astype(np.float32)
    m = (nib & 1).astype(np.float32)
    sign = np.where(s == 1, np.float32(-1.0), np.float32(1.0))
    normal = np.exp2(e - 1.0) * (1.0 + m / 2.0)
    sub = m / 2.0
    vals = (sign * np.where(e != 0, normal, sub)).astype(np.float32)
    # keep the sign of zero (code 8 is -0.0)
    vals = np.where((nib & 7) == 0, np.where(s == 1, np.float32(-0.0), np.float32(0.0)), vals)
    scale = np.repeat(e8m0_to_f32(scale_bytes), MXFP4_GROUP, axis=-1)
    return (vals * scale).astype(np.float32)


def _float_bits(values, kind: str):
    """Bit patterns of `values` in their own dtype: (uint array, width)."""
    if kind == "f32":
        return np.ascontiguousarray(np.asarray(values, np.float32)).view(np.uint32), 32
    if kind == "f16":
        return np.ascontiguousarray(np.asarray(values, np.float16)).view(np.uint16), 16
    if kind == "bf16":      # passed as uint16 bit patterns
        return np.asarray(values, np.uint16), 16
    raise Reject(f"MXFP4 values in {kind}")


def mxfp4_codes(values, kind: str = "f32") -> np.ndarray:
    """4-bit codes for values EXACTLY on the E2M1 grid, by bit-pattern
    equality in the values' own dtype; sign bit -> code bit 3 (so -0.0 is
    code 8); anything off the grid raises Reject
    (src/metaljax/qmm.py:300-332).  bf16 inputs are uint16 bit patterns."""
    bits, width = _float_bits(values, kind)
    one = bits.dtype.type
    sign = (bits >> one(width - 1)).astype(np.uint8)
    mag = bits & one((1 << (width - 1)) - 1)
    if kind == "f32":
        grid = np.array(E2M1_MAGS, np.float32).view(np.uint32)
    elif kind == "f16":
        grid = np.array(E2M1_MAGS, np.float16).view(np.uint16)
    else:
        grid = f32_to_bf16_bits(np.array(E2M1_MAGS, np.float32))
    codes = np.zeros(mag.shape, np.uint8)
    ok = np.zeros(mag.shape, bool)
    for i, g in enumerate(grid.tolist()):
        hit = mag == g
        codes = np.where(hit, np.uint8(i), codes)
        ok |= hit
    if not bool(ok.all()):
        raise Reject("weight values are not on the MXFP4 (E2M1) grid")
    return (codes | (sign << np.uint8(3))).astype(np.uint8)


def mxfp4_scale_bytes(scales) -> np.ndarray:
    """E8M0 bytes for scales that are exact positive normal powers of two:
    the byte is the float32 exponent field; sign or mantissa bits set, or a
    field of 0 / 255, raise Reject (src/metaljax/qmm.py:335-357)."""
    bits = np.ascontiguousarray(np.asarray(scales, np.float32)).view(np.uint32)
    exp = (bits >> np.uint32(23)) & np.uint32(0xFF)
    bad = ((bits & np.uint32(0x807FFFFF)) != 0) | (exp == 0) | (exp == 0xFF)
    if bool(bad.any()):
        raise Reject("MXFP4 group scales are not exact positive powers of two")
    return exp.astype(np.uint8)


# --------------------------------------------------------------------------
# A7/A8: group logic
# --------------------------------------------------------------------------


def group_const(x, gs: int) -> bool:
    """True iff `x` [..., K] is constant inside each contiguous run of `gs`
    along the last axis (src/metaljax/qmm.py:1204-1207).  Compared by value
    (so +0.0 == -0.0 and NaN != NaN, like the reference's `==`)."""
    x = np.asarray(x)
    k = x.shape[-1]
    v = x.reshape(-1, k // gs, gs)
    return bool(np.all(v == v[:, :, :1]))


def group_heads(x, gs: int) -> np.ndarray:
    """First element of each group: [..., K] -> [..., K/gs]
    (src/metaljax/qmm.py:1210-1215)."""
    x = np.asarray(x)
    k = x.shape[-1]
    return np.ascontiguousarray(x.reshape(x.shape[:-1] + (k // gs, gs))[..., 0])


def pick_group_heads(k: int, scale_heads, zero_heads):
    """Largest legal group size given the per-32 heads
    (src/metaljax/qmm.py:1230-1247)."""
    g0 = GROUP_SIZES[-1]
    for g in GROUP_SIZES:
        if g < g0 or k % g:
            continue
        r = g // g0
        if r == 1 or (group_const(scale_heads, r) and (
                zero_heads is None or group_const(zero_heads, r))):
            return g
    return None


def pick_group(k: int, scale_map, zero_map):
    """Largest legal group size the full maps are constant within, or None
    (src/metaljax/qmm.py:1218-1227)."""
    g0 = GROUP_SIZES[-1]
    if k % g0 or not group_const(scale_map, g0):
        return None
    if zero_map is not None and not group_const(zero_map, g0):
        return None
    return pick_group_heads(
        k, group_heads(scale_map, g0),
        None if zero_map is None else group_heads(zero_map, g0))


def regroup(k: int, maps):
    """A stable permutation of the contraction axis that makes the columns
    sharing one (scale, zero) column pair contiguous, or None when no legal
    group size results or the columns are already grouped
    (src/metaljax/qmm.py:418-457).

    The reference clusters by a 64-bit column digest and re-verifies
    exactness afterwards; clustering by the exact column bytes, as here, is
    the collision-free form of the same rule.
    """
    cols = []
    for x in maps:
        if x is None:
            continue
        x = np.asarray(x)
        x2 = x.reshape(-1, k)
        if x2.dtype.kind == "f":
            x2 = np.ascontiguousarray(x2.astype(np.float32)).view(np.uint32)
        else:
            x2 = x2.astype(np.int64)
        cols.append(np.ascontiguousarray(x2.T))
    keys = [b"".join(c[i].tobytes() for c in cols) for i in range(k)]
    first: dict = {}
    ids = np.empty(k, np.int64)
    for i, key in enumerate(keys):
        ids[i] = first.setdefault(key, len(first))
    runs = np.bincount(ids)
    g = 0
    for length in runs:
        g = math.gcd(g, int(length))
    if not any(g and g % s == 0 for s in GROUP_SIZES):
        return None
    perm = np.argsort(ids, kind="stable").astype(np.int32)
    if np.array_equal(perm, np.arange(k, dtype=np.int32)):
        return None
    return perm


# --------------------------------------------------------------------------
# A14/A15: the fused products
# --------------------------------------------------------------------------


def dequant(words, scales, biases, group_size, bits, mode) -> np.ndarray:
    """Dispatch on mode: affine (u32 words) or mxfp4 (u32 words or u8 blocks;
    the two are the same bytes on a little-endian host)."""
    if mode == "affine":
        return dequant_affine(words, scales, biases, group_size, bits)
    w = np.ascontiguousarray(words)
    if w.dtype == np.uint32:
        w = w.view(np.uint8)
    return dequant_mxfp4(w, scales)


def qmm(x, words, scales, biases, group_size=64, bits=4, mode="affine",
        weight_rounding: str = "f32", out: str = "f32") -> np.ndarray:
    """y[..., M, N] = x[..., M, K] . dequant(w)[..., N, K]^T
    (src/metaljax/qmm.py:2491-2499), accumulated in float64 here so the
    oracle sits at the exact answer.

    weight_rounding: "f32" keeps the exactly reconstructed weight (the fused
    kernel's semantics, tests/test_qmm.py:14-16); "bf16" rounds the weight
    tile once to bf16 first (the literal chain's semantics when the graph
    computes in bf16).  out: "f32" or "bf16" (one RNE of the f32 result).
    """
    w = dequant(words, scales, biases, group_size, bits, mode)
    if weight_rounding == "bf16":
        w = round_bf16(w)
    y = np.matmul(np.asarray(x, np.float32).astype(np.float64),
                  np.swapaxes(w.astype(np.float64), -1, -2)).astype(np.float32)
    return round_bf16(y) if out == "bf16" else y


def gather_qmm(x, words, scales, biases, lhs_idx, rhs_idx, group_size=64,
               bits=4, mode="affine", weight_rounding="f32") -> np.ndarray:
    """Per pair p: y[p] = x[lhs_idx[p]] (M x K) . dequant(w[rhs_idx[p]])^T
    -> [P, M, N] (src/metaljax/moe.py:1283-1340).  `x` is [T, M, K], the
    weight arrays carry a leading expert axis."""
    x = np.asarray(x, np.float32)
    outs = []
    for li, ri in zip(np.asarray(lhs_idx).tolist(), np.asarray(rhs_idx).tolist()):
        outs.append(qmm(x[li], words[ri], scales[ri],
                        None if biases is None else biases[ri],
                        group_size, bits, mode, weight_rounding))
    return np.stack(outs, axis=0)


def grouped_qmm(x, words, scales, biases, row_offsets, group_size=64, bits=4,
                mode="affine", weight_rounding="f32") -> np.ndarray:
    """Rows sorted by expert: rows [row_offsets[e], row_offsets[e+1]) of `x`
    [R, K] multiply expert e's weight -> [R, N].  The sorted-rows layout of
    the same per-pair product (src/metaljax/moe.py:1283-1340)."""
    x = np.asarray(x, np.float32)
    n = words.shape[-2]
    y = np.zeros((x.shape[0], n), np.float32)
    ro = np.asarray(row_offsets).tolist()
    for e in range(len(ro) - 1):
        a, b = ro[e], ro[e + 1]
        if b > a:
            y[a:b] = qmm(x[a:b], words[e], scales[e],
                         None if biases is None else biases[e],
                         group_size, bits, mode, weight_rounding)
    return y


def route_top_k(logits, k: int):
    """Softmax router + top-k: (weights [T,k] f32, experts [T,k] int32), ties
    broken toward the lower expert index."""
    z = np.asarray(logits, np.float64)
    p = np.exp(z - z.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    idx = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    return np.take_along_axis(p, idx, -1).astype(np.float32), idx.astype(np.int32)


def sort_pairs_by_expert(experts, n_experts: int):
    """Token-major (token, expert) pairs -> stable order by expert.
    Returns (order [P], token_of_row [P], row_offsets [E+1])."""
    e = np.asarray(experts).reshape(-1)
    t, k = np.asarray(experts).shape
    order = np.argsort(e, kind="stable").astype(np.int32)
    tok = (order // k).astype(np.int32)
    sizes = np.bincount(e, minlength=n_experts)
    ro = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    return order, tok, ro


def rel_l2(got, want) -> float:
    g = np.asarray(got, np.float64)
    w = np.asarray(want, np.float64)
    den = np.sqrt((w * w).sum())
    return float(np.sqrt(((g - w) ** 2).sum()) / (den if den else 1.0))
