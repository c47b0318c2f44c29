"""Properties of the host-side pack primitives that hold for every input, not
only for the seeded cases of test_packing.py: drawn by hypothesis over shapes,
widths, group layouts and table types.  Each property is stated against
arithmetic done another way (Python big integers, float64, a brute-force
loop), never against the function's own formula."""

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from metaljax_amd import packing as P
from oracle import qmm_oracle as O

FEW = settings(max_examples=60, deadline=None)
E2M1 = np.array(O.E2M1, np.float32)


@FEW
@given(bits=st.sampled_from([1, 2, 4, 8, 16]), rows=st.integers(1, 5), words=st.integers(1, 9),
       narrow=st.booleans(), seed=st.integers(0, 2**31 - 1))
def test_packed_words_are_the_rows_little_endian_bit_stream(bits, rows, words, narrow, seed):
    """Element i of a row occupies bits [i*bits, (i+1)*bits) of the row read as
    one little-endian integer (reference qmm.py:206-232) -- checked with Python
    integers; the byte-wise fast path (uint8 codes) gives the same words."""
    per = 32 // bits
    k = words * per
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 1 << bits, size=(rows, k), dtype=np.uint32)
    if narrow and bits <= 8:
        codes = codes.astype(np.uint8)
    got = P.pack_codes(codes, bits)
    assert got.dtype == np.uint32 and got.shape == (rows, words)
    for r in range(rows):
        stream = sum(int(c) << (i * bits) for i, c in enumerate(codes[r].tolist()))
        want = [(stream >> (32 * j)) & 0xFFFFFFFF for j in range(words)]
        assert got[r].tolist() == want
    # and back, one element at a time
    flat = got.astype(np.uint64)
    for i in (0, k // 2, k - 1):
        w, sh = divmod(i * bits, 32)
        np.testing.assert_array_equal((flat[:, w] >> np.uint64(sh)) & np.uint64((1 << bits) - 1), codes[:, i])


@FEW
@given(bits=st.sampled_from([4, 8]), gs=st.sampled_from([32, 64, 128]), n=st.integers(1, 6), groups=st.integers(1, 4),
       kind=st.sampled_from([None, "bf16", "f16"]), offset_shift=st.integers(-2, 2), seed=st.integers(0, 2**31 - 1))
def test_a_pack_reconstructs_scale_times_code_minus_zero_exactly(bits, gs, n, groups, kind, offset_shift, seed):
    """w = scale * (code - zero) in exact arithmetic equals fma(scale, q, bias)
    in float32 on the packed arrays, for scales with few significant bits and
    integer zero points, whatever code offset the pack uses and whether or not
    the tables were narrowed (reference qmm.py:235-286, tests/test_qmm.py:100-152)."""
    rng = np.random.default_rng(seed)
    k = gs * groups
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    codes = rng.integers(lo, hi + 1, size=(n, k)).astype(np.int32)
    zeros = rng.integers(lo, hi + 1, size=(n, groups)).astype(np.int32)
    # seven significant bits times a power of two: exact in bf16 and float16 alike
    scales = (rng.integers(64, 128, size=(n, groups)) * np.exp2(rng.integers(-14, -4, size=(n, groups)))).astype(np.float32)
    offset = (1 << (bits - 1)) + (offset_shift if bits == 8 else 0)
    if not (0 <= lo + offset and hi + offset < (1 << bits)):
        offset = 1 << (bits - 1)
    words, s, b = P.pack_exact(codes, scales, zeros, bits, scale_kind=kind, offset=offset)
    if kind is not None:
        # narrowed exactly when that loses nothing: the scales always fit, the biases (scale times a
        # small integer: up to fifteen significant bits) fit float16 more often than bf16
        b32 = -(scales * (zeros + offset).astype(np.float32))
        back = b32.astype(np.float16).astype(np.float32) if kind == "f16" else O.round_bf16(b32)
        fits = np.array_equal(back, b32) and np.isfinite(back).all()
        assert P.float_kind(s) == P.float_kind(b) == (kind if fits else "f32")
    q = O.unpack_codes(words, bits).astype(np.float64)
    s64, b64 = P.as_f32(s).astype(np.float64), P.as_f32(b).astype(np.float64)
    got = (np.repeat(s64, gs, axis=1) * q + np.repeat(b64, gs, axis=1))
    want = np.repeat(scales.astype(np.float64), gs, axis=1) * (codes - np.repeat(zeros, gs, axis=1))
    np.testing.assert_array_equal(got, want)                       # float64 holds both sides exactly
    np.testing.assert_array_equal(got.astype(np.float32).astype(np.float64), got)   # and float32 holds the result


@FEW
@given(groups=st.integers(1, 6), gs=st.sampled_from([32, 64, 128]), rows=st.integers(1, 3),
       layout=st.sampled_from(["grouped", "interleaved", "shuffled"]), with_zero=st.booleans(),
       seed=st.integers(0, 2**31 - 1))
def test_regrouping_makes_every_group_contiguous_and_keeps_column_order(groups, gs, rows, layout, with_zero, seed):
    """Columns that share one (scale, zero) column vector form a group wherever
    they lie along K.  `regroup` returns a permutation (a bijection) after
    which every group is one contiguous run in first-occurrence order with its
    members in their original order -- or None when the columns are grouped
    already (reference qmm.py:418-457, tests/test_qmm.py:510-617)."""
    rng = np.random.default_rng(seed)
    k = groups * gs
    label = np.repeat(np.arange(groups), gs)
    if layout == "interleaved":
        label = np.tile(np.arange(groups), gs)
    elif layout == "shuffled":
        label = rng.permutation(label)
    table = rng.standard_normal((rows, groups)).astype(np.float32)
    while len({tuple(c) for c in table.T.tolist()}) < groups:       # distinct groups
        table = rng.standard_normal((rows, groups)).astype(np.float32)
    scale_map = table[:, label]
    zero_map = rng.integers(-8, 8, size=(rows, groups)).astype(np.int8)[:, label] if with_zero else None
    perm = P.regroup(k, [scale_map, zero_map])
    already = bool((np.diff(label) != 0).sum() == groups - 1)
    if perm is None:
        assert already
        return
    assert not already
    assert sorted(perm.tolist()) == list(range(k))
    after = label[perm]
    firsts = [int(np.argmax(label == g)) for g in range(groups)]
    order = [g for _, g in sorted(zip(firsts, range(groups)))]
    np.testing.assert_array_equal(after, np.repeat(order, gs))     # contiguous runs, first occurrence first
    for g in range(groups):
        members = perm[after == g]
        assert (np.diff(members) > 0).all()                        # original order inside a group
    assert P.pick_group(k, P.take_k(scale_map, perm), None if zero_map is None else P.take_k(zero_map, perm)) is not None


@FEW
@given(shape=st.tuples(st.integers(1, 4), st.integers(1, 5).map(lambda g: 32 * g)),
       kind=st.sampled_from(["f32", "f16", "bf16"]), seed=st.integers(0, 2**31 - 1))
def test_every_e2m1_value_goes_back_to_its_code_sign_of_zero_included(shape, kind, seed):
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=shape).astype(np.uint8)
    values = np.where(codes & 8, -E2M1[codes & 7], E2M1[codes & 7]).astype(np.float32)
    assert np.signbit(values[codes == 8]).all()                    # -0.0 is a value of its own
    typed = {"f32": values, "f16": values.astype(np.float16), "bf16": P.BF16Array.from_f32(values)}[kind]
    np.testing.assert_array_equal(P.mxfp4_codes(typed), codes)
    # one value off the grid anywhere is refused
    off = values.copy()
    off.flat[int(rng.integers(off.size))] = 2.5
    with pytest.raises(P.Reject):
        P.mxfp4_codes(off)


@FEW
@given(st.lists(st.integers(1, 254), min_size=1, max_size=64))
def test_scale_bytes_are_the_exponent_of_exact_powers_of_two(exps):
    b = np.array(exps, np.uint8)
    scales = np.ldexp(np.float64(1.0), b.astype(np.int64) - 127).astype(np.float32)
    np.testing.assert_array_equal(P.mxfp4_scale_bytes(scales), b)
    for bad in (scales * np.float32(1.5), -scales, np.where(np.arange(len(b)) == 0, np.float32(0.0), scales)):
        with pytest.raises(P.Reject):
            P.mxfp4_scale_bytes(bad.astype(np.float32))
