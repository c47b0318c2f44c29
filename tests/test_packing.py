"""Host-side pack primitives (metaljax_amd.packing) against the oracle and the
reference's known-answer cases."""

import numpy as np
import pytest

from metaljax_amd import packing as P
from oracle import qmm_oracle as O

E2M1 = O.E2M1


@pytest.mark.parametrize("bits", [2, 4, 8, 16])
@pytest.mark.parametrize("shape", [(1, 32), (5, 128), (3, 4, 64)])
@pytest.mark.parametrize("dt", [np.uint8, np.uint32, np.int32])
def test_pack_codes(bits, shape, dt):
    if bits == 16 and dt == np.uint8:
        pytest.skip("codes do not fit")
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 1 << bits, size=shape).astype(dt)
    np.testing.assert_array_equal(P.pack_codes(codes, bits), O.pack_codes_bitstream(codes, bits))


def test_pack_codes_masks_and_errors():
    assert P.pack_codes(np.array([[0x1F, 0x23] + [0] * 6], np.uint8), 4)[0, 0] == 0x3F
    assert P.pack_codes(np.array([[0x1F, 0x23] + [0] * 6], np.int32), 4)[0, 0] == 0x3F
    with pytest.raises(ValueError):
        P.pack_codes(np.zeros((1, 32), np.uint32), 3)
    with pytest.raises(ValueError):
        P.pack_codes(np.zeros((1, 12), np.uint32), 4)


def test_bf16_bits_match_oracle():
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(1000).astype(np.float32),
                        np.array([np.nan, np.inf, -0.0, 1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8], np.float32)])
    np.testing.assert_array_equal(P.f32_to_bf16_bits(x), O.f32_to_bf16_bits(x))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("zp_kind", ["zero", "const", "random"])
@pytest.mark.parametrize("scale_kind", ["pow2", "bf16", "f32"])
def test_pack_exact_matches_oracle(bits, zp_kind, scale_kind):
    rng = np.random.default_rng(bits)
    n, k, gs = 16, 256, 64
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    codes = rng.integers(lo, hi + 1, size=(n, k)).astype(np.int32)
    s = (rng.random((n, k // gs)).astype(np.float32) + 0.5) * 0.03
    if scale_kind == "pow2":
        s = np.exp2(rng.integers(-8, 2, size=s.shape)).astype(np.float32)
    elif scale_kind == "bf16":
        s = O.round_bf16(s)
    zp = {"zero": np.zeros((n, k // gs), np.int32), "const": np.full((n, k // gs), 3, np.int32),
          "random": rng.integers(lo, hi + 1, (n, k // gs)).astype(np.int32)}[zp_kind]
    for kind in (None, "bf16"):
        w, sc, bi = P.pack_exact(codes, s, zp, bits, scale_kind=kind)
        ow, os_, ob, odt = O.pack_exact(codes, s, zp, bits, narrow=kind)
        np.testing.assert_array_equal(w, ow)
        assert P.float_kind(sc) == odt and P.float_kind(bi) == odt
        np.testing.assert_array_equal(P.as_f32(sc), os_)
        np.testing.assert_array_equal(P.as_f32(bi), ob)


def test_width_policy_cases():
    """reference tests/test_qmm.py:155-171."""
    rng = np.random.default_rng(1)
    codes = rng.integers(-8, 8, size=(8, 128)).astype(np.int32)
    scale = np.exp2(rng.integers(-6, 0, size=(8, 1))).astype(np.float32)
    _, s, b = P.pack_exact(codes, scale, None, 4, scale_kind="bf16")
    assert isinstance(s, P.BF16Array) and isinstance(b, P.BF16Array)
    scale = rng.random((8, 1)).astype(np.float32) + 1.0
    _, s, b = P.pack_exact(codes, scale, np.full((8, 1), 3, np.int32), 4, scale_kind="bf16")
    assert s.dtype == np.float32 and b.dtype == np.float32


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
def test_mxfp4_codes(kind):
    codes = np.tile(np.arange(16, dtype=np.uint8), 8).reshape(4, 32)
    vals = E2M1[codes]
    arg = {"f32": vals, "f16": vals.astype(np.float16), "bf16": P.BF16Array.from_f32(vals)}[kind]
    np.testing.assert_array_equal(P.mxfp4_codes(arg), codes)
    np.testing.assert_array_equal(
        P.mxfp4_codes(np.array([[0.0, -0.0] * 16], np.float32)), np.array([[0, 8] * 16], np.uint8))


@pytest.mark.parametrize("bad", [0.7, 5.0, 8.0, 0.25, np.nan])
def test_mxfp4_codes_rejects(bad):
    vals = np.concatenate([E2M1[:8], np.array([bad] * 8, np.float32)])
    with pytest.raises(P.Reject):
        P.mxfp4_codes(vals.reshape(1, 16))
    with pytest.raises(P.Reject):
        P.mxfp4_codes(np.zeros((1, 16), np.float64))


@pytest.mark.parametrize("byte", [1, 100, 127, 200, 254])
def test_scale_bytes_ok(byte):
    scale = np.full((2, 4), np.exp2(float(byte) - 127.0), np.float32)
    np.testing.assert_array_equal(P.mxfp4_scale_bytes(scale), np.full((2, 4), byte, np.uint8))


@pytest.mark.parametrize("bad", [3.0, 0.0, -2.0, np.inf, np.nan, 1.5e-38])
def test_scale_bytes_rejects(bad):
    with pytest.raises(P.Reject):
        P.mxfp4_scale_bytes(np.array([[1.0, float(bad)]], np.float32))


def test_group_logic_matches_oracle():
    rng = np.random.default_rng(3)
    k = 256
    for gs in (16, 32, 64, 128):
        m = rng.random((4, k // gs)).astype(np.float32).repeat(gs, axis=1)
        z = rng.integers(-3, 4, (4, k // 32)).astype(np.int8).repeat(32, axis=1)
        assert P.pick_group(k, m, None) == O.pick_group(k, m, None)
        assert P.pick_group(k, m, z) == O.pick_group(k, m, z)
        assert P.pick_group(k, P.BF16Array.from_f32(m), None) == O.pick_group(k, O.round_bf16(m), None)
    assert P.pick_group(96, np.ones((2, 96), np.float32), None) == 32
    assert P.pick_group(48, np.ones((2, 48), np.float32), None) is None


def test_regroup_matches_oracle_and_invariants():
    rng = np.random.default_rng(4)
    k = 256
    heads = rng.random((8, 4)).astype(np.float32)
    smap = heads[:, np.arange(k) % 4]
    zmap = rng.integers(-3, 4, (8, 4)).astype(np.int8)[:, np.arange(k) % 4]
    for maps in ([smap, None], [smap, zmap], [P.BF16Array.from_f32(smap), zmap]):
        perm = P.regroup(k, maps)
        omaps = [O.round_bf16(smap) if isinstance(m, P.BF16Array) else m for m in maps]
        np.testing.assert_array_equal(perm, O.regroup(k, omaps))
        assert sorted(perm.tolist()) == list(range(k))
        assert P.pick_group(k, P.take_k(maps[0], perm), None) == 64
    grouped = rng.random((4, 4)).astype(np.float32).repeat(64, axis=1)
    assert P.regroup(k, [grouped]) is None
    assert P.regroup(k, [rng.random((4, k)).astype(np.float32)]) is None
    split = np.concatenate([np.full((2, 129), 1.0), np.full((2, 127), 2.0)], 1).astype(np.float32)
    assert P.regroup(k, [split]) is None
    dup = np.array([[1.0, 2.0, 1.0, 3.0]], np.float32)[:, np.arange(k) % 4]
    perm = P.regroup(k, [dup])
    assert perm is not None and P.pick_group(k, dup[:, perm], None) is not None
