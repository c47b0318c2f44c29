"""Pins the CPU oracle against the reference's known-answer vectors, against
independent formulations, and against library routines.  None of these checks
re-types the oracle's own formula: each has a second source of truth."""

import json
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import qmm_oracle as O
from oracle import c_oracle as C

GOLD = os.path.join(os.path.dirname(__file__), "golden")


# ---------------------------------------------------------------- bf16 ----

def test_bf16_round_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([
        rng.standard_normal(4096).astype(np.float32) * 3,
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.4e38, -3.4e38,
                  np.inf, -np.inf, 1e-40, 65504.0], np.float32),
        # exact ties: 1 + 2^-8 (even below -> down), 1 + 3*2^-8 (odd -> up)
        np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], np.float32)])
    got = O.f32_to_bf16_bits(x)
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(
        O.bf16_bits_to_f32(got),
        torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    assert O.round_bf16(np.float32(1.0 + 2.0 ** -8)) == np.float32(1.0)
    assert O.round_bf16(np.float32(1.0 + 3 * 2.0 ** -8)) == np.float32(1.0 + 2.0 ** -6)


# ----------------------------------------------------------- layout (A1) ----

def test_pack_layout_hand_computed_nibble_words():
    """reference tests/test_qmm_mxfp4.py:162-174: element i at bits [4i,4i+4)."""
    codes = np.arange(32, dtype=np.uint8) % 16
    got = O.pack_codes(codes.reshape(1, 32), 4)
    want = [sum(int(codes[8 * w + i]) << (4 * i) for i in range(8)) for w in range(4)]
    assert want[0] == 0x76543210 and want[1] == 0xFEDCBA98
    np.testing.assert_array_equal(got[0], np.array(want, np.uint32))


def test_pack_layout_literal_fixture():
    with open(os.path.join(GOLD, "layout_kat.json")) as f:
        kat = json.load(f)
    for case in kat["pack"]:
        codes = np.array(case["codes"], np.uint32)
        want = np.array([int(w, 16) for w in case["words"]], np.uint32)
        np.testing.assert_array_equal(O.pack_codes(codes, case["bits"]), want)
        np.testing.assert_array_equal(O.unpack_codes(want, case["bits"]),
                                      codes & ((1 << case["bits"]) - 1))


@pytest.mark.parametrize("bits", [2, 4, 8, 16])
@pytest.mark.parametrize("shape", [(1, 32), (5, 128), (3, 4, 64)])
def test_pack_codes_vs_bitstream_writer(bits, shape):
    """reference tests/test_qmm.py:76-83 shapes; second source = per-bit writer."""
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 1 << bits, size=shape).astype(np.uint32)
    got = O.pack_codes(codes, bits)
    np.testing.assert_array_equal(got, O.pack_codes_bitstream(codes, bits))
    np.testing.assert_array_equal(O.unpack_codes(got, bits), codes)
    if bits <= 8:
        np.testing.assert_array_equal(C.unpack_codes(got, bits), codes)


def test_pack_codes_masks_out_of_range_and_rejects_bad_widths():
    codes = np.array([[0x1F, 0x23] + [0] * 6], np.uint32)
    assert O.pack_codes(codes, 4)[0, 0] == 0x3F
    with pytest.raises(ValueError):
        O.pack_codes(np.zeros((1, 32), np.uint32), 3)
    with pytest.raises(ValueError):
        O.pack_codes(np.zeros((1, 12), np.uint32), 4)


def test_u32_words_and_checkpoint_bytes_are_the_same_bytes():
    """low nibble of byte j = element 2j (reference tests/test_qmm_mxfp4.py:80-81)."""
    rng = np.random.default_rng(1)
    codes = rng.integers(0, 16, size=(3, 64)).astype(np.uint8)
    words = O.pack_codes(codes, 4)
    np.testing.assert_array_equal(words.view(np.uint8), O.pack_blocks(codes))


# ------------------------------------------------------------- fma / A3 ----

def _fma_exact(a, b, c):
    """float32 fma by exact rational arithmetic + one rounding (tiny inputs)."""
    v = Fraction(float(a)) * Fraction(float(b)) + Fraction(float(c))
    if v == 0:
        return np.float32(0.0)
    # round the exact rational to float32: go through the two f32 neighbours
    approx = np.float32(float(v))
    cands = {approx, np.nextafter(approx, np.float32(np.inf)),
             np.nextafter(approx, np.float32(-np.inf))}
    best = None
    for cnd in cands:
        if not np.isfinite(cnd):
            continue
        d = abs(Fraction(float(cnd)) - v)
        even = (int(np.float32(cnd).view(np.uint32)) & 1) == 0
        key = (d, 0 if even else 1)
        if best is None or key < best[0]:
            best = (key, np.float32(cnd))
    return best[1]


def test_fma_f32_is_correctly_rounded():
    rng = np.random.default_rng(2)
    n = 400
    s = (rng.random(n).astype(np.float32) + 0.5) * 0.03
    q = rng.integers(0, 256, n).astype(np.float32)
    b = -(s * rng.integers(0, 200, n).astype(np.float32))
    # adversarial: bias huge against the product, and exact cancellation
    s[:8] = np.float32(1.0000001)
    q[:8] = np.arange(8)
    b[:8] = np.float32(16777216.0)
    b[8:16] = -(s[8:16] * q[8:16])
    got = O.fma_f32(s, q, b)
    want = np.array([_fma_exact(*t) for t in zip(s, q, b)], np.float32)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def _scale_kind(kind, shape, rng):
    s = (rng.random(shape).astype(np.float32) + 0.5) * 0.03
    if kind == "pow2":
        return np.exp2(rng.integers(-8, 2, size=shape)).astype(np.float32)
    if kind == "bf16":
        return O.round_bf16(s)
    return s


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("zp_kind", ["zero", "const", "random"])
@pytest.mark.parametrize("scale_kind", ["pow2", "bf16", "f32"])
def test_pack_exact_exactness_matrix(bits, gs, zp_kind, scale_kind):
    """reference tests/test_qmm.py:96-132: dequant(pack_exact) vs float32
    scale*(code-zp); exact for zp==0 or pow2/bf16 scales, else rel<1e-5."""
    rng = np.random.default_rng(bits * 100 + gs)
    n, k = 16, 256
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    codes = rng.integers(lo, hi + 1, size=(n, k)).astype(np.int32)
    codes[0, :4] = [lo, hi, 0, -1]
    ng = k // gs
    scale = _scale_kind(scale_kind, (n, ng), rng)
    if zp_kind == "zero":
        zp = np.zeros((n, ng), np.int32)
    elif zp_kind == "const":
        zp = np.full((n, ng), 3, np.int32)
    else:
        zp = rng.integers(lo, hi + 1, size=(n, ng)).astype(np.int32)
    want = scale.repeat(gs, axis=1) * (codes.astype(np.float32)
                                       - zp.repeat(gs, axis=1).astype(np.float32))
    w, s, b, _ = O.pack_exact(codes, scale, zp, bits)
    got = O.dequant_affine(w, s, b, gs, bits)
    assert got.shape == want.shape
    if zp_kind == "zero" or scale_kind in ("pow2", "bf16"):
        np.testing.assert_array_equal(got, want)
    else:
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-5
    # the C oracle agrees bit for bit (f32 tables)
    np.testing.assert_array_equal(C.dequant(w, s, b, gs, bits, "affine"), got)


@pytest.mark.parametrize("shift", [0, 8, -20])
def test_pack_exact_arbitrary_code_offset(shift):
    """reference tests/test_qmm.py:135-152."""
    rng = np.random.default_rng(2)
    codes = rng.integers(-8, 8, size=(4, 128)).astype(np.int32) + shift
    scale = O.round_bf16((rng.random((4, 1)).astype(np.float32) + 0.5) * 0.1)
    want = scale * codes.astype(np.float32)
    w, s, b, _ = O.pack_exact(codes, scale, None, 4, offset=-int(codes.min()))
    np.testing.assert_array_equal(O.dequant_affine(w, s, b, 128, 4), want)


def test_pack_exact_width_policy():
    """reference tests/test_qmm.py:155-171."""
    rng = np.random.default_rng(1)
    codes = rng.integers(-8, 8, size=(8, 128)).astype(np.int32)
    scale = np.exp2(rng.integers(-6, 0, size=(8, 1))).astype(np.float32)
    _, s, b, dt = O.pack_exact(codes, scale, None, 4, narrow="bf16")
    assert dt == "bf16"
    np.testing.assert_array_equal(b, -8 * scale)
    scale = (rng.random((8, 1)).astype(np.float32) + 1.0)
    zp = np.full((8, 1), 3, np.int32)
    assert O.pack_exact(codes, scale, zp, 4, narrow="bf16")[3] == "f32"
    assert O.pack_exact(codes, scale, zp, 4, narrow="bf16", width="source")[3] == "bf16"
    assert O.pack_exact(codes, np.exp2(-3.0) * np.ones((8, 1), np.float32), None, 4,
                        narrow="bf16", width="f32")[3] == "f32"


def test_baseline_bias_makes_the_bf16_tile_one_rounding_of_an_exact_product():
    """With b = -8*s the f32 FMA is exact, so the bf16 tile equals
    bf16(s*(q-8)) -- the literal chain's value."""
    rng = np.random.default_rng(5)
    s = O.round_bf16(rng.uniform(0.005, 0.02, (8, 4)).astype(np.float32))
    b = -8 * s
    codes = rng.integers(0, 16, (8, 256)).astype(np.uint8)
    w = O.pack_codes(codes, 4)
    f = O.dequant_affine(w, s, b, 64, 4)
    want64 = s.astype(np.float64).repeat(64, 1) * (codes.astype(np.float64) - 8)
    np.testing.assert_array_equal(f.astype(np.float64), want64)       # exact in f32
    tile = O.dequant_affine_bf16(w, s, b, 64, 4)
    want = torch.from_numpy(want64).to(torch.bfloat16).float().numpy()
    np.testing.assert_array_equal(tile, want)
    s16, b16 = O.f32_to_bf16_bits(s), O.f32_to_bf16_bits(b)
    np.testing.assert_array_equal(C.dequant(w, s16, b16, 64, 4, "affine", True), tile)


# --------------------------------------------------------------- MXFP4 ----

E2M1 = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
                 -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], np.float32)


def _random_mxfp4(shape_nk, rng, exp_lo=118, exp_hi=132):
    """reference tests/test_qmm_mxfp4.py:100-108 generator."""
    *lead, k = shape_nk
    codes = rng.integers(0, 16, size=tuple(lead) + (k,)).astype(np.uint8)
    codes.reshape(-1, k)[0, :16] = np.arange(16)
    sb = rng.integers(exp_lo, exp_hi, size=tuple(lead) + (k // 32,)).astype(np.uint8)
    return codes, O.pack_blocks(codes), sb


def test_e2m1_grid_is_the_published_table():
    np.testing.assert_array_equal(O.E2M1.view(np.uint32), E2M1.view(np.uint32))


@pytest.mark.parametrize("shape", [(4, 64), (3, 2, 128)])
def test_mxfp4_table_and_arithmetic_decoders_agree_bitwise(shape):
    rng = np.random.default_rng(7 + sum(shape))
    _, blocks, sb = _random_mxfp4(shape, rng)
    a = O.dequant_mxfp4(blocks, sb)
    b = O.dequant_mxfp4_arith(blocks, sb)
    np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
    # exact in bf16 too (one mantissa bit) -- reference tests/test_qmm_mxfp4.py:250-262
    np.testing.assert_array_equal(O.round_bf16(a), a)
    flat = blocks.reshape(-1, blocks.shape[-1])
    got = C.dequant(flat.view(np.uint32), sb.reshape(flat.shape[0], -1), None, 32, 4, "mxfp4")
    np.testing.assert_array_equal(got.view(np.uint32), a.reshape(got.shape).view(np.uint32))


def test_mxfp4_decode_matches_torch_fp4_and_e8m0_dtypes():
    if not (hasattr(torch, "float4_e2m1fn_x2") and hasattr(torch, "float8_e8m0fnu")):
        pytest.skip("torch lacks the fp4 / e8m0 dtypes")
    sb = np.array([1, 100, 127, 200, 254], np.uint8)
    got = O.e8m0_to_f32(sb)
    try:
        want = torch.from_numpy(sb).view(torch.float8_e8m0fnu).float().numpy()
    except Exception as e:   # conversion kernel absent on this build
        pytest.skip(f"torch cannot convert e8m0 on CPU: {e}")
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("kind", ["f32", "bf16", "f16"])
def test_mxfp4_codes_recovers_every_code(kind):
    """reference tests/test_qmm_mxfp4.py:116-124."""
    codes = np.tile(np.arange(16, dtype=np.uint8), 8).reshape(4, 32)
    vals = E2M1[codes]
    arg = {"f32": vals, "f16": vals.astype(np.float16),
           "bf16": O.f32_to_bf16_bits(vals)}[kind]
    np.testing.assert_array_equal(O.mxfp4_codes(arg, kind), codes)


def test_mxfp4_codes_keeps_the_sign_of_zero():
    vals = np.array([[0.0, -0.0] * 16], np.float32)
    np.testing.assert_array_equal(O.mxfp4_codes(vals), np.array([[0, 8] * 16], np.uint8))


@pytest.mark.parametrize("byte", [1, 100, 127, 200, 254])
def test_mxfp4_scale_bytes_round_trip(byte):
    scale = np.full((2, 4), np.exp2(float(byte) - 127.0), np.float32)
    np.testing.assert_array_equal(O.mxfp4_scale_bytes(scale), np.full((2, 4), byte, np.uint8))
    np.testing.assert_array_equal(O.e8m0_to_f32(np.uint8(byte)), scale[0, 0])


@pytest.mark.parametrize("bad", [3.0, 0.0, -2.0, np.inf, np.nan, 1.5e-38])
def test_mxfp4_scale_bytes_rejects(bad):
    with pytest.raises(O.Reject):
        O.mxfp4_scale_bytes(np.array([[1.0, float(bad)]], np.float32))


@pytest.mark.parametrize("bad", [0.7, 5.0, 8.0, 0.25, np.nan])
def test_mxfp4_codes_rejects_off_grid(bad):
    vals = np.concatenate([E2M1[:8], np.array([bad] * 8, np.float32)])
    with pytest.raises(O.Reject):
        O.mxfp4_codes(vals.reshape(1, 16))


# --------------------------------------------------------- group logic ----

def test_group_const_and_pick_group():
    k = 256
    rng = np.random.default_rng(3)
    for gs in (32, 64, 128):
        heads = rng.random((4, k // gs)).astype(np.float32)
        m = heads.repeat(gs, axis=1)
        assert O.group_const(m, gs) and O.pick_group(k, m, None) == gs
        np.testing.assert_array_equal(O.group_heads(m, gs), heads)
        z = rng.integers(-3, 4, (4, k // 32)).astype(np.float32).repeat(32, axis=1)
        assert O.pick_group(k, m, z) == 32
    m = rng.random((4, k // 16)).astype(np.float32).repeat(16, axis=1)
    assert O.pick_group(k, m, None) is None          # block 16 -> no legal size
    assert O.pick_group(96, np.ones((2, 96), np.float32), None) == 32   # 96 % 64 != 0
    assert O.pick_group(48, np.ones((2, 48), np.float32), None) is None


def _check_perm(k, maps, perm):
    assert sorted(perm.tolist()) == list(range(k))
    for m in maps:
        assert O.pick_group(k, np.asarray(m)[..., perm], None) is not None


def test_regroup_uninterleaves_and_is_stable():
    """Groups interleaved h-major vs n-major (reference tests/test_qmm.py:408-501)."""
    rng = np.random.default_rng(4)
    n_, h = 4, 64                      # K = 256; canonical axis runs h-major
    k = n_ * h
    heads = rng.random((8, n_)).astype(np.float32)
    # column j = hh*n_ + nn belongs to group nn
    smap = heads[:, np.arange(k) % n_]
    perm = O.regroup(k, [smap, None])
    _check_perm(k, [smap], perm)
    # stable: members of a cluster keep their relative order
    ids = np.arange(k) % n_
    for g in range(n_):
        members = perm[ids[perm] == g]
        assert np.all(np.diff(members) > 0)
    # clusters laid out in first-occurrence order
    np.testing.assert_array_equal(ids[perm], np.repeat(np.arange(n_), h))


def test_regroup_returns_none_cases():
    """reference tests/test_qmm.py:510-571."""
    rng = np.random.default_rng(5)
    k = 256
    m = rng.random((4, k // 64)).astype(np.float32).repeat(64, axis=1)
    assert O.regroup(k, [m]) is None                       # already grouped
    assert O.regroup(k, [rng.random((4, k)).astype(np.float32)]) is None   # all distinct
    split = np.concatenate([np.full((2, 129), 1.0), np.full((2, 127), 2.0)], 1).astype(np.float32)
    assert O.regroup(k, [split]) is None                   # 129/127 split
    # duplicate groups merge into one double-length run: still legal
    heads = np.array([[1.0, 2.0, 1.0, 3.0]], np.float32)
    inter = heads[:, np.arange(k) % 4]
    perm = O.regroup(k, [inter])
    _check_perm(k, [inter], perm)


# ---------------------------------------------------------- the products ----

@pytest.mark.parametrize("mode,bits", [("affine", 4), ("affine", 8), ("mxfp4", 4)])
def test_qmm_equals_library_matmul_on_dequantized_weight(mode, bits):
    rng = np.random.default_rng(11)
    m, n, k = 5, 48, 256
    x = O.round_bf16(rng.standard_normal((m, k)).astype(np.float32))
    if mode == "affine":
        codes = rng.integers(0, 1 << bits, (n, k)).astype(np.uint8)
        words = O.pack_codes(codes, bits)
        s = O.round_bf16(rng.uniform(0.005, 0.02, (n, k // 64)).astype(np.float32))
        b = -(1 << (bits - 1)) * s
        wd = s.repeat(64, 1).astype(np.float64) * (codes.astype(np.float64) - (1 << (bits - 1)))
        sc, bc = O.f32_to_bf16_bits(s), O.f32_to_bf16_bits(b)
    else:
        codes, blocks, sb = _random_mxfp4((n, k), rng)
        words, s, b = blocks.view(np.uint32), sb, None
        wd = E2M1[codes].astype(np.float64) * np.exp2(sb.astype(np.float64) - 127).repeat(32, 1)
        sc, bc = sb, None
    want = torch.matmul(torch.from_numpy(x).double(), torch.from_numpy(wd).T).numpy()
    got = O.qmm(x, words, s, b, 64, bits, mode)
    assert O.rel_l2(got, want) < 1e-7
    got_c = C.qmm(O.f32_to_bf16_bits(x), words, sc, bc, 64, bits, mode)
    assert O.rel_l2(got_c, want) < 1e-6
    # transposed-operand mistake would fail: x @ w (no transpose) has another shape/values
    assert got.shape == (m, n)


def test_gather_and_grouped_forms_against_brute_force():
    rng = np.random.default_rng(12)
    t, topk, e, n, k = 6, 2, 4, 16, 128
    x = O.round_bf16(rng.standard_normal((t, k)).astype(np.float32))
    codes = rng.integers(0, 16, (e, n, k)).astype(np.uint8)
    words = O.pack_codes(codes, 4)
    s = O.round_bf16(rng.uniform(0.005, 0.02, (e, n, k // 64)).astype(np.float32))
    b = -8 * s
    wd = s.repeat(64, 2).astype(np.float64) * (codes.astype(np.float64) - 8)
    _, experts = O.route_top_k(rng.standard_normal((t, e)), topk)
    experts[0] = [3, 3 - 1]           # leave expert structure arbitrary
    lhs = np.repeat(np.arange(t), topk)
    rhs = experts.reshape(-1)
    got = O.gather_qmm(x[:, None, :], words, s, b, lhs, rhs)
    for p in range(t * topk):          # brute force, pair by pair, element by element
        for j in range(n):
            want = float(np.dot(x[lhs[p]].astype(np.float64), wd[rhs[p], j]))
            assert abs(got[p, 0, j] - want) <= 1e-6 * max(1.0, abs(want))
    order, tok, ro = O.sort_pairs_by_expert(experts, e)
    assert ro[0] == 0 and ro[-1] == t * topk and np.all(np.diff(ro) >= 0)
    np.testing.assert_array_equal(np.sort(order), np.arange(t * topk))
    assert np.all(np.diff(rhs[order]) >= 0)
    yg = O.grouped_qmm(x[tok], words, s, b, ro)
    np.testing.assert_allclose(yg, got[order, 0], rtol=0, atol=0)
    yc = C.grouped_qmm(O.f32_to_bf16_bits(x[tok]), words, O.f32_to_bf16_bits(s),
                       O.f32_to_bf16_bits(b), ro, 64, 4, "affine")
    assert O.rel_l2(yc, yg) < 1e-6


def test_router_top_k():
    logits = np.array([[0.0, 2.0, 1.0, -1.0], [1.0, 1.0, 0.0, 0.0]])
    w, idx = O.route_top_k(logits, 2)
    np.testing.assert_array_equal(idx, [[1, 2], [0, 1]])
    p = np.exp(logits[0]) / np.exp(logits[0]).sum()
    np.testing.assert_allclose(w[0], [p[1], p[2]], rtol=1e-6)
