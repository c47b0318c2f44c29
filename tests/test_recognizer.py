"""The quantized-matmul recognizer on the host: StableHLO text -> structural
match -> first-execute verification and packing, with the accept / reject
catalogue and the exact counter expectations of the reference's own tests
(reference tests/test_qmm.py:285-373 accept, :606-735 fallbacks, :408-501
regrouping, :768-802 decode loop; tests/test_qmm_mxfp4.py:339-380, :536-668).
No GPU: `emit` is replaced by an oracle-backed stand-in where a whole program
has to run."""

import numpy as np
import pytest

import stablehlo_text as T
from metaljax_amd import engine, interpreter as I, ir, packing, packs, qmm
from oracle import qmm_oracle as O


@pytest.fixture(autouse=True)
def _fresh():
    qmm.reset_stats()
    qmm._BUILT.clear()
    qmm._SHARED.clear()
    yield


def host_args_dense(packed, scale, zero, g_idx, x, el="bf16"):
    return [I.from_numpy(packed), I.from_numpy(scale, el), I.from_numpy(zero),
            I.from_numpy(g_idx), I.from_numpy(x, el)]


def _without_a_gpu(fn):
    """Packs are uploaded when a GPU is visible; the kernel stand-ins read them as host arrays."""
    import torch
    return pytest.mark.skipif(torch.cuda.is_available(),
                              reason="stands in for the kernels on a machine without a GPU")(fn)


def pack_tables_f32(pk):
    s = pk.scales.to_f32() if isinstance(pk.scales, packing.BF16Array) else np.asarray(pk.scales, np.float32)
    b = None
    if pk.biases is not None:
        b = pk.biases.to_f32() if isinstance(pk.biases, packing.BF16Array) else np.asarray(pk.biases, np.float32)
    return s, b


def dequant_pack(pk):
    s, b = pack_tables_f32(pk)
    if pk.mode == "mxfp4":
        return O.dequant_mxfp4(np.ascontiguousarray(pk.w).view(np.uint8), np.asarray(pk.scales))
    return O.dequant_affine(np.asarray(pk.w), s, b, pk.gs, pk.bits)


def oracle_emit(interp, m, env):
    """Stand-in for the device `emit`: the same plumbing, the product from the oracle."""
    pk = m.packs[0]
    x = I.host(env[m.lhs]).a
    x = np.transpose(x, m.lperm).reshape(([m.B] if m.bshape else []) + [m.M, m.K])
    if m.has_perm:
        x = x[..., np.asarray(pk.perm)]
    w = dequant_pack(pk)
    y = np.matmul(x.astype(np.float32), np.swapaxes(w, -1, -2))
    if m.swapped:
        y = np.swapaxes(y, -1, -2).reshape(m.bshape + m.nshape + m.mshape)
    else:
        y = y.reshape(m.bshape + m.mshape + m.nshape)
    return [I.settle(y, m.out_dtype)]


# ------------------------------------------------------------------ accept ---

@pytest.mark.parametrize("block,gs", [(128, 128), (64, 64), (32, 32), (-1, 128)])
def test_dense_subchannel_is_recognized_and_packed_exactly(block, gs):
    k, n, m = 256, 128, 4
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, block)
    ng = scale.shape[0]
    x = T.bf16_round(np.random.default_rng(3).standard_normal((m, k)).astype(np.float32) * 0.5)
    ex = engine.compile_program(T.dense_sub(k, n, ng, m))
    st = qmm.analyze(ex.interp)
    assert len(st.matches) == 1 and qmm.stats()["recognized"] == 1
    mt = st.matches[0]
    assert (mt.M, mt.K, mt.N, mt.B, mt.mode, mt.swapped) == (m, k, n, 1, "affine", False)
    assert mt.arg_indices == (0, 1, 2, 3)                 # everything but the activation
    assert qmm.emit_reads(mt) == (mt.lhs,) and qmm.emit_bytes(mt) == m * k * 2
    args = host_args_dense(packed, scale, zero, g_idx, x)
    assert qmm.prologue(ex.interp, args) is False
    assert qmm.stats() == {**{k_: 0 for k_ in qmm.STATS}, "recognized": 1, "packs": 1}
    pk = mt.packs[0]
    assert (pk.gs, pk.bits, pk.mode, pk.perm) == (gs, 4, "affine", None)
    # q_hat = code + 8, biases = -scale*(8 + zero): the reconstruction is the
    # exact float32 weight whenever the bias is representable (always without
    # zero points), and within 1e-5 otherwise
    got = dequant_pack(pk)                                # [N, K]
    if block < 0:
        assert isinstance(pk.scales, packing.BF16Array)   # lossless: source width kept
        np.testing.assert_array_equal(got, wref.T)
    else:
        np.testing.assert_allclose(got, wref.T, rtol=1e-5, atol=1e-7)
    codes = O.unpack_codes(np.asarray(pk.w), 4)
    np.testing.assert_array_equal(codes.astype(np.int64) - 8, q.T)


def test_int8_codes_take_eight_bits():
    """Codes that need all 8 bits (reference tests/test_qmm.py:296-313)."""
    k, n, m = 128, 64, 2
    q, _, scale, zero, g_idx, wref = T.quantize(k, n, 64, seed=5, bits=8)
    ex = engine.compile_program(T.dense_i8_codes(k, n, 2, m))
    st = qmm.analyze(ex.interp)
    args = host_args_dense(q, scale, zero, g_idx, np.zeros((m, k), np.float32))
    qmm.prologue(ex.interp, args)
    pk = st.matches[0].packs[0]
    assert (pk.bits, pk.gs) == (8, 64) and qmm.stats()["packs"] == 1
    np.testing.assert_allclose(dequant_pack(pk), wref.T, rtol=1e-5, atol=1e-7)


def test_codes_in_0_15_use_their_own_offset():
    """Unsigned [0, 15] codes do not fit offset 8: the offset becomes -lo
    (reference tests/test_qmm.py:135-152)."""
    k, n, m = 128, 64, 2
    q, _, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=5)
    q = (q.astype(np.int16) + 8).astype(np.int8)            # [0, 15]
    ex = engine.compile_program(T.dense_i8_codes(k, n, 2, m))
    st = qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, host_args_dense(q, scale, zero, g_idx, np.zeros((m, k), np.float32)))
    pk = st.matches[0].packs[0]
    assert pk.bits == 4
    np.testing.assert_array_equal(O.unpack_codes(np.asarray(pk.w), 4), q.T.astype(np.uint8))
    gi = g_idx.astype(np.int32)
    want = scale[gi] * (q.astype(np.float32) - zero[gi].astype(np.float32))
    np.testing.assert_allclose(dequant_pack(pk), want.T, rtol=1e-5, atol=1e-7)


def test_perchannel_divide_form():
    k, n, m = 128, 64, 3
    q, packed, _, _, _, _ = T.quantize(k, n, -1, seed=2)
    scale = T.bf16_round(np.random.default_rng(9).uniform(8.0, 40.0, n).astype(np.float32))
    x = T.bf16_round(np.random.default_rng(4).standard_normal((m, k)).astype(np.float32))
    ex = engine.compile_program(T.dense_perchannel(k, n, m))
    st = qmm.analyze(ex.interp)
    assert [mm.recip for mm in st.matches] == [True]
    mt = st.matches[0]
    assert mt.root.name == "stablehlo.divide" and mt.arg_indices == (0, 1)
    args = [I.from_numpy(packed), I.from_numpy(scale, "bf16"), I.from_numpy(x, "bf16")]
    qmm.prologue(ex.interp, args)
    assert qmm.stats()["packs"] == 1 and qmm.stats()["fallbacks"] == 0
    pk = mt.packs[0]
    assert pk.gs == 128 and pk.bits == 4
    s, b = pack_tables_f32(pk)
    np.testing.assert_array_equal(s[:, 0], (np.float32(1.0) / scale).astype(np.float32))
    got = dequant_pack(pk)
    np.testing.assert_allclose(got, (q.astype(np.float32) / scale).T, rtol=2e-7)


def test_int4_typed_weights_with_a_per_channel_scale():
    """Weights stored with the four-bit integer element type and one scale per
    output channel (reference tests/test_qmm.py:342-358): four-bit codes, one
    group spanning as much of K as a legal group size allows, exact."""
    k, n, m = 128, 64, 2
    rng = np.random.default_rng(50)
    codes = rng.integers(-8, 8, size=(k, n)).astype(np.int8)
    scale = T.bf16_round((rng.random(n).astype(np.float32) + 0.5) * 0.02)
    ex = engine.compile_program(T.dense_i4_perchannel(k, n, m))
    st = qmm.analyze(ex.interp)
    assert len(st.matches) == 1
    args = [I.from_numpy(codes, "i4"), I.from_numpy(scale, "bf16"), I.from_numpy(np.zeros((m, k), np.float32), "bf16")]
    qmm.prologue(ex.interp, args)
    assert qmm.stats()["recognized"] == 1 and qmm.stats()["packs"] == 1 and qmm.stats()["fallbacks"] == 0
    pk = st.matches[0].packs[0]
    assert pk.bits == 4 and pk.gs == 128
    np.testing.assert_array_equal(dequant_pack(pk), (codes.astype(np.float32) * scale).T)


@pytest.mark.parametrize("el", ["bf16", "f32"])
def test_mxfp4_chain_packs_bit_exactly(el):
    n, k, t = 48, 128, 5
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=1)
    x = T.bf16_round(np.random.default_rng(2).standard_normal((t, k)).astype(np.float32))
    ex = engine.compile_program(T.dense_mxfp4(n, k, t, el))
    st = qmm.analyze(ex.interp)
    assert [mm.mode for mm in st.matches] == ["mxfp4"]
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, el)]
    # the literal reconstruction is exact in the chain's own dtype
    env = dict(zip(ex.interp.main.body.args, args))
    lit = qmm._eval(ex.interp, st.matches[0].root.operands[1], env)
    np.testing.assert_array_equal(lit.a, w)
    qmm.prologue(ex.interp, args)
    # float32 chains are served like bf16 ones (the library splits float32
    # activations into exact bf16 terms)
    assert st.matches[0].act_dtype == el and not st.matches[0].disabled
    assert qmm.stats() == {**{k_: 0 for k_ in qmm.STATS}, "recognized": 1, "packs": 1, "mxfp4": 1}
    pk = st.matches[0].packs[0]
    np.testing.assert_array_equal(np.asarray(pk.w), O.pack_codes(codes, 4))
    np.testing.assert_array_equal(np.asarray(pk.scales), sb)
    assert pk.biases is None and pk.gs == 32 and pk.bits == 4
    np.testing.assert_array_equal(dequant_pack(pk), w)


def test_batched_expert_dot_keeps_the_expert_axis():
    e, n, k, t = 3, 32, 64, 4
    codes, blocks, sb, w = T.random_mxfp4((e, n, k), seed=7)
    x = T.bf16_round(np.random.default_rng(2).standard_normal((e, t, k)).astype(np.float32))
    ex = engine.compile_program(T.experts_mxfp4(e, n, k, t))
    st = qmm.analyze(ex.interp)
    mt = st.matches[0]
    assert (mt.B, mt.bshape, mt.M, mt.N, mt.K) == (e, [e], t, n, k)
    qmm.prologue(ex.interp, [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")])
    assert qmm.stats()["batched"] == 1 and qmm.stats()["mxfp4"] == 1
    pk = mt.packs[0]
    assert np.asarray(pk.w).shape == (e, n, k // 8) and np.asarray(pk.scales).shape == (e, n, k // 32)
    np.testing.assert_array_equal(dequant_pack(pk), w)


def test_ordinary_float_graph_recognizes_nothing():
    ex = engine.compile_program(T.float_dot(64, 32, 4))
    st = qmm.analyze(ex.interp)
    assert st.matches == [] and not st.active and qmm.stats()["recognized"] == 0


# ---------------------------------------------------------------- regroup ----

def test_interleaved_groups_are_fused_through_a_permutation():
    k, n, m, ng = 256, 64, 4, 2
    g_idx = (np.arange(k) % ng).astype(np.float32)          # groups interleaved along K
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, k // ng, seed=11, g_idx=g_idx)
    x = T.bf16_round(np.random.default_rng(3).standard_normal((m, k)).astype(np.float32))
    ex = engine.compile_program(T.dense_sub(k, n, ng, m))
    st = qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, host_args_dense(packed, scale, zero, g_idx, x))
    assert qmm.stats()["packs"] == 1 and qmm.stats()["perms"] == 1
    mt = st.matches[0]
    pk = mt.packs[0]
    assert mt.has_perm and mt.nvals == 4
    perm = np.asarray(pk.perm)
    assert sorted(perm.tolist()) == list(range(k))
    np.testing.assert_allclose(dequant_pack(pk), wref.T[:, perm], rtol=1e-5, atol=1e-7)


def _fused_and_literal(monkeypatch, text, args):
    """The program's first result with the recognized dot replaced by the
    oracle-backed stand-in, and from the literal chain."""
    literal = I.host(I.Interpreter(text).run(args)[0]).a
    monkeypatch.setattr(qmm, "emit", oracle_emit)
    ex = engine.compile_program(text)
    st = qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, args)
    (y,) = ex.interp.run(args)
    return st, I.host(y).a, literal


def test_einsum_with_two_output_axes(monkeypatch):
    """`btd,dnh->btnh`: the weight is reshaped to [d, n, h] behind the chain
    and the dot keeps both N axes (reference tests/test_qmm.py:329-339)."""
    d, heads, hd, b, t = 256, 4, 32, 1, 2
    q, packed, scale, zero, g_idx, wref = T.quantize(d, heads * hd, 128, seed=7)
    x = T.bf16_round(np.random.default_rng(8).standard_normal((b, t, d)).astype(np.float32) * 0.3)
    st, fused, literal = _fused_and_literal(monkeypatch, T.einsum_sub(d, heads, hd, 2, b, t),
                                            host_args_dense(packed, scale, zero, g_idx, x))
    assert qmm.stats()["recognized"] == 1 and qmm.stats()["packs"] == 1 and qmm.stats()["perms"] == 0
    mt = st.matches[0]
    assert (mt.M, mt.K, mt.N) == (b * t, d, heads * hd) and list(mt.nshape) == [heads, hd]
    exact = np.einsum("btd,dnh->btnh", x, wref.reshape(d, heads, hd))
    assert fused.shape == exact.shape
    assert np.abs(fused - exact).max() <= 1.5 * np.abs(literal - exact).max() + 1e-6


@pytest.mark.parametrize("nh,h,block", [(8, 32, 128), (4, 64, 64), (16, 16, 128)])
def test_einsum_out_projection_interleaved_groups(monkeypatch, nh, h, block):
    """`btnh,nhd->btd` with the reversed pairing jax emits: the quantization
    groups of the n-major weight arrive interleaved along the canonical K, and
    a permutation of K (the same one on the activations) makes them contiguous
    (reference tests/test_qmm.py:409-426)."""
    d, b, t = 64, 1, 3
    rows = nh * h
    q, packed, scale, zero, g_idx, wref = T.quantize(rows, d, block, seed=100)
    x = T.bf16_round(np.random.default_rng(9).standard_normal((b, t, nh, h)).astype(np.float32) * 0.3)
    st, fused, literal = _fused_and_literal(monkeypatch, T.einsum_out_proj(nh, h, d, rows // block, b, t),
                                            host_args_dense(packed, scale, zero, g_idx, x))
    stats = qmm.stats()
    assert stats["recognized"] == 1 and stats["packs"] == 1 and stats["fallbacks"] == 0
    assert stats["perms"] == 1                              # n-major groups, h-major K: always interleaved
    exact = np.einsum("btnh,nhd->btd", x, wref.reshape(nh, h, d))
    assert np.abs(fused - exact).max() <= 1.5 * np.abs(literal - exact).max() + 1e-6


def test_identity_permutation_is_the_zero_overhead_path():
    """Groups that are already contiguous carry no permutation: three packed
    values, no `take` on the activations (reference tests/test_qmm.py:575-586)."""
    k, n, m = 256, 128, 4
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, 128, seed=124)
    x = np.zeros((m, k), np.float32)
    ex = engine.compile_program(T.dense_sub(k, n, 2, m))
    st = qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, host_args_dense(packed, scale, zero, g_idx, x))
    mt = st.matches[0]
    assert qmm.stats()["packs"] == 1 and qmm.stats()["perms"] == 0
    assert not mt.has_perm and mt.nvals == 3 and mt.packs[0].perm is None
    np.testing.assert_allclose(dequant_pack(mt.packs[0]), wref.T, rtol=1e-5, atol=1e-7)


def test_shuffled_g_idx_is_regrouped():
    """A g_idx that scatters each group's members across K still has equal
    groups of identical (scale, zero) columns: the permutation recovers them
    (reference tests/test_qmm.py:606-619)."""
    k, n, m, block = 256, 64, 2, 128
    rng = np.random.default_rng(12)
    g_idx = rng.permutation(np.arange(k) // block).astype(np.float32)
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, block, seed=13, g_idx=g_idx)
    ex = engine.compile_program(T.dense_sub(k, n, k // block, m))
    st = qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32)))
    assert qmm.stats()["packs"] == 1 and qmm.stats()["perms"] == 1 and qmm.stats()["fallbacks"] == 0
    pk = st.matches[0].packs[0]
    perm = np.asarray(pk.perm)
    assert sorted(perm.tolist()) == list(range(k))
    np.testing.assert_allclose(dequant_pack(pk), wref.T[:, perm], rtol=1e-5, atol=1e-7)


def test_second_weight_set_with_a_different_permutation():
    """Two weight sets whose groups interleave differently through one
    executable: the permutation is a packed value of the pack, so the second
    set must get its own (reference tests/test_qmm.py:472-501)."""
    k, n, m, ng = 256, 64, 2, 2
    ex = engine.compile_program(T.dense_sub(k, n, ng, m))
    st = qmm.analyze(ex.interp)
    x = np.zeros((m, k), np.float32)
    perms, wrefs, held = [], [], []
    for seed, g_idx in ((100, (np.arange(k) % ng)), (110, ((np.arange(k) // 2) % ng))):
        q, packed, scale, zero, g, wref = T.quantize(k, n, k // ng, seed=seed, g_idx=g_idx.astype(np.float32))
        held.append(host_args_dense(packed, scale, zero, g, x))
        qmm.prologue(ex.interp, held[-1])
        pk = st.matches[0].packs[0]
        perms.append(np.asarray(pk.perm).copy())
        np.testing.assert_allclose(dequant_pack(pk), wref.T[:, perms[-1]], rtol=1e-5, atol=1e-7)
    assert qmm.stats()["packs"] == 2 and qmm.stats()["perms"] == 2
    assert not np.array_equal(perms[0], perms[1])


# --------------------------------------------------------------- fallbacks ---

def _one_fallback(ex, args):
    st = qmm.analyze(ex.interp)
    assert len(st.matches) == 1
    changed = qmm.prologue(ex.interp, args)
    assert changed and st.matches[0].disabled and not st.active
    assert qmm.stats()["fallbacks"] == 1 and qmm.stats()["packs"] == 0


def test_group_of_16_falls_back():
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 16, seed=4)
    x = np.zeros((m, k), np.float32)
    ex = engine.compile_program(T.dense_sub(k, n, k // 16, m))
    _one_fallback(ex, host_args_dense(packed, scale, zero, g_idx, x))


def test_uneven_group_sizes_fall_back():
    """Groups of 129 and 127 columns line up on no legal group boundary: the
    literal chain runs (reference tests/test_qmm.py:622-634)."""
    k, n, m = 256, 64, 2
    g_idx = (np.arange(k) >= 129).astype(np.float32)
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 128, seed=13, g_idx=g_idx)
    ex = engine.compile_program(T.dense_sub(k, n, 2, m))
    _one_fallback(ex, host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32)))


def test_mxfp4_scales_over_blocks_of_sixteen_are_turned_down_at_analysis():
    """The block-scaled form has exactly one legal block: a scale that
    broadcasts one value per 16 elements is no MXFP4 weight, and no affine one
    either (its values are not integer codes); nothing is ever evaluated
    (reference tests/test_qmm_mxfp4.py:643-668)."""
    n, k, t = 48, 128, 2                                      # (N * K / 32 must not be the 256 of the scale table)
    text = T.dense_mxfp4(n, k, t)
    # the same chain with sixteen-wide blocks: [N, K/16] scale bytes, [N, K/16, 16] products
    narrow = (text.replace(f"tensor<{n}x{k // 32}x32x", f"tensor<{n}x{k // 16}x16x")
                  .replace(f"tensor<{n}x{k // 32}x", f"tensor<{n}x{k // 16}x")
                  .replace(f"tensor<{n * k // 32}x", f"tensor<{n * k // 16}x"))
    assert narrow != text
    ex = engine.compile_program(narrow)
    st = qmm.analyze(ex.interp)
    assert st.matches == [] and qmm.stats()["recognized"] == 0
    # ... and the program still runs literally
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=8)
    sb16 = np.repeat(sb, 2, axis=1)
    x = T.bf16_round(np.random.default_rng(8).standard_normal((t, k)).astype(np.float32) * 0.4)
    (y,) = ex.interp.run([I.from_numpy(blocks), I.from_numpy(sb16), I.from_numpy(x, "bf16")])
    exact = x @ w.T
    np.testing.assert_allclose(I.host(y).a, exact, rtol=2e-2, atol=2e-2 * np.abs(exact).max())


def test_off_grid_e2m1_value_falls_back():
    n, k, t = 16, 64, 2
    vt = list(T.E2M1) + [-v for v in T.E2M1]
    vt[3] = 1.25                                            # not an E2M1 value
    codes, blocks, sb, _ = T.random_mxfp4((n, k), seed=3)
    ex = engine.compile_program(T.dense_mxfp4(n, k, t, "bf16", vtable=vt))
    _one_fallback(ex, [I.from_numpy(blocks), I.from_numpy(sb),
                       I.from_numpy(np.zeros((t, k), np.float32), "bf16")])


def test_scale_byte_255_is_not_a_power_of_two():
    n, k, t = 16, 64, 2
    codes, blocks, sb, _ = T.random_mxfp4((n, k), seed=3)
    sb[2, 1] = 255                                          # NaN in the E8M0 table
    ex = engine.compile_program(T.dense_mxfp4(n, k, t))
    _one_fallback(ex, [I.from_numpy(blocks), I.from_numpy(sb),
                       I.from_numpy(np.zeros((t, k), np.float32), "bf16")])


@pytest.mark.parametrize("zero_value,wraps", [(3, False), (125, True)])
def test_integer_zero_point_subtraction_must_not_wrap(zero_value, wraps):
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=6)
    zero[:] = zero_value                                    # codes reach -8: -8-125 wraps in i8
    ex = engine.compile_program(T.dense_int_sub(k, n, k // 64, m))
    args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32))
    st = qmm.analyze(ex.interp)
    assert st.matches[0].sub_range == (-128, 127)
    if wraps:
        _one_fallback(ex, args)
    else:
        assert qmm.prologue(ex.interp, args) is False and qmm.stats()["packs"] == 1


def test_weight_with_a_second_consumer_is_not_rewritten():
    ex = engine.compile_program(T.dense_sub(128, 64, 2, 2, twice=True))
    st = qmm.analyze(ex.interp)
    assert st.matches == [] and qmm.stats()["recognized"] == 0


def test_donated_weight_is_not_rewritten():
    text = T.dense_sub(128, 64, 2, 2).replace(
        "%packed: tensor<128x32xi8>", "%packed: tensor<128x32xi8> {tf.aliasing_output = 0 : i32}")
    ex = engine.compile_program(text)
    assert ex.donated_params == [0]
    assert qmm.analyze(ex.interp).matches == []


def test_k_not_a_multiple_of_32_is_not_a_candidate():
    ex = engine.compile_program(T.dense_sub(48, 32, 1, 2))
    assert qmm.analyze(ex.interp).matches == []


def test_disabled_recognizer(monkeypatch):
    monkeypatch.setattr(qmm, "QMM_ENABLED", False)
    ex = engine.compile_program(T.dense_sub(128, 64, 2, 2))
    st = qmm.analyze(ex.interp)
    assert st.matches == [] and not st.active


# ------------------------------------------------------------ pack caching ---

def test_packs_are_keyed_by_buffer_identity_and_repack_storms_give_up(monkeypatch):
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=8)
    x = np.zeros((m, k), np.float32)
    ex = engine.compile_program(T.dense_sub(k, n, 2, m))
    args = host_args_dense(packed, scale, zero, g_idx, x)
    qmm.prologue(ex.interp, args)
    qmm.prologue(ex.interp, args)                           # same buffers: identity hit
    x2 = I.from_numpy(np.ones((m, k), np.float32), "bf16")
    qmm.prologue(ex.interp, args[:4] + [x2])                # a new activation is not a new weight
    assert qmm.stats()["packs"] == 1
    args2 = host_args_dense(packed.copy(), scale, zero, g_idx, x)
    qmm.prologue(ex.interp, args2)                          # new weight buffers: repack, no stale pack
    assert qmm.stats()["packs"] == 2 and ex.interp._qmm.matches[0].repacks == 2
    assert qmm.stats()["shared"] == 1                       # same bytes: the arrays are shared
    monkeypatch.setattr(packs, "MAX_REPACKS", 3)
    keep = []
    for i in range(3):
        keep.append(host_args_dense(packed.copy(), scale, zero, g_idx, x))
        qmm.prologue(ex.interp, keep[-1])
    assert ex.interp._qmm.matches[0].disabled and qmm.stats()["fallbacks"] == 1


@_without_a_gpu
def test_a_weight_tensor_rewritten_in_place_is_packed_again():
    """The reference's buffers are immutable, so a buffer's identity names its
    contents; a tensor can be refilled.  Packs (and the cross-executable build
    cache) also hold each source tensor's write counter."""
    import torch
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=8)
    _, packed2, _, _, _, _ = T.quantize(k, n, 64, seed=9)
    host_args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32))
    wt = torch.from_numpy(packed.copy())
    args = [wt] + host_args[1:]
    ex = engine.compile_program(T.dense_sub(k, n, 2, m))
    qmm.prologue(ex.interp, args)
    qmm.prologue(ex.interp, args)
    assert qmm.stats()["packs"] == 1
    first = ex.interp._qmm.matches[0].packs[0]
    wt.copy_(torch.from_numpy(packed2))                     # the same tensor object, other codes
    qmm.prologue(ex.interp, args)
    assert qmm.stats()["packs"] == 2 and qmm.stats()["build_hits"] == 0
    second = ex.interp._qmm.matches[0].packs[0]
    assert second is not first and not np.array_equal(np.asarray(second.w), np.asarray(first.w))
    ex2 = engine.compile_program(T.dense_sub(k, n, 2, m))   # another executable: the build cache's entry is the new one
    qmm.prologue(ex2.interp, args)
    assert qmm.stats()["build_hits"] == 1 and ex2.interp._qmm.matches[0].packs[0].w is second.w


def test_build_cache_serves_a_second_executable_over_the_same_buffers():
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=8)
    args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32))
    ex1 = engine.compile_program(T.dense_sub(k, n, 2, m))
    ex2 = engine.compile_program(T.dense_sub(k, n, 2, 8))    # another batch size, same weight chain
    qmm.prologue(ex1.interp, args)
    args8 = args[:4] + [I.from_numpy(np.zeros((8, k), np.float32), "bf16")]
    qmm.prologue(ex2.interp, args8)
    assert qmm.stats()["packs"] == 1 and qmm.stats()["build_hits"] == 1
    assert ex2.interp._qmm.matches[0].packs[0].w is ex1.interp._qmm.matches[0].packs[0].w
    # other buffers with the same structure do not hit
    ex3 = engine.compile_program(T.dense_sub(k, n, 2, m))
    qmm.prologue(ex3.interp, host_args_dense(packed.copy(), scale, zero, g_idx, np.zeros((m, k), np.float32)))
    assert qmm.stats()["packs"] == 2 and qmm.stats()["build_hits"] == 1


def test_pack_tables_are_bounded_and_zero_turns_them_off(monkeypatch):
    """METALJAX_QMM_BUILD_CACHE / METALJAX_QMM_SHARE are entry counts (reference
    qmm.py:1653, :2209-2211): 0 turns the table off, a full table is swept of
    its dead entries and dropped whole if that does not make room."""
    k, n, m = 128, 64, 2

    def packed_executable(seed):
        q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=seed)
        args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32))
        ex = engine.compile_program(T.dense_sub(k, n, 2, m))
        qmm.prologue(ex.interp, args)
        return ex, args

    monkeypatch.setattr(packs, "MAX_BUILT", 0)
    monkeypatch.setattr(packs, "MAX_SHARED", 0)
    ex1, args = packed_executable(1)
    ex2 = engine.compile_program(T.dense_sub(k, n, 2, m))
    qmm.prologue(ex2.interp, args)                                   # same buffers, other executable: built again
    ex3 = engine.compile_program(T.dense_sub(k, n, 2, m))
    qmm.prologue(ex3.interp, [I.HostArray(np.array(a.a, copy=True), a.el) for a in args])      # same bytes: no sharing
    st = qmm.stats()
    assert (st["packs"], st["build_hits"], st["shared"]) == (3, 0, 0) and not qmm._BUILT and not qmm._SHARED
    monkeypatch.setattr(packs, "MAX_BUILT", 2)
    monkeypatch.setattr(packs, "MAX_SHARED", 2)
    held = [packed_executable(seed) for seed in (2, 3)]
    assert len(qmm._BUILT) == 2 and len(qmm._SHARED) == 2
    del held[0]                                                       # its pack and buffers die: a dead entry
    import gc
    gc.collect()
    held.append(packed_executable(4))                                 # full: the sweep makes room, the live entry stays
    assert len(qmm._BUILT) == 2 and len(qmm._SHARED) == 2
    ex5 = engine.compile_program(T.dense_sub(k, n, 2, m))
    qmm.prologue(ex5.interp, held[0][1])
    assert qmm.stats()["build_hits"] == 1                             # executable 3's entry survived the sweep
    held.append(packed_executable(5))                                 # full of live entries: dropped whole
    assert len(qmm._BUILT) == 1 and len(qmm._SHARED) == 1


def test_different_weight_content_misses_the_build_cache():
    """Same shapes and types, different bytes in different buffers: the key
    names buffers by identity, so nothing is reused and each executable's pack
    holds its own weight (reference tests/test_qmm.py:1213-1243)."""
    k, n, m = 128, 64, 2
    packs_seen = []
    for seed in (42, 43):
        q, packed, scale, zero, g_idx, wref = T.quantize(k, n, 64, seed=seed, bf16=False)
        ex = engine.compile_program(T.dense_sub(k, n, 2, m, el="f32"))
        st = qmm.analyze(ex.interp)
        args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32), el="f32")
        qmm.prologue(ex.interp, args)
        packs_seen.append((st.matches[0].packs[0], wref, args))
    assert qmm.stats()["build_hits"] == 0 and qmm.stats()["packs"] == 2
    for pk, wref, _ in packs_seen:
        np.testing.assert_allclose(dequant_pack(pk), wref.T, rtol=1e-5, atol=1e-7)   # f32 scales, nonzero zero points: the exactness matrix of reference tests/test_qmm.py:117-132
    assert packs_seen[0][0].w is not packs_seen[1][0].w


def test_one_different_constant_misses_the_build_cache():
    """Same buffers, same shapes, one constant of the chain apart (the group
    count the indices are clamped to): a wrong hit would hand the second
    executable the first one's weight (reference tests/test_qmm.py:1247-1275)."""
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, 64, seed=45)
    args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32))
    text = T.dense_sub(k, n, 2, m)
    other = text.replace("%gns = stablehlo.constant dense<2>", "%gns = stablehlo.constant dense<3>")
    assert other != text
    ex1, ex2 = engine.compile_program(text), engine.compile_program(other)
    qmm.prologue(ex1.interp, args)
    qmm.prologue(ex2.interp, args)
    assert qmm.stats()["build_hits"] == 0 and qmm.stats()["packs"] == 2


def test_the_fused_dot_is_what_the_cost_model_charges():
    """`emit_reads` names exactly the activation, and `emit_bytes` is the
    packed operands plus activation and result -- far below the literal chain's
    traffic (reference tests/test_qmm.py:930-957 through qmm.py:2424-2466)."""
    k, n, m = 128, 128, 1
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 128, seed=40)
    ex = engine.compile_program(T.dense_sub(k, n, 1, m))
    st = qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32)))
    mt = st.matches[0]
    assert tuple(qmm.emit_reads(mt)) == (mt.lhs,)
    fused = qmm.emit_bytes(mt)
    literal = 3 * k * n * 2                                   # the dequantized weight written, re-read and multiplied
    assert 0 < fused < literal // 4, (fused, literal)


def test_fingerprint_reads_callee_bodies_not_their_names():
    """Two programs that differ only in the name of a private callee are the
    same weight chain (a build hit over the same buffers); one constant inside
    the callee's body apart, they are not (reference
    tests/test_qmm_mxfp4.py:895-928)."""
    n, k, t = 64, 128, 2
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=7)
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(np.zeros((t, k), np.float32), "bf16")]
    text = T.dense_mxfp4_rows(n, k, t)
    renamed = text.replace("@_take", "@_take_17")
    wrap = "%ns = stablehlo.constant dense<16> : tensor<i32>"
    assert renamed != text and wrap in text
    other_body = text.replace(wrap, "%ns = stablehlo.constant dense<32> : tensor<i32>")   # what a negative index wraps by
    ex1, ex2, ex3 = (engine.compile_program(x) for x in (text, renamed, other_body))
    qmm.prologue(ex1.interp, args)
    qmm.prologue(ex2.interp, args)
    assert qmm.stats()["packs"] == 1 and qmm.stats()["build_hits"] == 1
    qmm.prologue(ex3.interp, args)
    assert qmm.stats()["packs"] == 2 and qmm.stats()["build_hits"] == 1


def test_a_big_constant_declines_the_build_cache(monkeypatch):
    """A decode table too big to serialize: no cache entry, no wrong reuse,
    the chain is simply built for every executable (reference
    tests/test_qmm_mxfp4.py:858-876; here the E2M1 table is put over the limit)."""
    monkeypatch.setattr(packs, "FP_DENSE_ELEMS", 8)
    n, k = 64, 128
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=78)
    args = [I.from_numpy(blocks), I.from_numpy(sb)]
    for t in (2, 5):
        ex = engine.compile_program(T.dense_mxfp4(n, k, t))
        qmm.prologue(ex.interp, args + [I.from_numpy(np.zeros((t, k), np.float32), "bf16")])
        np.testing.assert_array_equal(np.asarray(ex.interp._qmm.matches[0].packs[0].w), O.pack_codes(codes, 4))
    st = qmm.stats()
    assert st["build_declines"] == 2 and st["build_hits"] == 0 and st["packs"] == 2


def test_identical_mxfp4_weights_in_two_buffers_share_one_pack():
    """Content-addressed sharing: the same bytes arriving in other buffers are
    packed again (identity misses) but end up aliasing the first pack's arrays;
    different bytes do not (reference tests/test_qmm_mxfp4.py:423-480)."""
    n, k, t = 64, 128, 2
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=8)
    _, blocks2, sb2, _ = T.random_mxfp4((n, k), seed=9)
    x = I.from_numpy(np.zeros((t, k), np.float32), "bf16")
    text = T.dense_mxfp4(n, k, t)
    exs = [engine.compile_program(text) for _ in range(3)]
    qmm.prologue(exs[0].interp, [I.from_numpy(blocks), I.from_numpy(sb), x])
    qmm.prologue(exs[1].interp, [I.from_numpy(blocks.copy()), I.from_numpy(sb.copy()), x])
    qmm.prologue(exs[2].interp, [I.from_numpy(blocks2), I.from_numpy(sb2), x])
    assert qmm.stats()["packs"] == 3 and qmm.stats()["shared"] == 1
    p0, p1, p2 = (e.interp._qmm.matches[0].packs[0] for e in exs)
    assert p1.w is p0.w and p1.scales is p0.scales and p2.w is not p0.w


# --------------------------------------------------- decode loop, run path ---

def test_decode_loop_weights_are_hoisted_out_of_the_carry():
    k, m, steps = 128, 2, 3
    q, packed, scale, zero, g_idx, wref = T.quantize(k, k, 64, seed=10)
    ex = engine.compile_program(T.decode_loop(k, 2, m, steps))
    st = qmm.analyze(ex.interp)
    assert len(st.matches) == 1 and st.matches[0].arg_indices == (0, 1, 2, 3)
    x = T.bf16_round(np.random.default_rng(1).standard_normal((m, k)).astype(np.float32))
    args = host_args_dense(packed, scale * 0.2, zero, g_idx, x)
    args[1] = I.from_numpy(T.bf16_round(scale * 0.2), "bf16")
    qmm.prologue(ex.interp, args)
    qmm.prologue(ex.interp, args)
    assert qmm.stats()["packs"] == 1 and qmm.stats()["fallbacks"] == 0


def test_interleaved_groups_in_a_decode_loop(monkeypatch):
    """The permutation of K travels into the loop with the other packed values:
    packed once, applied to the activations in every step, and the loop's
    result follows the literal chain (reference tests/test_qmm.py:429-469)."""
    k, m, steps, ng = 128, 2, 3, 2
    g_idx = (np.arange(k) % ng).astype(np.float32)
    q, packed, scale, zero, g_idx, wref = T.quantize(k, k, k // ng, seed=21, g_idx=g_idx)
    x = T.bf16_round(np.random.default_rng(2).standard_normal((m, k)).astype(np.float32))
    args = host_args_dense(packed, scale * 0.2, zero, g_idx, x)
    args[1] = I.from_numpy(T.bf16_round(scale * 0.2), "bf16")
    st, fused, literal = _fused_and_literal(monkeypatch, T.decode_loop(k, ng, m, steps), args)
    assert qmm.stats()["packs"] == 1 and qmm.stats()["perms"] == 1 and qmm.stats()["fallbacks"] == 0
    assert st.matches[0].has_perm and st.matches[0].nvals == 4
    w = T.bf16_round(scale * 0.2)[g_idx.astype(np.int32)] * (q.astype(np.float32) - zero[g_idx.astype(np.int32)])
    exact = x
    for _ in range(steps):
        exact = T.bf16_round(exact @ w)
    np.testing.assert_allclose(fused, literal, rtol=3e-2, atol=3e-2 * np.abs(exact).max())
    np.testing.assert_allclose(fused, exact, rtol=3e-2, atol=3e-2 * np.abs(exact).max())


def test_rewritten_program_runs_the_root_and_never_the_absorbed_ops(monkeypatch):
    k, n, m = 256, 128, 4
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, 64, seed=12)
    x = T.bf16_round(np.random.default_rng(3).standard_normal((m, k)).astype(np.float32) * 0.5)
    text = T.dense_sub(k, n, k // 64, m)
    args = host_args_dense(packed, scale, zero, g_idx, x)
    literal = I.host(I.Interpreter(text).run(args)[0]).a
    exact = x @ wref
    assert np.abs(literal - exact).max() / np.abs(exact).max() < 2e-2

    ran = []
    for name in ("stablehlo.gather", "stablehlo.multiply", "stablehlo.dot_general", "stablehlo.xor"):
        orig = I.REGISTRY[name]
        monkeypatch.setitem(I.REGISTRY, name,
                            lambda interp, op, ins, env, _o=orig, _n=name: (ran.append(_n), _o(interp, op, ins, env))[1])
    monkeypatch.setattr(qmm, "emit", oracle_emit)
    ex = engine.compile_program(text)
    qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, args)
    ran.clear()                                            # the pack itself replays the chain once
    (y,) = ex.interp.run(args)
    assert ran == []                                       # chain absorbed, dot replaced
    fused = I.host(y).a
    assert np.abs(fused - exact).max() <= 1.5 * np.abs(literal - exact).max() + 1e-6
    np.testing.assert_allclose(fused, literal, rtol=2e-2, atol=1e-2 * np.abs(exact).max())


def test_values_travel_as_explicit_inputs():
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=8)
    ex = engine.compile_program(T.dense_sub(k, n, 2, m))
    qmm.prologue(ex.interp, host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32)))
    vals = qmm.values(ex.interp)
    mt = ex.interp._qmm.matches[0]
    assert len(vals) == 3 and (mt.slot, mt.nvals) == (0, 3)
    assert qmm.pack_arrays(ex.interp, mt) == vals[0:3]
    tok = qmm.push(ex.interp, ["w", "s", "b"])
    assert qmm.pack_arrays(ex.interp, mt) == ["w", "s", "b"]
    qmm.pop(ex.interp, tok)
    assert qmm.values(ex.interp) is vals


def test_emit_fails_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=8)
    ex = engine.compile_program(T.dense_sub(k, n, 2, m))
    args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32))
    with pytest.raises(Exception) as e:
        engine.execute(ex, args)
    assert not isinstance(e.value, I.UnsupportedOp)


def test_a_device_failure_while_packing_is_not_a_fallback(monkeypatch):
    """A weight that does not verify disables its match (the program runs
    literally, reference qmm.py:2348-2355); the device failing while a pack is
    built is not that: a HIP error from the library, or a torch accelerator
    error, reaches the caller instead of being hidden behind the literal chain."""
    from metaljax_amd import _lib, packs
    k, n, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(k, n, 64, seed=8)
    args = host_args_dense(packed, scale, zero, g_idx, np.zeros((m, k), np.float32))

    def boom(err):
        def pack_for(*a, **kw):
            raise err
        return pack_for
    for err in (_lib.QmmError(5, "hipErrorIllegalAddress"), RuntimeError("HIP error: an illegal memory access")):
        ex = engine.compile_program(T.dense_sub(k, n, 2, m))
        monkeypatch.setattr(packs, "pack_for", boom(err))
        with pytest.raises(type(err)):
            qmm.prologue(ex.interp, args)
        assert not ex.interp._qmm.matches[0].disabled
    # an ordinary failure still falls back
    ex = engine.compile_program(T.dense_sub(k, n, 2, m))
    monkeypatch.setattr(packs, "pack_for", boom(ValueError("does not verify")))
    assert qmm.prologue(ex.interp, args) is True and ex.interp._qmm.matches[0].disabled


# ------------------------------------------------------- engine surface ----

def test_engine_surface_is_what_the_pjrt_plugin_calls_by_name():
    """Names, argument meaning and result types as the reference's plugin uses
    them: compile_program(code, fmt, options) -> object whose name /
    fingerprint are str, num_outputs / num_params ints, out_types a list of
    PJRT_Buffer_Type integers, out_dims a list of int lists, donated_params a
    list of ints (plugin/metal_pjrt.cc:547-580); execute(exec, [buffer]) -> a
    list of num_outputs objects with data, type_enum, dims, nbytes (:284-299,
    :990-1010); buffer_from_host(memoryview, type_enum, dims, byte_strides,
    offset) (:662-664); buffer_pointer(buffer) -> int (:1125); to_host(buffer)
    -> bytes of nbytes length (:1168-1172); device_kind() -> str,
    stablehlo_version() -> ints (:382, :440)."""
    import numpy as np
    from metaljax_amd import engine
    text = T.float_dot(8, 16, 4, el="f32")          # y = x @ (w * r[:, None]): w [8,16], r [8], x [4,8]
    ex = engine.compile_program(text.encode(), "mlir", None)
    assert isinstance(ex.name, str) and ex.name == "main"
    assert isinstance(ex.fingerprint, str) and len(ex.fingerprint) == 64
    assert (ex.num_params, ex.num_outputs) == (3, 1)
    f32 = engine.PJRT_TYPES.index("F32")
    assert f32 == 11 and engine.PJRT_TYPES.index("BF16") == 13       # PJRT_Buffer_Type values of the C API
    assert ex.out_types == [f32] and all(type(t) is int for t in ex.out_types)
    assert ex.out_dims == [[4, 16]] and ex.donated_params == []
    rng = np.random.default_rng(0)
    w = rng.standard_normal((8, 16)).astype(np.float32)
    r = rng.standard_normal((8,)).astype(np.float32)
    x = rng.standard_normal((4, 8)).astype(np.float32)
    # a transposed host view arrives with strides
    wt = np.ascontiguousarray(w.T)
    bw = engine.buffer_from_host(memoryview(wt), f32, [8, 16], [4, 4 * 8], 0)
    br = engine.buffer_from_host(memoryview(r), f32, [8], None, 0)
    bx = engine.buffer_from_host(memoryview(x), f32, [4, 8], None, 0)
    assert bx.nbytes == x.nbytes and bx.dims == [4, 8] and bx.type_enum == f32
    ptr = engine.buffer_pointer(bx)
    assert type(ptr) is int and ptr != 0
    outs = engine.execute(ex, [bw, br, bx])
    assert isinstance(outs, list) and len(outs) == ex.num_outputs
    y = outs[0]
    assert y.type_enum == f32 and y.dims == [4, 16] and y.nbytes == 4 * 16 * 4
    assert hasattr(y, "data")
    raw = engine.to_host(y)
    assert type(raw) is bytes and len(raw) == y.nbytes
    got = np.frombuffer(raw, np.float32).reshape(4, 16)
    np.testing.assert_allclose(got, x @ (w * r[:, None]), rtol=1e-5, atol=1e-5)
    # an output buffer is a valid input of the next execute
    (y2,) = engine.execute(ex, [bw, br, bx])
    assert engine.to_host(y2) == raw
    # bf16 bytes round-trip as 16-bit patterns
    bits = np.array([0x3F80, 0xC000, 0x0000], np.uint16)
    bf = engine.buffer_from_host(memoryview(bits), engine.PJRT_TYPES.index("BF16"), [3], None, 0)
    assert bf.nbytes == 6 and engine.to_host(bf) == bits.tobytes()
    with pytest.raises(TypeError, match="Unsupported"):      # "Unsupported" in the class or text -> UNIMPLEMENTED (:185-226)
        engine.buffer_from_host(None, engine.PJRT_TYPES.index("C64"), [1], None, 0)
    assert isinstance(engine.device_kind(), str)
    ver = engine.stablehlo_version()
    assert len(ver) == 3 and all(type(v) is int for v in ver)


# --------------------------------------------------- packing by row blocks ----

def _packs_built(monkeypatch, text, args, block_elems):
    """Pack `text`'s weights on fresh copies of `args` with a given block size;
    returns (pack arrays, stats).  Both pack tables are cleared first: two
    builds of one weight are identical and would otherwise alias each other,
    and comparing an array with itself proves nothing."""
    qmm._SHARED.clear()
    qmm._BUILT.clear()
    qmm.reset_stats()
    monkeypatch.setattr(packs, "BLOCK_ELEMS", block_elems)
    ex = engine.compile_program(text)
    fresh = [I.HostArray(np.array(a.a, copy=True), a.el) for a in args]
    qmm.prologue(ex.interp, fresh)
    st = ex.interp._qmm
    built = [[np.array(np.asarray(a.bits if isinstance(a, packing.BF16Array) else a)) for a in pk.arrays()]
             for mt in st.matches for pk in mt.packs[:1]]
    return built, qmm.stats(), st


def _same_packs(a, b):
    assert len(a) == len(b)
    for pa, pb in zip(a, b):
        assert len(pa) == len(pb)
        for x, y in zip(pa, pb):
            assert x.dtype == y.dtype and x.shape == y.shape
            np.testing.assert_array_equal(x, y)


def test_blocked_affine_pack_is_bit_identical(monkeypatch):
    """Packing an affine weight by blocks of rows gives the bits a whole
    evaluation gives: codes, scale and bias tables (reference
    tests/test_qmm.py:1029-1057).  The codes are walked twice when blocked
    (the offset is one number for the whole weight)."""
    n, k, gs, t = 256, 128, 64, 3
    q, scale, zero, ref = T.affine_grouped_data(n, k, gs, 21)
    x = T.bf16_round(np.random.default_rng(22).standard_normal((t, k)).astype(np.float32) * 0.3)
    args = [I.from_numpy(q), I.from_numpy(scale), I.from_numpy(zero), I.from_numpy(x, "bf16")]
    text = T.affine_grouped(n, k, gs, t)
    whole, st_w, _ = _packs_built(monkeypatch, text, args, 1 << 40)
    small, st_b, state = _packs_built(monkeypatch, text, args, 1 << 10)     # 8 rows a block
    assert st_w["packs"] == st_b["packs"] == 1 and st_w["fallbacks"] == st_b["fallbacks"] == 0
    assert st_w["blocked"] == 0 and st_b["blocked"] == 1
    assert state.matches[0].packs[0].blocked
    _same_packs(whole, small)
    pk = state.matches[0].packs[0]
    assert (pk.gs, pk.bits, pk.perm) == (gs, 4, None)
    # the packed weight is the graph's weight: scale * (q - zero) with bf16 scales
    want = T.bf16_round(scale)[:, np.arange(k) // gs] * (q.astype(np.float32) - zero[:, np.arange(k) // gs])
    np.testing.assert_allclose(dequant_pack(pk), want, rtol=1e-6, atol=1e-7)


def _three_grouped_weights(n, k, gs, t):
    """y = x.W1^T + x.W2^T + x.W3^T, each weight as in T.affine_grouped."""
    ng = k // gs
    t3, q3, tab = f"tensor<{n}x{ng}x{gs}xbf16>", f"tensor<{n}x{ng}x{gs}xi8>", f"tensor<{n}x{ng}xbf16>"
    nk, tn, tk = f"tensor<{n}x{k}xbf16>", f"tensor<{t}x{n}xbf16>", f"tensor<{t}x{k}xbf16>"
    params, body = [], []
    for i in (1, 2, 3):
        params += [f"%q{i}: tensor<{n}x{k}xi8>", f"%scale{i}: tensor<{n}x{ng}xf32>", f"%zero{i}: tensor<{n}x{ng}xi8>"]
        body.append(f"""
    %qs{i} = stablehlo.reshape %q{i} : (tensor<{n}x{k}xi8>) -> {q3}
    %qf{i} = stablehlo.convert %qs{i} : ({q3}) -> {t3}
    %sc{i} = stablehlo.convert %scale{i} : (tensor<{n}x{ng}xf32>) -> {tab}
    %sb{i} = stablehlo.broadcast_in_dim %sc{i}, dims = [0, 1] : ({tab}) -> {t3}
    %zc{i} = stablehlo.convert %zero{i} : (tensor<{n}x{ng}xi8>) -> {tab}
    %zb{i} = stablehlo.broadcast_in_dim %zc{i}, dims = [0, 1] : ({tab}) -> {t3}
    %d{i} = stablehlo.subtract %qf{i}, %zb{i} : {t3}
    %w3{i} = stablehlo.multiply %d{i}, %sb{i} : {t3}
    %w{i} = stablehlo.reshape %w3{i} : ({t3}) -> {nk}
    %y{i} = stablehlo.dot_general %x, %w{i}, contracting_dims = [1] x [1] : ({tk}, {nk}) -> {tn}""")
    return f"""
module @jit_three {{
  func.func public @main({", ".join(params)}, %x: {tk}) -> {tn} {{{"".join(body)}
    %s = stablehlo.add %y1, %y2 : {tn}
    %out = stablehlo.add %s, %y3 : {tn}
    return %out : {tn}
  }}
}}
"""


def test_pack_builds_reclaim_what_they_leave_behind(monkeypatch):
    """A build that evaluated its weight whole reclaims at once, row-blocked
    builds every METALJAX_QMM_GC_EVERY of them, a prologue that built anything
    once more at its end, one that built nothing not at all (reference
    qmm.py:165, :2326-2347, :2382-2386)."""
    n, k, gs, t = 256, 128, 64, 3
    text = _three_grouped_weights(n, k, gs, t)
    data = [T.affine_grouped_data(n, k, gs, seed)[:3] for seed in (31, 32, 33)]
    x = T.bf16_round(np.random.default_rng(34).standard_normal((t, k)).astype(np.float32) * 0.3)

    def reclaims(block_elems, every):
        qmm._BUILT.clear()
        qmm.reset_stats()
        monkeypatch.setattr(packs, "BLOCK_ELEMS", block_elems)
        monkeypatch.setattr(qmm, "GC_EVERY", every)
        ex = engine.compile_program(text)
        args = [I.from_numpy(a.copy()) for three in data for a in three] + [I.from_numpy(x, "bf16")]
        before = qmm.RECLAIMS[0]
        qmm.prologue(ex.interp, args)
        first = qmm.RECLAIMS[0] - before
        qmm.prologue(ex.interp, args)                       # the same buffers: nothing built
        blocked = [m.packs[0].blocked for m in ex.interp._qmm.matches]
        assert qmm.stats()["packs"] == 3 and qmm.stats()["fallbacks"] == 0
        assert qmm.RECLAIMS[0] - before == first
        return first, blocked

    assert reclaims(1 << 40, 8) == (4, [False] * 3)         # after each whole build, and at the end
    assert reclaims(1 << 10, 8) == (1, [True] * 3)          # blocked builds wait for the end ...
    assert reclaims(1 << 10, 1) == (4, [True] * 3)          # ... or for every one of them,
    assert reclaims(1 << 10, 2) == (2, [True] * 3)          # or for every second


def test_blocked_affine_falls_back_when_groups_interleave(monkeypatch):
    """Groups scattered along K: the permutation that gathers them is a
    property of the whole contraction axis, so the blocked pass gives up and
    the weight packs from a whole evaluation -- the same pack the unblocked
    path builds (reference tests/test_qmm.py:1060-1090)."""
    n, k, gs, t = 128, 128, 64, 2
    q, scale, zero, ref = T.affine_grouped_data(n, k, gs, 23, interleave=True)
    x = T.bf16_round(np.random.default_rng(24).standard_normal((t, k)).astype(np.float32) * 0.3)
    args = [I.from_numpy(q), I.from_numpy(scale), I.from_numpy(zero), I.from_numpy(x, "bf16")]
    text = T.affine_grouped(n, k, gs, t, interleave=True)
    whole, st_w, _ = _packs_built(monkeypatch, text, args, 1 << 40)
    small, st_b, state = _packs_built(monkeypatch, text, args, 1 << 10)
    assert st_b["packs"] == 1 and st_b["blocked"] == 0 and st_b["perms"] == 1 and st_b["fallbacks"] == 0
    assert st_w["perms"] == 1
    _same_packs(whole, small)
    assert state.matches[0].has_perm


def test_blocked_mxfp4_pack_is_bit_identical_through_a_take_callee(monkeypatch):
    """The E2M1 decode as jax lowers it -- a private @_take callee whose body
    is declared for the full extent -- evaluated inside the callee, block by
    block (reference tests/test_qmm_mxfp4.py:895-928)."""
    n, k, t = 96, 128, 4
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=5)
    x = T.bf16_round(np.random.default_rng(6).standard_normal((t, k)).astype(np.float32))
    text = T.dense_mxfp4_rows(n, k, t)
    assert "@_take" in text
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")]
    whole, st_w, _ = _packs_built(monkeypatch, text, args, 1 << 40)
    small, st_b, state = _packs_built(monkeypatch, text, args, 1 << 11)     # 16 rows a block
    assert st_w["blocked"] == 0 and st_b["blocked"] == 1 and st_b["mxfp4"] == 1
    _same_packs(whole, small)
    pk = state.matches[0].packs[0]
    np.testing.assert_array_equal(np.asarray(pk.w), O.pack_codes(codes, 4))
    np.testing.assert_array_equal(np.asarray(pk.scales), sb)
    # the literal run of the same module agrees with the exact weight
    lit = I.host(I.Interpreter(text).run(args)[0]).a
    np.testing.assert_allclose(lit, T.bf16_round(x @ w.T), rtol=2e-2, atol=1e-2 * np.abs(x @ w.T).max())


def test_blocked_pack_bounds_the_transient(monkeypatch):
    """The point of blocking: the pack costs a block, not a weight.  The MXFP4
    chain is several times wider than the weight it reconstructs (index
    tensors, gathered values, broadcast scales), so the peak of live host
    memory during a whole evaluation is many times the packed result; by
    blocks it must be well under half of that (reference
    tests/test_qmm_mxfp4.py:745-777)."""
    import tracemalloc
    e, n, k, t = 4, 512, 512, 2
    codes, blocks, sb, _ = T.random_mxfp4((e, n, k), seed=12)
    x = np.zeros((e, t, k), np.float32)
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")]
    text = T.dense_mxfp4_rows(n, k, t, e=e)                 # every op keeps the expert axis leading: one expert a block

    def peak(block_elems):
        tracemalloc.start()
        try:
            built, st, _ = _packs_built(monkeypatch, text, args, block_elems)
            return built, st, tracemalloc.get_traced_memory()[1]
        finally:
            tracemalloc.stop()
    whole, st_w, peak_whole = peak(1 << 40)
    small, st_b, peak_blocked = peak(1 << 14)
    assert st_w["blocked"] == 0 and st_b["blocked"] == 1
    _same_packs(whole, small)
    assert peak_blocked < peak_whole / 2, (peak_blocked, peak_whole)


def test_blocked_pack_reads_a_decode_table_whole(monkeypatch):
    """Sixteen experts and a sixteen-entry E2M1 table: whether a value is cut
    into blocks is decided by the demand coming down from the weight, not by
    its shape -- the gather's indices are blocked, the table it gathers
    through is read whole (reference tests/test_qmm_mxfp4.py:782-806)."""
    e, n, k, t = 16, 64, 128, 2
    codes, blocks, sb, w = T.random_mxfp4((e, n, k), seed=13)
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(np.zeros((e, t, k), np.float32), "bf16")]
    text = T.dense_mxfp4_rows(n, k, t, e=e)
    whole, st_w, _ = _packs_built(monkeypatch, text, args, 1 << 40)
    small, st_b, state = _packs_built(monkeypatch, text, args, 1 << 10)
    assert st_b["blocked"] == 1 and st_b["fallbacks"] == 0
    _same_packs(whole, small)
    pk = state.matches[0].packs[0]
    np.testing.assert_array_equal(np.asarray(pk.w), O.pack_codes(codes, 4))
    np.testing.assert_array_equal(dequant_pack(pk), w)


def test_a_chain_that_is_not_row_local_packs_whole(monkeypatch):
    """A reshape that folds N into other axes (the decode over a flat index
    list) is not row-local: blocks are refused and the pack is the whole
    evaluation's.  A weight stored K-first cannot be blocked by rows at all."""
    n, k, t = 48, 128, 5
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=1)
    x = T.bf16_round(np.random.default_rng(2).standard_normal((t, k)).astype(np.float32))
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")]
    whole, _, _ = _packs_built(monkeypatch, T.dense_mxfp4(n, k, t), args, 1 << 40)
    small, st_b, _ = _packs_built(monkeypatch, T.dense_mxfp4(n, k, t), args, 1 << 9)
    assert st_b["packs"] == 1 and st_b["blocked"] == 0 and st_b["fallbacks"] == 0
    _same_packs(whole, small)
    kk, nn, m = 128, 64, 2
    q, packed, scale, zero, g_idx, _ = T.quantize(kk, nn, 64)
    ex = engine.compile_program(T.dense_sub(kk, nn, 2, m))
    st = qmm.analyze(ex.interp)
    monkeypatch.setattr(packs, "BLOCK_ELEMS", 1 << 8)
    src = packs.WeightRows(ex.interp, st.matches[0], host_args_dense(packed, scale, zero, g_idx, np.zeros((m, kk), np.float32)))
    assert not src.blocked() and src.blocks() == [(0, kk)]


def test_block_size_comes_from_the_environment():
    import os
    import subprocess
    import sys
    ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    code = "from metaljax_amd import packs; print(packs.BLOCK_ELEMS)"
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True,
                         env={**os.environ, "METALJAX_QMM_BLOCK": "4096"}, cwd=ROOT)
    assert out.stdout.strip() == "4096", out.stderr


# ------------------------------------------------------- expert dispatch ----

def _moe_inputs(E, T, H, Ii, seed=None):
    rng = np.random.default_rng(E if seed is None else seed)
    gu_c, gu_s, gu_ref = T_.make_mxfp4_experts(2 * Ii, H, E, seed=E)
    d_c, d_s, d_ref = T_.make_mxfp4_experts(H, Ii, E, seed=E + 1)
    x = (rng.standard_normal((T, H)) / 8).astype(np.float32)
    wr = (rng.standard_normal((H, E)) / 8).astype(np.float32)
    br = rng.standard_normal(E).astype(np.float32)
    bgu = (rng.standard_normal((E, 2 * Ii)) / 8).astype(np.float32)
    bd = (rng.standard_normal((E, H)) / 8).astype(np.float32)
    return (x, wr, br, gu_c, gu_s, d_c, d_s, bgu, bd), (gu_ref, d_ref)


T_ = T


@pytest.mark.parametrize("composite", [False, True])
def test_dense_moe_block_is_planned_over_pairs(composite):
    """The gpt-oss block (reference tests/test_moe.py:500-557): one dispatch,
    both expert projections read quantized packs, the router is proven and
    checked on synthetic logits, and the dense [tokens, experts] scores and
    their one-hot are no longer computed."""
    from metaljax_amd import moe
    moe.reset_stats()
    E, Tk, H, Ii, K = 4, 3, 64, 32, 2
    ex = engine.compile_program(T.moe_block_mxfp4(E, Tk, H, Ii, K, composite=composite))
    st = qmm.analyze(ex.interp)
    assert [m.mode for m in st.matches] == ["mxfp4", "mxfp4"] and all(m.absorbed for m in st.matches)
    assert len(st.moe) == 1 and moe.stats()["recognized"] == 1
    g = st.moe[0]
    assert (g.E, g.T, g.K, g.P, g.out_shape) == (E, Tk, K, Tk * K, [Tk, H])
    assert g.matches == st.matches and g.plan.dots == 2
    r = g.router
    assert r.indices.type.shape == (Tk, K) and r.weights.type.shape == (Tk, K) and moe.is_top_k(r.top_k)
    # the rewrite: the root is the dispatch, the dots and the router's dense tail are skipped
    assert st.roots == {g.key: g}
    names = {k.op.name for k in g.skip_keys}
    assert {"stablehlo.dot_general", "stablehlo.compare", "stablehlo.iota", "stablehlo.logistic"} <= names
    by_name = {v.name: v for b in ir.walk_blocks(ex.interp.main.body) for o in b.ops for v in o.results}
    assert by_name["s"] in g.skip_keys and by_name["hw"] in g.skip_keys          # scores and one-hot product
    assert by_name["w"] not in g.skip_keys and by_name["logits"] not in g.skip_keys
    assert set(qmm.emit_reads(g)) >= {r.indices, r.weights, by_name["bd"] if "bd" in by_name else r.weights}
    args, _ = _moe_inputs(E, Tk, H, Ii)
    changed = qmm.prologue(ex.interp, [I.from_numpy(a) for a in args])
    assert changed is False and moe.stats()["verified"] == 1 and moe.stats()["fallbacks"] == 0
    assert qmm.stats()["mxfp4"] == 2 and qmm.stats()["packs"] == 2


def _oracle_expert_product(calls):
    """A stand-in for moe.emit_dot on host tensors: the per-pair products by the
    oracle (the kernel's place in a dispatch that runs on torch CPU tensors)."""
    import torch
    from oracle import qmm_oracle as O

    def product(x, arrays, mode, gs, bits, tidx, eidx, experts, out_dtype=None, has_perm=False):
        from metaljax_amd import moe
        assert not has_perm and isinstance(x, torch.Tensor) and x.device.type == "cpu" and x.is_contiguous()
        biases = arrays[2] if mode == "affine" else None
        w, scales = moe.split_experts([np.asarray(arrays[0]), np.asarray(arrays[1])], experts)
        pairs = int(eidx.numel())
        lhs = np.arange(pairs) if tidx is None else tidx.numpy()
        assert x.shape[0] == (pairs if tidx is None else x.shape[0])
        y = O.gather_qmm(x.float().numpy(), w, scales, biases, lhs, eidx.numpy(), gs, bits, mode)
        calls.append((tuple(x.shape), tidx is None))
        return torch.from_numpy(y).to(out_dtype or torch.float32)
    return product


@_without_a_gpu
@pytest.mark.parametrize("composite", [False, True])
def test_the_dispatchs_tensor_program_gives_the_dense_blocks_result(composite, monkeypatch):
    """Everything a planned dispatch does around its two expert products --
    gathers on the way in, the bias adds, the gated activation's slices,
    clamps and products, the hand-over from the first product to the second,
    the routing-weighted sum -- on torch CPU tensors, the products themselves
    by the oracle: equal to the dense block run literally and to its numpy
    restatement (reference tests/test_moe.py:500-557 checks the same block
    end to end)."""
    from metaljax_amd import moe
    moe.reset_stats()
    calls = []
    monkeypatch.setattr(qmm, "DEVICE", "cpu")
    monkeypatch.setattr(moe, "emit_dot", _oracle_expert_product(calls))
    E, Tk, H, Ii, K = 4, 5, 64, 32, 2
    text = T.moe_block_mxfp4(E, Tk, H, Ii, K, composite=composite)
    raw, (gu_ref, d_ref) = _moe_inputs(E, Tk, H, Ii)
    args = [I.from_numpy(a) for a in raw]
    ex = engine.compile_program(text)
    (buf,) = engine.execute(ex, args)
    st = moe.stats()
    assert st["recognized"] == 1 and st["dispatches"] == 1 and st["fallbacks"] == 0, st
    # the first product reads the tokens' rows through the pairs' token numbers, the second one pair rows
    assert calls == [((Tk, 1, H), False), ((Tk * K, 1, Ii), True)]
    got = I.host(buf.data).a
    x, wr, br, _, _, _, _, bgu, bd = raw
    want = T.moe_block_reference(x, wr, br, gu_ref, d_ref, bgu, bd, K)
    np.testing.assert_allclose(got, want, rtol=3e-5, atol=3e-6 * max(1.0, np.abs(want).max()))
    qmm_was = qmm.ENABLED
    monkeypatch.setattr(qmm, "ENABLED", False)
    (lit,) = engine.execute(engine.compile_program(text), args)
    monkeypatch.setattr(qmm, "ENABLED", qmm_was)
    np.testing.assert_allclose(got, I.host(lit.data).a, rtol=3e-5, atol=3e-6 * max(1.0, np.abs(want).max()))


@_without_a_gpu
def test_the_dispatchs_tensor_program_in_bf16(monkeypatch):
    """The same block with bf16 activations: every op between the products
    rounds to bf16 as the literal path does (widened, computed in float32,
    rounded once), so the two agree to the last bf16 place or two of the
    result's scale (the expert products sum in another order)."""
    from metaljax_amd import moe
    moe.reset_stats()
    monkeypatch.setattr(qmm, "DEVICE", "cpu")
    monkeypatch.setattr(moe, "emit_dot", _oracle_expert_product([]))
    E, Tk, H, Ii, K = 4, 5, 64, 32, 2
    text = T.moe_block_mxfp4(E, Tk, H, Ii, K, el="bf16")
    raw, _ = _moe_inputs(E, Tk, H, Ii)
    args = [I.from_numpy(a, "bf16") if a.dtype == np.float32 else I.from_numpy(a) for a in raw]
    (buf,) = engine.execute(engine.compile_program(text), args)
    assert moe.stats()["dispatches"] == 1 and moe.stats()["fallbacks"] == 0
    got = I.host(buf.data)
    assert got.el == "bf16"
    monkeypatch.setattr(qmm, "ENABLED", False)
    (lit,) = engine.execute(engine.compile_program(text), args)
    lit = I.host(lit.data).a
    assert np.abs(got.a - lit).max() <= 2.0 ** -6 * np.abs(lit).max()


@_without_a_gpu
@pytest.mark.parametrize("Tk", [1, 6])
@pytest.mark.parametrize("E,K", [(4, 2), (8, 4)])
def test_gemma4_block_is_gathered_also_at_one_token(E, K, Tk, monkeypatch):
    """keras-hub's Gemma4 block (reference tests/test_moe.py:192-262) with
    MXFP4 experts: a softmax -> top-k -> renormalise router, three expert
    products, and a per-expert output scale [E] -> [E, 1, 1] broadcast over
    [E, T, H].  At T = 1 (every decode step) that broadcast's token axis is a
    unit axis on both sides and must be read as a broadcast, not as the token
    axis.  The dispatch's tensor program runs on torch CPU tensors, the three
    products by the oracle."""
    from metaljax_amd import moe
    moe.reset_stats()
    calls = []
    monkeypatch.setattr(qmm, "DEVICE", "cpu")
    monkeypatch.setattr(moe, "emit_dot", _oracle_expert_product(calls))
    H, Ii = 64, 32
    rng = np.random.default_rng(Tk * 100 + E)
    g_c, g_s, g_ref = T.make_mxfp4_experts(Ii, H, E, seed=E)
    u_c, u_s, u_ref = T.make_mxfp4_experts(Ii, H, E, seed=E + 1)
    d_c, d_s, d_ref = T.make_mxfp4_experts(H, Ii, E, seed=E + 2)
    x = (rng.standard_normal((Tk, H)) / 8).astype(np.float32)
    proj = rng.standard_normal((H, E)).astype(np.float32)
    per_dim = (1.0 + rng.standard_normal(H) / 8).astype(np.float32)
    escale = (1.0 + rng.standard_normal(E) / 8).astype(np.float32)
    text = T.moe_block_gemma4_mxfp4(E, Tk, H, Ii, K)
    args = [I.from_numpy(a) for a in (x, proj, per_dim, g_c, g_s, u_c, u_s, d_c, d_s, escale)]
    ex = engine.compile_program(text)
    (buf,) = engine.execute(ex, args)
    st = moe.stats()
    assert st["recognized"] == 1 and st["verified"] == 1 and st["dispatches"] == 1 and st["fallbacks"] == 0, st
    assert qmm.stats()["mxfp4"] == 3 and all(m.absorbed for m in ex.interp._qmm.matches)
    # gate and up read the tokens' rows through the pairs' token numbers, down reads pair rows
    assert sorted(calls) == sorted([((Tk, 1, H), False)] * 2 + [((Tk * K, 1, Ii), True)])
    got = I.host(buf.data).a
    assert got.shape == (Tk, H)
    want = T.gemma4_block_reference(x, proj, per_dim, g_ref, u_ref, d_ref, escale, K)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5 * max(1.0, np.abs(want).max()))
    monkeypatch.setattr(qmm, "ENABLED", False)
    (lit,) = engine.execute(engine.compile_program(text), args)
    np.testing.assert_allclose(got, I.host(lit.data).a, rtol=1e-4, atol=1e-5 * max(1.0, np.abs(want).max()))


@_without_a_gpu
@pytest.mark.parametrize("el", ["f32", "bf16"])
def test_gemma4_prefill_and_a_decode_step_inside_a_while_body_are_both_gathered(el, monkeypatch):
    """What a sampler emits (reference tests/test_moe.py:262-296): the block
    over [T, H], then a loop whose body is the block over the [1, H] row of
    the step before; the loop's weights are carries returned unchanged.  Both
    dispatches are planned, verified and run; the six recognized weights are
    three buffers, so three packs are built and the loop body's matches reuse
    them."""
    from metaljax_amd import moe
    moe.reset_stats()
    calls = []
    monkeypatch.setattr(qmm, "DEVICE", "cpu")
    monkeypatch.setattr(moe, "emit_dot", _oracle_expert_product(calls))
    E, Tk, H, Ii, K, steps = 8, 5, 64, 32, 2, 3
    rng = np.random.default_rng(57)
    g_c, g_s, _ = T.make_mxfp4_experts(Ii, H, E, seed=58)
    u_c, u_s, _ = T.make_mxfp4_experts(Ii, H, E, seed=59)
    d_c, d_s, _ = T.make_mxfp4_experts(H, Ii, E, seed=60)
    x = (rng.standard_normal((Tk, H)) / 8).astype(np.float32)
    proj = rng.standard_normal((H, E)).astype(np.float32)
    per_dim = (1.0 + rng.standard_normal(H) / 8).astype(np.float32)
    escale = (1.0 + rng.standard_normal(E) / 8).astype(np.float32)
    text = T.moe_gemma4_decode_loop(E, Tk, H, Ii, K, steps, el=el)
    args = [I.from_numpy(a, el) if a.dtype == np.float32 else I.from_numpy(a)
            for a in (x, proj, per_dim, g_c, g_s, u_c, u_s, d_c, d_s, escale)]
    ex = engine.compile_program(text)
    pre, tok = engine.execute(ex, args)
    st, qst = moe.stats(), qmm.stats()
    assert st["recognized"] == 2 and st["verified"] == 2 and st["fallbacks"] == 0, st
    assert st["dispatches"] == 1 + steps and len(calls) == 3 * (1 + steps)
    assert qst["recognized"] == 6 and qst["fallbacks"] == 0 and qst["packs"] + qst["build_hits"] + qst["shared"] >= 3, qst
    assert qst["packs"] - qst["shared"] == 3, qst            # three weights' worth of packed arrays, whoever built them
    monkeypatch.setattr(qmm, "ENABLED", False)
    lit_pre, lit_tok = engine.execute(engine.compile_program(text), args)
    tol = 4e-2 if el == "bf16" else 1e-4
    for got, want in ((pre, lit_pre), (tok, lit_tok)):
        got, want = I.host(got.data).a, I.host(want.data).a
        assert got.shape == want.shape
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol * max(1e-2, np.abs(want).max()))


from hypothesis import HealthCheck, given, settings, strategies as st  # noqa: E402


@_without_a_gpu
@settings(max_examples=20, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(E=st.sampled_from([2, 4, 8]), kfrac=st.sampled_from([1, 2, 4]), Tk=st.integers(1, 6),
       H=st.sampled_from([32, 64, 96]), Ii=st.sampled_from([32, 64]), gemma=st.booleans(), seed=st.integers(0, 1000))
def test_expert_blocks_over_drawn_sizes(E, kfrac, Tk, H, Ii, gemma, seed):
    """Both expert blocks over drawn expert counts, selection widths (down to
    one expert a token, up to every expert), token counts and widths: always
    one verified dispatch whose result is the dense block's."""
    from metaljax_amd import moe
    K = max(1, E // kfrac)
    moe.reset_stats()
    qmm.reset_stats()
    qmm._BUILT.clear()
    qmm._SHARED.clear()
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((Tk, H)) / 8).astype(np.float32)
    if gemma:
        packs3 = [T.make_mxfp4_experts(r, c, E, seed=seed + i) for i, (r, c) in enumerate(((Ii, H), (Ii, H), (H, Ii)))]
        raw = (x, rng.standard_normal((H, E)).astype(np.float32), (1.0 + rng.standard_normal(H) / 8).astype(np.float32),
               packs3[0][0], packs3[0][1], packs3[1][0], packs3[1][1], packs3[2][0], packs3[2][1],
               (1.0 + rng.standard_normal(E) / 8).astype(np.float32))
        text = T.moe_block_gemma4_mxfp4(E, Tk, H, Ii, K)
    else:
        gu_c, gu_s, _ = T.make_mxfp4_experts(2 * Ii, H, E, seed=seed)
        d_c, d_s, _ = T.make_mxfp4_experts(H, Ii, E, seed=seed + 1)
        raw = (x, (rng.standard_normal((H, E)) / 8).astype(np.float32), rng.standard_normal(E).astype(np.float32),
               gu_c, gu_s, d_c, d_s, (rng.standard_normal((E, 2 * Ii)) / 8).astype(np.float32),
               (rng.standard_normal((E, H)) / 8).astype(np.float32))
        text = T.moe_block_mxfp4(E, Tk, H, Ii, K)
    args = [I.from_numpy(a) for a in raw]
    with pytest.MonkeyPatch.context() as mp:
        mp.setattr(qmm, "DEVICE", "cpu")
        mp.setattr(moe, "emit_dot", _oracle_expert_product([]))
        (buf,) = engine.execute(engine.compile_program(text), args)
        st_ = moe.stats()
        assert st_["recognized"] == 1 and st_["verified"] == 1 and st_["dispatches"] == 1 and st_["fallbacks"] == 0, st_
        got = I.host(buf.data).a
        mp.setattr(qmm, "ENABLED", False)
        (lit,) = engine.execute(engine.compile_program(text), args)
    want = I.host(lit.data).a
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-5 * max(1.0, np.abs(want).max()))


def test_expert_dispatch_disabled_by_its_flag(monkeypatch):
    """METALJAX_MOE=0 (the reference's tests flip moe.ENABLED at run time,
    tests/test_moe.py:406-417): the block stays dense, its quantized dots are
    still fused one by one; the reference's names for the planner are there."""
    from metaljax_amd import moe
    moe.reset_stats()
    monkeypatch.setattr(moe, "ENABLED", False)
    st = qmm.analyze(engine.compile_program(T.moe_block_mxfp4(4, 3, 64, 32, 2)).interp)
    assert st.moe == [] and len(st.matches) == 2 and not any(m.absorbed for m in st.matches)
    assert moe.stats()["recognized"] == 0 and moe.stats()["gather_mm"] == 0
    monkeypatch.setattr(moe, "ENABLED", True)
    st = qmm.analyze(engine.compile_program(T.moe_block_mxfp4(4, 3, 64, 32, 2)).interp)
    assert len(st.moe) == 1 and isinstance(st.moe[0], moe.Match) and callable(moe.analyze)


def test_a_router_that_is_not_a_top_k_scatter_is_refused():
    from metaljax_amd import moe
    E, Tk, H, Ii, K = 4, 3, 64, 32, 2
    text = T.moe_block_mxfp4(E, Tk, H, Ii, K)
    # the one-hot compares with LT instead of EQ: not a scatter of the selection
    bad = text.replace("stablehlo.compare EQ, %idxb, %io", "stablehlo.compare LT, %idxb, %io")
    ex = engine.compile_program(bad)
    st = qmm.analyze(ex.interp)
    assert st.moe == [] and not any(m.absorbed for m in st.matches) and len(st.roots) == 2
    # the expert outputs are also returned: a region value read outside the region
    shared = text.replace("-> tensor<3x64xf32> {", "-> (tensor<3x64xf32>, tensor<4x3x64xf32>) {", 1).replace(
        "return %out : tensor<3x64xf32>", "return %out, %y : tensor<3x64xf32>, tensor<4x3x64xf32>")
    st = qmm.analyze(engine.compile_program(shared).interp)
    assert st.moe == []


def test_near_misses_of_the_expert_sum_are_refused():
    """The root must be a sum over experts of outputs times top-k scores
    (reference tests/test_moe.py:328-385): a max over experts, and scores that
    are a dense function of the logits, leave the block dense."""
    E, Tk, H, Ii, K = 4, 3, 64, 32, 2
    text = T.moe_block_mxfp4(E, Tk, H, Ii, K)
    root = "%out = stablehlo.reduce(%ys init: %zero) applies stablehlo.add across dimensions = [0]"
    assert root in text
    as_max = text.replace(root, "%out = stablehlo.reduce(%ys init: %ninf) applies stablehlo.maximum across dimensions = [0]")
    st = qmm.analyze(engine.compile_program(as_max).interp)
    assert st.moe == [] and len(st.roots) == 2 and not any(m.absorbed for m in st.matches)
    # every expert really routed: the scores are exp(logits), no selection anywhere near them
    scores = f"%s = stablehlo.reduce(%hw init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<{Tk}x{K}x{E}xf32>, tensor<f32>) -> tensor<{Tk}x{E}xf32>"
    assert scores in text
    dense = text.replace(scores, f"%s = stablehlo.exponential %logits : tensor<{Tk}x{E}xf32>")
    st = qmm.analyze(engine.compile_program(dense).interp)
    assert st.moe == [] and len(st.roots) == 2


def test_values_around_the_expert_sum_do_not_stop_the_dispatch():
    """The dense scores also returned (they then stay computed), and a shared
    branch added outside the sum (reference tests/test_moe.py:157-187): the
    block is still one dispatch."""
    from metaljax_amd import moe
    E, Tk, H, Ii, K = 4, 3, 64, 32, 2
    text = T.moe_block_mxfp4(E, Tk, H, Ii, K)
    sig, ret = f"-> tensor<{Tk}x{H}xf32> {{", f"return %out : tensor<{Tk}x{H}xf32>"
    assert sig in text and ret in text
    with_scores = text.replace(sig, f"-> (tensor<{Tk}x{H}xf32>, tensor<{Tk}x{E}xf32>) {{", 1).replace(
        ret, f"return %out, %s : tensor<{Tk}x{H}xf32>, tensor<{Tk}x{E}xf32>")
    ex = engine.compile_program(with_scores)
    st = qmm.analyze(ex.interp)
    assert len(st.moe) == 1
    by_name = {v.name: v for b in ir.walk_blocks(ex.interp.main.body) for o in b.ops for v in o.results}
    g = st.moe[0]
    assert by_name["s"] not in g.skip_keys and by_name["ys"] in g.skip_keys      # the scores live on, the dense product does not
    shared = text.replace(ret, f"%side = stablehlo.tanh %x : tensor<{Tk}x{H}xf32>\n    %both = stablehlo.add %out, %side : tensor<{Tk}x{H}xf32>\n    return %both : tensor<{Tk}x{H}xf32>")
    st = qmm.analyze(engine.compile_program(shared).interp)
    assert len(st.moe) == 1 and st.moe[0].out_shape == [Tk, H]


def test_the_one_pass_dead_sweep_agrees_with_a_fixpoint(monkeypatch):
    """`sweep_dead` walks the block once from the last op to the first; the
    argument for that is that it finds what rescanning to a fixpoint finds
    (reference tests/test_moe.py:609-636).  Here both run on the real block and
    must give the same set, and the sweep must add something."""
    from metaljax_amd import moe
    seen = []
    one_pass = moe.sweep_dead

    def both(block, skip, g):
        before = set(skip)
        got = set(one_pass(block, set(skip), g))
        keep, todo = set(), list(g.reads) + [g.router.indices, g.router.weights]
        while todo:
            v = todo.pop()
            if v not in keep:
                keep.add(v)
                if moe._producer(v) is not None:
                    todo.extend(moe._producer(v).operands)
        ref, changed = set(before), True
        while changed:
            changed = False
            for op in block.ops:
                key = moe.op_key(op)
                if (key is None or key in ref or key is g.key or op.name in moe.OPAQUE_OPS
                        or (op.regions and op.name != "stablehlo.reduce") or any(r in keep for r in op.results)):
                    continue
                readers = [u for r in op.results for u in r.uses]
                if readers and all(moe.op_key(u) is g.key or moe.op_key(u) in ref for u in readers):
                    ref.add(key)
                    changed = True
        assert got == ref, (got - ref, ref - got)
        seen.append((len(before), len(got)))
        return one_pass(block, skip, g)

    monkeypatch.setattr(moe, "sweep_dead", both)
    st = qmm.analyze(engine.compile_program(T.moe_block_mxfp4(4, 5, 64, 32, 2)).interp)
    assert len(st.moe) == 1 and seen and any(after > before for before, after in seen), seen


def test_a_dispatch_that_fails_its_check_runs_densely(monkeypatch):
    """Verification closes a structurally accepted but wrong reading: here the
    check itself is made to fail, and the dispatch is disabled, its matches
    emit their own dense products again."""
    from metaljax_amd import moe
    moe.reset_stats()
    E, Tk, H, Ii, K = 4, 1, 64, 32, 2          # one token: the decode step
    ex = engine.compile_program(T.moe_block_mxfp4(E, Tk, H, Ii, K))
    st = qmm.analyze(ex.interp)
    assert len(st.moe) == 1

    def broken(interp, g):
        raise moe.Reject("scores differ")
    monkeypatch.setattr(moe, "verify", broken)
    args, _ = _moe_inputs(E, Tk, H, Ii)
    assert qmm.prologue(ex.interp, [I.from_numpy(a) for a in args]) is True
    assert st.moe[0].disabled and moe.stats()["fallbacks"] == 1
    assert not any(m.absorbed for m in st.matches) and set(st.roots) == {m.key for m in st.matches}


def test_scores_that_are_not_a_top_k_scatter_leave_the_block_dense():
    """Scores masked by a threshold instead of scattered from a top-k
    (reference tests/test_moe.py:340-352), and Gemma4's router with the top-k
    taken out -- every expert weighted by its softmax probability
    (tests/test_moe.py:355-372), at one token and at several: no dispatch, the
    quantized products are still fused one by one."""
    from metaljax_amd import moe
    E, Tk, H, Ii, K = 4, 3, 64, 32, 2
    text = T.moe_block_mxfp4(E, Tk, H, Ii, K)
    scores = f"%s = stablehlo.reduce(%hw init: %zero) applies stablehlo.add across dimensions = [1] : (tensor<{Tk}x{K}x{E}xf32>, tensor<f32>) -> tensor<{Tk}x{E}xf32>"
    assert scores in text
    te, tei1 = f"tensor<{Tk}x{E}xf32>", f"tensor<{Tk}x{E}xi1>"
    masked = text.replace(scores, f"""%thrs = stablehlo.constant dense<2.000000e-01> : tensor<f32>
    %thr = stablehlo.broadcast_in_dim %thrs, dims = [] : (tensor<f32>) -> {te}
    %zte = stablehlo.broadcast_in_dim %zero, dims = [] : (tensor<f32>) -> {te}
    %pex = stablehlo.exponential %logits : {te}
    %keep = stablehlo.compare GT, %pex, %thr, FLOAT : ({te}, {te}) -> {tei1}
    %s = stablehlo.select %keep, %pex, %zte : {tei1}, {te}""")
    moe.reset_stats()
    st = qmm.analyze(engine.compile_program(masked).interp)
    assert st.moe == [] and moe.stats()["recognized"] == 0 and len(st.roots) == 2
    for tokens in (1, 6):
        text = T.moe_block_gemma4_mxfp4(E, tokens, H, Ii, K)
        scatter = text[text.index("    %vals, %idx = chlo.top_k"):text.index("    %g0 = stablehlo.dot_general")]
        dense = text.replace(scatter, f"    %s = stablehlo.add %probs, %probs : tensor<{tokens}x{E}xf32>\n")
        moe.reset_stats()
        st = qmm.analyze(engine.compile_program(dense).interp)
        assert st.moe == [] and moe.stats()["recognized"] == 0 and len(st.roots) == 3, tokens


@_without_a_gpu
def test_an_expert_weight_that_does_not_pack_leaves_the_block_dense_and_correct():
    """One down-projection value sits off the E2M1 grid (reference
    tests/test_moe.py:561-573 has the whole weight off it): that weight cannot
    be packed, so the dispatch must not claim its pack -- it is disabled at
    the first call, the other product is still fused on its own (here: by the
    stand-in), and the result is the dense block's."""
    from metaljax_amd import kernels, moe
    moe.reset_stats()
    E, Tk, H, Ii, K = 4, 3, 64, 32, 2
    text = T.moe_block_mxfp4(E, Tk, H, Ii, K)
    # the decode table's entry for code 5 (3.0) becomes 3.25: no E2M1 value
    assert text.count("3.000000e+00") >= 2
    head, sep, tail = text.rpartition("3.000000e+00")
    bad = head + "3.250000e+00" + tail                      # in the down projection's table (the second one)
    raw, _ = _moe_inputs(E, Tk, H, Ii)
    args = [I.from_numpy(a) for a in raw]
    ex = engine.compile_program(bad)
    st = qmm.analyze(ex.interp)
    assert len(st.moe) == 1
    assert qmm.prologue(ex.interp, args) is True
    assert st.moe[0].disabled and moe.stats()["fallbacks"] == 1 and qmm.stats()["fallbacks"] == 1
    live = [m for m in st.matches if not m.disabled]
    assert len(live) == 1 and not live[0].absorbed and set(st.roots) == {live[0].key}
    want = I.host(I.Interpreter(bad).run(args)[0]).a
    with pytest.MonkeyPatch.context() as mp:
        calls = {"qmm": [], "take_k": 0}
        mp.setattr(qmm, "DEVICE", "cpu")
        mp.setattr(kernels, "quantized_matmul", _oracle_dense_product(calls))
        (buf,) = engine.execute(ex, args)
    assert len(calls["qmm"]) == 1 and moe.stats()["dispatches"] == 0
    np.testing.assert_allclose(I.host(buf.data).a, want, rtol=3e-5, atol=3e-6 * max(1.0, np.abs(want).max()))


def _oracle_dense_product(calls):
    """A stand-in for kernels.quantized_matmul on host tensors (the oracle)."""
    import torch
    from oracle import qmm_oracle as O

    def product(x, w, scales, biases, transpose=True, group_size=64, bits=4, mode="affine", out_dtype=None):
        tables = np.asarray(scales) if mode == "mxfp4" else pack_tables_like(scales)
        y = O.qmm(x.float().numpy(), np.asarray(w), tables, None if biases is None else pack_tables_like(biases),
                  group_size, bits, mode)
        calls["qmm"].append(tuple(x.shape))
        return torch.from_numpy(y).to(out_dtype or x.dtype)
    return product


def pack_tables_like(a):
    return (a.to_f32() if isinstance(a, packing.BF16Array) else np.asarray(a)).astype(np.float32)


def test_router_check_catches_a_misplaced_weight(monkeypatch):
    """`verify` compares the evaluated scores with the scatter of the matched
    weights at the matched indices: a router record pointing at other weights
    (what a misread axis would amount to) fails it."""
    from metaljax_amd import moe
    E, Tk, H, Ii, K = 4, 3, 64, 32, 2
    ex = engine.compile_program(T.moe_block_mxfp4(E, Tk, H, Ii, K))
    g = qmm.analyze(ex.interp).moe[0]
    moe.verify(ex.interp, g)                               # the true reading passes
    by_name = {v.name: v for o in ex.interp.main.body.ops for v in o.results}
    g.router.weights = by_name["ex"]                       # un-normalised exponentials
    with pytest.raises(moe.Reject):
        moe.verify(ex.interp, g)
