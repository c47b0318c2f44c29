"""Recognized programs executed for real: StableHLO text -> recognizer ->
pack -> the HIP kernels through `emit`, against the literal interpretation of
the same program and the exact float32 product (the comparison of reference
tests/test_qmm.py:261-282: the fused result must be no worse than the literal
chain, and within rtol 2e-2 / atol 1e-2*max of it)."""

import numpy as np
import pytest
import torch

import stablehlo_text as T
from metaljax_amd import engine, interpreter as I, moe, qmm

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh():
    qmm.reset_stats()
    moe.reset_stats()
    qmm._BUILT.clear()
    qmm._SHARED.clear()
    yield


def compare(text, args, exact, packs=1):
    lit = I.Interpreter(text)
    want = I.host(lit.run(args)[0]).a.astype(np.float32)
    ex = engine.compile_program(text)
    (buf,) = engine.execute(ex, args)
    y = buf.data
    assert isinstance(y, torch.Tensor) and y.is_cuda          # the fused op ran on the device
    got = y.float().cpu().numpy()
    assert qmm.stats()["packs"] == packs and qmm.stats()["fallbacks"] == 0
    scale = np.abs(exact).max()
    err_fused = np.abs(got - exact).max() / scale
    err_lit = np.abs(want - exact).max() / scale
    assert got.shape == want.shape
    assert err_fused <= err_lit * 1.5 + 1e-6, (err_fused, err_lit)
    np.testing.assert_allclose(got, want, rtol=2e-2, atol=1e-2 * scale)
    return ex


def dense_args(packed, scale, zero, g_idx, x):
    return [I.from_numpy(packed), I.from_numpy(scale, "bf16"), I.from_numpy(zero),
            I.from_numpy(g_idx), I.from_numpy(x, "bf16")]


@pytest.mark.parametrize("m,block", [(4, 128), (1, 64), (40, 32), (16, -1)])
def test_dense_subchannel(m, block):
    k, n = 256, 128
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, block, seed=m)
    x = T.bf16_round(np.random.default_rng(3).standard_normal((m, k)).astype(np.float32) * 0.5)
    compare(T.dense_sub(k, n, scale.shape[0], m), dense_args(packed, scale, zero, g_idx, x), x @ wref)


def test_dense_int8_codes():
    k, n, m = 128, 64, 24
    q, _, scale, zero, g_idx, wref = T.quantize(k, n, 64, seed=5, bits=8)
    x = T.bf16_round(np.random.default_rng(3).standard_normal((m, k)).astype(np.float32) * 0.5)
    compare(T.dense_i8_codes(k, n, 2, m), dense_args(q, scale, zero, g_idx, x), x @ wref)


def test_perchannel():
    k, n, m = 128, 64, 3
    q, packed, _, _, _, _ = T.quantize(k, n, -1, seed=2)
    scale = T.bf16_round(np.random.default_rng(9).uniform(8.0, 40.0, n).astype(np.float32))
    x = T.bf16_round(np.random.default_rng(4).standard_normal((m, k)).astype(np.float32))
    args = [I.from_numpy(packed), I.from_numpy(scale, "bf16"), I.from_numpy(x, "bf16")]
    compare(T.dense_perchannel(k, n, m), args, (x @ q.astype(np.float32)) / scale)


def test_interleaved_groups_run_through_the_permutation():
    k, n, m, ng = 256, 64, 4, 2
    g_idx = (np.arange(k) % ng).astype(np.float32)
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, k // ng, seed=11, g_idx=g_idx)
    x = T.bf16_round(np.random.default_rng(3).standard_normal((m, k)).astype(np.float32))
    compare(T.dense_sub(k, n, ng, m), dense_args(packed, scale, zero, g_idx, x), x @ wref)
    assert qmm.stats()["perms"] == 1


@pytest.mark.parametrize("t,k", [(5, 128), (40, 512)])
def test_dense_mxfp4(t, k):
    n = 48
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=1)
    x = T.bf16_round(np.random.default_rng(2).standard_normal((t, k)).astype(np.float32))
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")]
    compare(T.dense_mxfp4(n, k, t), args, x @ w.T)
    assert qmm.stats()["mxfp4"] == 1


def test_batched_experts_mxfp4():
    e, n, k, t = 3, 32, 64, 4
    codes, blocks, sb, w = T.random_mxfp4((e, n, k), seed=7)
    x = T.bf16_round(np.random.default_rng(2).standard_normal((e, t, k)).astype(np.float32))
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")]
    compare(T.experts_mxfp4(e, n, k, t), args, np.einsum("etk,enk->etn", x, w))
    assert qmm.stats()["batched"] == 1


def test_decode_loop_packs_once_across_steps_and_calls():
    k, m, steps = 128, 2, 3
    q, packed, scale, zero, g_idx, wref = T.quantize(k, k, 64, seed=10)
    scale = T.bf16_round(scale * 0.2)
    wref = wref * 0.0 + scale[g_idx.astype(np.int32)] * (q.astype(np.float32) - zero[g_idx.astype(np.int32)])
    x = T.bf16_round(np.random.default_rng(1).standard_normal((m, k)).astype(np.float32))
    text = T.decode_loop(k, 2, m, steps)
    args = dense_args(packed, scale, zero, g_idx, x)
    want = I.host(I.Interpreter(text).run(args)[0]).a
    ex = engine.compile_program(text)
    for _ in range(2):
        (y,) = engine.execute(ex, args)
    got = I.host(y).a
    assert qmm.stats()["packs"] == 1
    np.testing.assert_allclose(got, want, rtol=4e-2, atol=2e-2 * np.abs(want).max())
    # new weight buffers repack, and the result follows the new weights
    args2 = dense_args(packed.copy(), T.bf16_round(scale * 0.5), zero, g_idx, x)
    (y2,) = engine.execute(ex, args2)
    want2 = I.host(I.Interpreter(text).run(args2)[0]).a
    assert qmm.stats()["packs"] == 2
    np.testing.assert_allclose(I.host(y2).a, want2, rtol=4e-2, atol=2e-2 * np.abs(want2).max())


def test_gathered_expert_dispatch_over_a_recognized_pack():
    """Top-2 routing over experts whose weights the recognizer packed: the
    expert-indexed product + weighted sum against the dense reference
    (reference tests/test_moe.py:514-557)."""
    e, n, k, t, topk = 4, 64, 128, 12, 2
    codes, blocks, sb, w = T.random_mxfp4((e, n, k), seed=21)
    xe = T.bf16_round(np.random.default_rng(2).standard_normal((e, 1, k)).astype(np.float32))
    ex = engine.compile_program(T.experts_mxfp4(e, n, k, 1))
    st = qmm.analyze(ex.interp)
    qmm.prologue(ex.interp, [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(xe, "bf16")])
    mt = st.matches[0]
    rng = np.random.default_rng(5)
    x = T.bf16_round(rng.standard_normal((t, k)).astype(np.float32))
    logits = rng.standard_normal((t, e)).astype(np.float32)
    idx = np.argsort(-logits, axis=1)[:, :topk]
    p = np.exp(logits - logits.max(1, keepdims=True))
    p = p / p.sum(1, keepdims=True)
    wts = np.take_along_axis(p, idx, 1)
    xd = qmm.to_device(I.from_numpy(x, "bf16"))
    y = moe.expert_dispatch(ex.interp, mt, xd, torch.from_numpy(idx).cuda(),
                            torch.from_numpy(wts).cuda())
    want = np.zeros((t, n), np.float32)
    for i in range(t):
        for j in range(topk):
            want[i] += wts[i, j] * (x[i] @ w[idx[i, j]].T)
    got = y.float().cpu().numpy()
    assert moe.stats()["gather_qmm"] == 1 and moe.stats()["dispatches"] == 1
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-2



@pytest.mark.parametrize("E,K", [(4, 2), (8, 4)])
@pytest.mark.parametrize("Tk", [1, 3])
def test_mxfp4_experts_gathered(E, K, Tk):
    """The gpt-oss block end to end (reference tests/test_moe.py:514-557):
    the dense dispatch is recognized, both projections run as expert-indexed
    quantized products on the device, the routing-weighted sum follows there,
    and the result matches the dense block on exactly dequantized weights
    (float32 graph: rtol 3e-5) and the literal run of the same module."""
    import stablehlo_text as S
    moe.reset_stats()
    H, Ii = 64, 32
    rng = np.random.default_rng(E)
    gu_c, gu_s, gu_ref = S.make_mxfp4_experts(2 * Ii, H, E, seed=E)
    d_c, d_s, d_ref = S.make_mxfp4_experts(H, Ii, E, seed=E + 1)
    x = (rng.standard_normal((Tk, H)) / 8).astype(np.float32)
    wr = (rng.standard_normal((H, E)) / 8).astype(np.float32)
    br = rng.standard_normal(E).astype(np.float32)
    bgu = (rng.standard_normal((E, 2 * Ii)) / 8).astype(np.float32)
    bd = (rng.standard_normal((E, H)) / 8).astype(np.float32)
    text = S.moe_block_mxfp4(E, Tk, H, Ii, K)
    args = [I.from_numpy(a) for a in (x, wr, br, gu_c, gu_s, d_c, d_s, bgu, bd)]
    ex = engine.compile_program(text)
    (buf,) = engine.execute(ex, args)
    st, qst = moe.stats(), qmm.stats()
    assert st["recognized"] == 1 and st["verified"] == 1 and st["fallbacks"] == 0, st
    assert st["gather_qmm"] >= 2 and st["dispatches"] == 1, st       # both projections read packs
    assert qst["mxfp4"] == 2 and qst["fallbacks"] == 0, qst
    assert isinstance(buf.data, torch.Tensor) and buf.data.is_cuda
    got = buf.data.float().cpu().numpy()
    want = S.moe_block_reference(x, wr, br, gu_ref, d_ref, bgu, bd, K)
    np.testing.assert_allclose(got, want, rtol=3e-5, atol=3e-6 * max(1.0, np.abs(want).max()))
    lit = I.host(I.Interpreter(text).run(args)[0]).a
    np.testing.assert_allclose(got, lit, rtol=3e-5, atol=3e-6 * max(1.0, np.abs(want).max()))
    # a second execute on the same buffers packs nothing new
    engine.execute(ex, args)
    assert qmm.stats()["packs"] == 2 and moe.stats()["dispatches"] == 2


def test_the_dispatch_runs_between_its_projections_on_the_device():
    """The gpt-oss block at the model's own widths (hidden and intermediate size
    2880, reference scripts/model_bench/mxfp4_gpt_oss.py:90-110; eight experts,
    top-4, 16 tokens): the buffers are device-resident, and from the first
    expert-indexed product to the routing-weighted sum nothing is copied back to
    the host -- the second projection reads the first one's result where it
    lies (reference moe.py:1283-1340, :1425-1461 run the closure list on device
    arrays)."""
    import stablehlo_text as S
    moe.reset_stats()
    E, K, Tk, H, Ii = 8, 4, 16, 2880, 2880
    rng = np.random.default_rng(2880)
    gu_c, gu_s, gu_ref = S.make_mxfp4_experts(2 * Ii, H, E, seed=51)
    d_c, d_s, d_ref = S.make_mxfp4_experts(H, Ii, E, seed=52)
    x = (rng.standard_normal((Tk, H)) / 8).astype(np.float32)
    wr = (rng.standard_normal((H, E)) / 8).astype(np.float32)
    br = rng.standard_normal(E).astype(np.float32)
    bgu = (rng.standard_normal((E, 2 * Ii)) / 8).astype(np.float32)
    bd = (rng.standard_normal((E, H)) / 8).astype(np.float32)
    text = S.moe_block_mxfp4(E, Tk, H, Ii, K)
    f32, u8 = engine._ENUM["F32"], engine._ENUM["U8"]
    bufs = [engine.buffer_from_host(a, f32 if a.dtype == np.float32 else u8, a.shape)
            for a in (x, wr, br, gu_c, gu_s, d_c, d_s, bgu, bd)]
    assert all(b.data.is_cuda for b in bufs)
    ex = engine.compile_program(text)
    (buf,) = engine.execute(ex, bufs)
    st, qst = moe.stats(), qmm.stats()
    assert st["recognized"] == 1 and st["verified"] == 1 and st["fallbacks"] == 0, st
    assert st["gather_qmm"] == 2 and st["dispatches"] == 1, st
    assert st["host_copies"] == 0, st                      # nothing came back between the projections
    assert qst["mxfp4"] == 2 and qst["fallbacks"] == 0, qst
    assert buf.data.is_cuda
    got = buf.data.float().cpu().numpy()
    want = S.moe_block_reference(x, wr, br, gu_ref, d_ref, bgu, bd, K)
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 1e-4
    (again,) = engine.execute(ex, bufs)                    # a decode step later: same packs, still no copy back
    assert qmm.stats()["packs"] == 2 and moe.stats()["dispatches"] == 2 and moe.stats()["host_copies"] == 0
    assert torch.equal(again.data, buf.data)


def test_an_expert_nobody_selects_is_never_evaluated():
    """The one intended divergence from the dense block (reference
    tests/test_moe.py:428-458): an expert whose output is not finite and whose
    router logit keeps every token away from it gives NaN in the dense sum
    (inf times an exact zero) and nothing at all in the dispatch, which never
    evaluates it."""
    import stablehlo_text as S
    moe.reset_stats()
    E, K, Tk, H, Ii = 4, 2, 2, 64, 32
    rng = np.random.default_rng(37)
    gu_c, gu_s, gu_ref = S.make_mxfp4_experts(2 * Ii, H, E, seed=37)
    d_c, d_s, d_ref = S.make_mxfp4_experts(H, Ii, E, seed=38)
    x = (rng.standard_normal((Tk, H)) / 8).astype(np.float32)
    wr = (rng.standard_normal((H, E)) / 8).astype(np.float32)
    br = rng.standard_normal(E).astype(np.float32)
    bgu = (rng.standard_normal((E, 2 * Ii)) / 8).astype(np.float32)
    bd = (rng.standard_normal((E, H)) / 8).astype(np.float32)
    bd[3] = np.inf
    br[3] = -1e4
    text = S.moe_block_mxfp4(E, Tk, H, Ii, K)
    args = [I.from_numpy(a) for a in (x, wr, br, gu_c, gu_s, d_c, d_s, bgu, bd)]
    (buf,) = engine.execute(engine.compile_program(text), args)
    assert moe.stats()["recognized"] == 1 and moe.stats()["dispatches"] == 1 and moe.stats()["fallbacks"] == 0
    got = buf.data.float().cpu().numpy()
    lit = I.host(I.Interpreter(text).run(args)[0]).a
    assert np.isnan(lit).any(), "the dense block should carry the NaN"
    assert np.isfinite(got).all(), "the dispatch should stay finite"
    bd0 = bd.copy()
    bd0[3] = 0.0
    want = S.moe_block_reference(x, wr, br, gu_ref, d_ref, bgu, bd0, K)
    np.testing.assert_allclose(got, want, rtol=3e-5, atol=3e-6 * max(1.0, np.abs(want).max()))


def test_gather_qmm_with_several_rows_per_pair():
    """x [T, M, K]: every pair multiplies M rows (mx.gather_qmm's general
    form, reference src/metaljax/moe.py:1293-1301)."""
    from metaljax_amd import kernels as K
    from oracle import qmm_oracle as O
    rng = np.random.default_rng(3)
    e, n, k, t, m, pairs = 3, 72, 256, 5, 4, 7
    codes = rng.integers(0, 16, size=(e, n, k), dtype=np.uint8)
    words = O.pack_codes(codes, 4)
    s = O.round_bf16(rng.uniform(0.005, 0.02, (e, n, k // 64)).astype(np.float32))
    b = O.round_bf16(-8 * s)
    x = O.round_bf16(rng.standard_normal((t, m, k)).astype(np.float32))
    lhs = rng.integers(0, t, size=pairs).astype(np.int32)
    rhs = rng.integers(0, e, size=pairs).astype(np.int32)
    dev = lambda a: torch.from_numpy(O.f32_to_bf16_bits(a).view(np.int16)).cuda().view(torch.bfloat16)
    y = K.gather_qmm(dev(x), torch.from_numpy(words.view(np.int32)).cuda(), dev(s), dev(b),
                     torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), group_size=64, bits=4,
                     out_dtype=torch.float32)
    assert tuple(y.shape) == (pairs, m, n)
    want = O.gather_qmm(x, words, s, b, lhs, rhs, 64, 4)
    assert O.rel_l2(y.cpu().numpy(), want) <= 2e-5
    y0 = K.gather_qmm(dev(x[:pairs]), torch.from_numpy(words.view(np.int32)).cuda(), dev(s), dev(b), None,
                      torch.from_numpy(rhs[:t]).cuda(), group_size=64, bits=4, out_dtype=torch.float32)
    want0 = O.gather_qmm(x, words, s, b, np.arange(t), rhs[:t], 64, 4)
    assert O.rel_l2(y0.cpu().numpy(), want0) <= 2e-5


def test_a_dot_left_to_the_interpreter_runs_on_the_device():
    """A dot that is not rewritten (here: an ordinary float projection) is one
    library matmul on the GPU, float32 accumulate, rounded once to the result
    type -- the literal dot of reference src/metaljax/ops/linalg.py:91-142."""
    k, n, m = 512, 384, 64
    rng = np.random.default_rng(9)
    w = T.bf16_round(rng.standard_normal((k, n)).astype(np.float32))
    r = T.bf16_round(rng.standard_normal((k,)).astype(np.float32))
    x = T.bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    ex = engine.compile_program(T.float_dot(k, n, m))
    (buf,) = engine.execute(ex, [I.from_numpy(w, "bf16"), I.from_numpy(r, "bf16"), I.from_numpy(x, "bf16")])
    assert qmm.stats()["recognized"] == 0
    assert isinstance(buf.data, torch.Tensor) and buf.data.is_cuda and buf.data.dtype == torch.bfloat16
    want = x.astype(np.float64) @ T.bf16_round(w * r[:, None]).astype(np.float64)
    got = buf.data.float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-2 * np.abs(want).max())
    from metaljax_amd.packing import f32_to_bf16_bits
    assert engine.to_host(buf) == f32_to_bf16_bits(got).tobytes()


# ------------------------------------------ device-resident engine buffers ----

def test_engine_buffers_live_on_the_device():
    """`buffer_from_host` uploads once (reference engine.py:118-159: a buffer's
    data is a device array): the tensor has the advertised element type,
    `buffer_pointer` is its device address and `to_host` gives the bytes back."""
    from metaljax_amd.packing import f32_to_bf16_bits
    rng = np.random.default_rng(0)
    cases = [("BF16", f32_to_bf16_bits(rng.standard_normal((3, 8)).astype(np.float32)), torch.bfloat16),
             ("F32", rng.standard_normal((2, 5)).astype(np.float32), torch.float32),
             ("S8", rng.integers(-8, 8, (4, 4)).astype(np.int8), torch.int8),
             ("U32", rng.integers(0, 2**32, (3, 3), dtype=np.uint64).astype(np.uint32), torch.uint32),
             ("PRED", rng.integers(0, 2, (7,)).astype(np.bool_), torch.bool)]
    for name, arr, dt in cases:
        b = engine.buffer_from_host(arr, engine._ENUM[name], arr.shape)
        assert isinstance(b.data, torch.Tensor) and b.data.is_cuda and b.data.dtype == dt, name
        assert b.nbytes == arr.nbytes and engine.buffer_pointer(b) == b.data.data_ptr()
        assert engine.to_host(b) == arr.tobytes(), name


def test_execute_reads_resident_buffers_without_host_copies():
    """After the first call has packed the weight, `execute` on device-resident
    buffers copies nothing back to the host: the activation goes to the kernel
    as it lies, the result stays a device tensor (reference engine.py:385-417)."""
    from metaljax_amd import synth
    from metaljax_amd.packing import f32_to_bf16_bits
    m, n, k = 4, 128, 512
    rng = np.random.default_rng(12)
    q = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    s = T.bf16_round(rng.uniform(0.005, 0.02, size=(n, k // 64)).astype(np.float32))
    z = rng.integers(-2, 3, size=(n, k // 64)).astype(np.int8)
    x = T.bf16_round(rng.standard_normal((m, k)).astype(np.float32))
    ex = engine.compile_program(synth.affine_program_text(m, n, k))
    bufs = [engine.buffer_from_host(q, engine._ENUM["S8"], q.shape),
            engine.buffer_from_host(f32_to_bf16_bits(s), engine._ENUM["BF16"], s.shape),
            engine.buffer_from_host(z, engine._ENUM["S8"], z.shape),
            engine.buffer_from_host(f32_to_bf16_bits(x), engine._ENUM["BF16"], x.shape)]
    assert all(b.data.is_cuda for b in bufs)
    (y0,) = engine.execute(ex, bufs)
    assert qmm.stats()["packs"] == 1 and qmm.stats()["fallbacks"] == 0
    before = I.HOST_COPIES[0]
    (y1,) = engine.execute(ex, bufs)
    assert I.HOST_COPIES[0] == before                      # nothing came back to the host
    assert qmm.stats()["packs"] == 1                       # the pack was found by buffer identity
    assert y1.data.is_cuda and y1.data.dtype == torch.bfloat16
    w = (q.astype(np.float32) - np.repeat(z, 64, axis=1)) * np.repeat(s, 64, axis=1)
    want = x @ w.T
    got = np.frombuffer(engine.to_host(y1), np.uint16).reshape(m, n)
    got = (got.astype(np.uint32) << 16).view(np.float32)
    assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()
    assert engine.to_host(y0) == engine.to_host(y1)
