"""`qmm.emit`'s own work -- which operand is the activation, how its axes are
permuted and flattened into [B, M, K], the gather through a pack's
permutation, how the kernel's [B, M, N] goes back into the dot's result
shape, packs bound per call inside a loop body -- on the catalogue of
recognized programs, without a GPU: the two kernel calls are stood in for by
the oracle on torch CPU tensors, everything around them is the product's
code.  (The same programs run on the real kernels in test_gpu_recognizer.py;
the comparison is the one of reference tests/test_qmm.py:261-282.)"""

import numpy as np
import pytest
import torch

import stablehlo_text as T
from metaljax_amd import engine, interpreter as I, kernels, packing, qmm
from oracle import qmm_oracle as O


# Packs are uploaded when a GPU is visible; the stand-ins below read them as host arrays.
pytestmark = pytest.mark.skipif(torch.cuda.is_available(),
                                reason="stands in for the kernels on a machine without a GPU; with one, "
                                       "test_gpu_recognizer.py runs the same programs on the kernels")


def _f32(a):
    if a is None:
        return None
    return a.to_f32() if isinstance(a, packing.BF16Array) else np.asarray(a)


@pytest.fixture(autouse=True)
def _kernels_stood_in_for(monkeypatch):
    qmm.reset_stats()
    qmm._BUILT.clear()
    qmm._SHARED.clear()
    calls = {"qmm": [], "take_k": 0}

    def quantized_matmul(x, w, scales, biases, transpose=True, group_size=64, bits=4, mode="affine",
                         out_dtype=None):
        assert transpose and isinstance(x, torch.Tensor) and x.device.type == "cpu" and x.is_contiguous()
        words = np.asarray(w)
        tables = np.asarray(scales) if mode == "mxfp4" else _f32(scales).astype(np.float32)
        y = O.qmm(x.float().numpy(), words, tables, None if biases is None else _f32(biases).astype(np.float32),
                  group_size, bits, mode)
        calls["qmm"].append((tuple(x.shape), tuple(words.shape), mode, group_size, bits))
        return torch.from_numpy(y).to(out_dtype or x.dtype)

    def take_k(x, perm):
        calls["take_k"] += 1
        return x[..., torch.from_numpy(np.asarray(perm).astype(np.int64))].contiguous()

    monkeypatch.setattr(qmm, "DEVICE", "cpu")
    monkeypatch.setattr(kernels, "quantized_matmul", quantized_matmul)
    monkeypatch.setattr(kernels, "take_k", take_k)
    yield calls


def compare(text, args, exact, packs=1):
    want = I.host(I.Interpreter(text).run(args)[0]).a.astype(np.float32)
    ex = engine.compile_program(text)
    (buf,) = engine.execute(ex, args)
    got = I.host(buf.data).a.astype(np.float32)
    assert qmm.stats()["packs"] == packs and qmm.stats()["fallbacks"] == 0
    scale = np.abs(exact).max()
    err_fused = np.abs(got - exact).max() / scale
    err_lit = np.abs(want - exact).max() / scale
    assert got.shape == want.shape == exact.shape
    assert err_fused <= err_lit * 1.5 + 1e-6, (err_fused, err_lit)
    np.testing.assert_allclose(got, want, rtol=2e-2, atol=1e-2 * scale)
    return ex


def dense_args(packed, scale, zero, g_idx, x):
    return [I.from_numpy(packed), I.from_numpy(scale, "bf16"), I.from_numpy(zero),
            I.from_numpy(g_idx), I.from_numpy(x, "bf16")]


def _x(seed, shape, mul=0.5):
    return T.bf16_round(np.random.default_rng(seed).standard_normal(shape).astype(np.float32) * mul)


@pytest.mark.parametrize("m,block", [(4, 128), (1, 64), (40, 32), (16, -1)])
def test_dense_subchannel(m, block, _kernels_stood_in_for):
    k, n = 256, 128
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, block, seed=m)
    x = _x(3, (m, k))
    compare(T.dense_sub(k, n, scale.shape[0], m), dense_args(packed, scale, zero, g_idx, x), x @ wref)
    (call,) = _kernels_stood_in_for["qmm"]
    assert call[0] == (m, k) and call[1][0] == n


def test_dense_int8_codes():
    k, n, m = 128, 64, 24
    q, _, scale, zero, g_idx, wref = T.quantize(k, n, 64, seed=5, bits=8)
    x = _x(3, (m, k))
    compare(T.dense_i8_codes(k, n, 2, m), dense_args(q, scale, zero, g_idx, x), x @ wref)


def test_perchannel():
    k, n, m = 128, 64, 3
    q, packed, _, _, _, _ = T.quantize(k, n, -1, seed=2)
    scale = T.bf16_round(np.random.default_rng(9).uniform(8.0, 40.0, n).astype(np.float32))
    x = _x(4, (m, k), 1.0)
    args = [I.from_numpy(packed), I.from_numpy(scale, "bf16"), I.from_numpy(x, "bf16")]
    compare(T.dense_perchannel(k, n, m), args, (x @ q.astype(np.float32)) / scale)


def test_interleaved_groups_run_through_the_permutation(_kernels_stood_in_for):
    k, n, m, ng = 256, 64, 4, 2
    g_idx = (np.arange(k) % ng).astype(np.float32)
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, k // ng, seed=11, g_idx=g_idx)
    x = _x(3, (m, k), 1.0)
    compare(T.dense_sub(k, n, ng, m), dense_args(packed, scale, zero, g_idx, x), x @ wref)
    assert qmm.stats()["perms"] == 1 and _kernels_stood_in_for["take_k"] == 1


@pytest.mark.parametrize("t,k", [(5, 128), (40, 512)])
def test_dense_mxfp4(t, k):
    n = 48
    codes, blocks, sb, w = T.random_mxfp4((n, k), seed=1)
    x = _x(2, (t, k), 1.0)
    compare(T.dense_mxfp4(n, k, t), [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")], x @ w.T)
    assert qmm.stats()["mxfp4"] == 1


def test_batched_experts_mxfp4(_kernels_stood_in_for):
    e, n, k, t = 3, 32, 64, 4
    codes, blocks, sb, w = T.random_mxfp4((e, n, k), seed=7)
    x = _x(2, (e, t, k), 1.0)
    args = [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")]
    compare(T.experts_mxfp4(e, n, k, t), args, np.einsum("etk,enk->etn", x, w))
    assert qmm.stats()["batched"] == 1
    (call,) = _kernels_stood_in_for["qmm"]
    assert call[0] == (e, t, k) and call[1][:2] == (e, n)


def test_einsum_projections_keep_their_axes():
    """[B, T, D] x W -> [B, T, heads, head_dim] and back: the activation's
    leading axes flatten into M, the weight's free axes come back split
    (reference tests/test_qmm.py:283-330)."""
    d, heads, hd, b, t = 128, 4, 16, 2, 3
    q, packed, scale, zero, g_idx, wref = T.quantize(d, heads * hd, 64, seed=12)
    x = _x(5, (b, t, d))
    exact = (x.reshape(b * t, d) @ wref).reshape(b, t, heads, hd)
    compare(T.einsum_sub(d, heads, hd, 2, b, t), dense_args(packed, scale, zero, g_idx, x), exact)
    qmm.reset_stats()
    nh, h, dd = 4, 16, 128
    q, packed, scale, zero, g_idx, wref = T.quantize(nh * h, dd, 32, seed=13)
    x = _x(6, (b, t, nh, h))
    exact = (x.reshape(b * t, nh * h) @ wref).reshape(b, t, dd)
    compare(T.einsum_out_proj(nh, h, dd, scale.shape[0], b, t), dense_args(packed, scale, zero, g_idx, x), exact)


def test_decode_loop_packs_once_across_steps_and_calls(_kernels_stood_in_for):
    k, m, steps = 128, 2, 3
    q, packed, scale, zero, g_idx, wref = T.quantize(k, k, 64, seed=10)
    scale = T.bf16_round(scale * 0.2)
    x = _x(1, (m, k), 1.0)
    text = T.decode_loop(k, 2, m, steps)
    args = dense_args(packed, scale, zero, g_idx, x)
    want = I.host(I.Interpreter(text).run(args)[0]).a
    ex = engine.compile_program(text)
    for _ in range(2):
        (y,) = engine.execute(ex, args)
    assert qmm.stats()["packs"] == 1 and len(_kernels_stood_in_for["qmm"]) == 2 * steps
    np.testing.assert_allclose(I.host(y).a, want, rtol=4e-2, atol=2e-2 * np.abs(want).max())
    args2 = dense_args(packed.copy(), T.bf16_round(scale * 0.5), zero, g_idx, x)
    (y2,) = engine.execute(ex, args2)
    want2 = I.host(I.Interpreter(text).run(args2)[0]).a
    assert qmm.stats()["packs"] == 2
    np.testing.assert_allclose(I.host(y2).a, want2, rtol=4e-2, atol=2e-2 * np.abs(want2).max())


def test_weight_as_the_left_operand_comes_back_transposed(_kernels_stood_in_for):
    """`nk,tk->nt`: the packed weight is the dot's left operand, so the
    kernel's [T, N] is handed back as [N, T]."""
    n, k, gs, t = 64, 128, 64, 5
    q, scale, zero, ref = T.affine_grouped_data(n, k, gs, 41)
    x = _x(42, (t, k), 0.3)
    text = T.affine_grouped(n, k, gs, t)
    tk, nk, tn, nt = (f"tensor<{t}x{k}xbf16>", f"tensor<{n}x{k}xbf16>", f"tensor<{t}x{n}xbf16>",
                      f"tensor<{n}x{t}xbf16>")
    dot = f"%y = stablehlo.dot_general %x, %w, contracting_dims = [1] x [1] : ({tk}, {nk}) -> {tn}"
    assert dot in text
    text = text.replace(dot, f"%y = stablehlo.dot_general %w, %x, contracting_dims = [1] x [1] : ({nk}, {tk}) -> {nt}")
    text = text.replace(f"-> {tn} {{", f"-> {nt} {{").replace(f"return %y : {tn}", f"return %y : {nt}")
    args = [I.from_numpy(q), I.from_numpy(scale), I.from_numpy(zero), I.from_numpy(x, "bf16")]
    want_w = T.bf16_round(scale)[:, np.arange(k) // gs] * (q.astype(np.float32) - zero[:, np.arange(k) // gs])
    ex = compare(text, args, want_w @ x.T)
    assert ex.interp._qmm.matches[0].swapped
    (call,) = _kernels_stood_in_for["qmm"]
    assert call[0] == (t, k)


from hypothesis import HealthCheck, given, settings, strategies as st  # noqa: E402


@settings(max_examples=40, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(k=st.sampled_from([64, 128, 192, 256, 384]), n=st.integers(4, 40).map(lambda v: 8 * v),
       block=st.sampled_from([32, 64, 128, -1]), m=st.integers(1, 40), el=st.sampled_from(["bf16", "f32"]),
       bits=st.sampled_from([4, 8]), seed=st.integers(0, 10_000))
def test_dense_subchannel_over_drawn_shapes(k, n, block, m, el, bits, seed):
    """The sub-channel chain over drawn sizes, group widths, code widths and
    element types: recognized, packed once, and the fused result within the
    literal chain's distance of the exact product."""
    if block > 0 and k % block:
        block = 32
    qmm.reset_stats()
    qmm._BUILT.clear()
    qmm._SHARED.clear()
    q, packed, scale, zero, g_idx, wref = T.quantize(k, n, block, seed=seed, bits=bits, bf16=el == "bf16")
    x = np.random.default_rng(seed + 1).standard_normal((m, k)).astype(np.float32) * 0.5
    if el == "bf16":
        x = T.bf16_round(x)
    ng = scale.shape[0]
    text = T.dense_sub(k, n, ng, m, el=el) if bits == 4 else T.dense_i8_codes(k, n, ng, m, el=el)
    args = [I.from_numpy(packed if bits == 4 else q), I.from_numpy(scale, el), I.from_numpy(zero),
            I.from_numpy(g_idx), I.from_numpy(x, el)]
    compare(text, args, x @ wref)
    assert qmm.stats()["recognized"] == 1


@settings(max_examples=30, deadline=None, suppress_health_check=[HealthCheck.function_scoped_fixture])
@given(n=st.integers(1, 12).map(lambda v: 8 * v), k=st.integers(1, 12).map(lambda v: 32 * v), t=st.integers(1, 24),
       experts=st.sampled_from([None, 2, 3]), rows_form=st.booleans(), seed=st.integers(0, 10_000))
def test_mxfp4_chains_over_drawn_shapes(n, k, t, experts, rows_form, seed):
    """MXFP4 weights of drawn sizes, dense and batched over experts, in both
    spellings of the E2M1 decode (a gather of the value table in line, or jax's
    private @_take callee): recognized, packed, the fused result the exact
    product up to the activations' rounding."""
    qmm.reset_stats()
    qmm._BUILT.clear()
    qmm._SHARED.clear()
    lead = () if experts is None else (experts,)
    codes, blocks, sb, w = T.random_mxfp4(lead + (n, k), seed=seed)
    x = _x(seed + 1, lead + (t, k), 1.0)
    if rows_form:
        text = T.dense_mxfp4_rows(n, k, t, e=experts)
    else:
        text = T.dense_mxfp4(n, k, t) if experts is None else T.experts_mxfp4(experts, n, k, t)
    exact = x @ w.T if experts is None else np.einsum("etk,enk->etn", x, w)
    compare(text, [I.from_numpy(blocks), I.from_numpy(sb), I.from_numpy(x, "bf16")], exact)
    assert qmm.stats()["mxfp4"] == 1 and qmm.stats()["batched"] == (0 if experts is None else 1)
