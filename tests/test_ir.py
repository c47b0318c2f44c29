"""The StableHLO text front end and the literal op handlers."""

import numpy as np
import pytest

from metaljax_amd import interpreter as I, ir


def run(text, *args):
    return [I.host(v) for v in I.Interpreter(text).run(list(args))]


def test_parser_reads_pretty_and_generic_forms():
    m = ir.parse_module("""
    module @jit_f attributes {mhlo.num_partitions = 1 : i32} {
      func.func public @main(%arg0: tensor<4x8xbf16> {jax.buffer_donor = true}, %arg1: tensor<8xi32>) -> (tensor<4x8xbf16> {jax.result_info = ""}) {
        %c = stablehlo.constant dense<1> : tensor<i32>
        %0 = stablehlo.broadcast_in_dim %c, dims = [] : (tensor<i32>) -> tensor<8xi32>
        %1 = stablehlo.add %arg1, %0 : tensor<8xi32>
        %2:2 = "stablehlo.while"(%c, %arg0) ({
          ^cond(%i: tensor<i32>, %x: tensor<4x8xbf16>):
            %p = stablehlo.compare LT, %i, %c, SIGNED : (tensor<i32>, tensor<i32>) -> tensor<i1>
            stablehlo.return %p : tensor<i1>
        }, {
          ^body(%i: tensor<i32>, %x: tensor<4x8xbf16>):
            stablehlo.return %i, %x : tensor<i32>, tensor<4x8xbf16>
        }) : (tensor<i32>, tensor<4x8xbf16>) -> (tensor<i32>, tensor<4x8xbf16>)
        %3 = func.call @helper(%2#1) : (tensor<4x8xbf16>) -> tensor<4x8xbf16>
        return %3 : tensor<4x8xbf16>
      }
      func.func private @helper(%a: tensor<4x8xbf16>) -> tensor<4x8xbf16> {
        %0 = stablehlo.transpose %a, dims = [1, 0] : (tensor<4x8xbf16>) -> tensor<8x4xbf16>
        %1 = stablehlo.reshape %0 : (tensor<8x4xbf16>) -> tensor<4x8xbf16>
        return %1 : tensor<4x8xbf16>
      }
    }""")
    main = m.main
    assert [str(a.type) for a in main.body.args] == ["tensor<4x8xbf16>", "tensor<8xi32>"]
    assert main.arg_attrs[0] == {"jax.buffer_donor": True}
    wh = next(o for o in main.body.ops if o.name == "stablehlo.while")
    assert len(wh.results) == 2 and len(wh.regions) == 2 and len(wh.regions[1].args) == 2
    add = main.body.ops[2]
    assert add.operands[0] is main.body.args[1] and add in main.body.args[1].uses
    assert m.funcs["helper"].visibility == "private"
    assert sum(1 for _ in ir.walk_blocks(main.body)) == 3


def test_dense_payload_forms():
    ty = ir.parse_type("tensor<2x2xbf16>")
    a = ir.dense_to_np(("dense", "[[1.0, -0.5], [3.140625, 0.0]]", ty), ty)
    np.testing.assert_array_equal(a, np.array([[1.0, -0.5], [3.140625, 0.0]], np.float32))
    assert ir.dense_to_np(("dense", "0xFF80", ir.parse_type("tensor<bf16>")), ir.parse_type("tensor<bf16>")) == -np.inf
    raw = np.arange(4, dtype=np.float32).tobytes().hex().upper()
    t4 = ir.parse_type("tensor<4xf32>")
    np.testing.assert_array_equal(ir.dense_to_np(("dense", f'"0x{raw}"', t4), t4), np.arange(4, dtype=np.float32))
    ti = ir.parse_type("tensor<3xi8>")
    np.testing.assert_array_equal(ir.dense_to_np(("dense", "-7", ti), ti), np.full(3, -7, np.int8))


def test_shift_semantics_follow_xla():
    text = """
    func.func @main(%a: tensor<4xi8>, %s: tensor<4xi8>) -> (tensor<4xi8>, tensor<4xi8>, tensor<4xi8>) {
      %0 = stablehlo.shift_right_arithmetic %a, %s : tensor<4xi8>
      %1 = stablehlo.shift_right_logical %a, %s : tensor<4xi8>
      %2 = stablehlo.shift_left %a, %s : tensor<4xi8>
      return %0, %1, %2 : tensor<4xi8>, tensor<4xi8>, tensor<4xi8>
    }"""
    a = np.array([-16, 120, -1, 5], np.int8)
    s = np.array([4, 4, 9, 1], np.int8)                      # 9 >= the width
    sra, srl, shl = run(text, a, s)
    np.testing.assert_array_equal(sra.a, np.array([-1, 7, -1, 2], np.int8))
    np.testing.assert_array_equal(srl.a, np.array([15, 7, 0, 2], np.int8))
    np.testing.assert_array_equal(shl.a, np.array([0, -128, 0, 10], np.int8))


def test_bf16_arithmetic_rounds_once_per_op():
    text = """
    func.func @main(%a: tensor<2xbf16>, %b: tensor<2xbf16>) -> tensor<2xbf16> {
      %0 = stablehlo.multiply %a, %b : tensor<2xbf16>
      return %0 : tensor<2xbf16>
    }"""
    a = I.from_numpy(np.array([1.0078125, 3.0], np.float32), "bf16")
    b = I.from_numpy(np.array([1.0078125, 0.3333], np.float32), "bf16")
    (y,) = run(text, a, b)
    want = I.round_bf16(a.a * b.a)
    np.testing.assert_array_equal(y.a, want)
    assert y.el == "bf16" and float(y.a[0]) == 1.015625      # 1.01568 rounds to nearest even


def test_gather_take_rows_and_index_clamp():
    text = """
    func.func @main(%t: tensor<4x3xf32>, %i: tensor<5x1xi32>) -> tensor<5x3xf32> {
      %0 = "stablehlo.gather"(%t, %i) <{dimension_numbers = #stablehlo.gather<offset_dims = [1], collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = 1>, slice_sizes = array<i64: 1, 3>}> : (tensor<4x3xf32>, tensor<5x1xi32>) -> tensor<5x3xf32>
      return %0 : tensor<5x3xf32>
    }"""
    t = np.arange(12, dtype=np.float32).reshape(4, 3)
    i = np.array([[0], [3], [9], [-2], [1]], np.int32)        # out of range: clamped
    (y,) = run(text, t, i)
    np.testing.assert_array_equal(y.a, t[[0, 3, 3, 0, 1]])


def test_four_bit_integers_wrap():
    text = """
    func.func @main(%a: tensor<3xi8>) -> tensor<3xi8> {
      %0 = stablehlo.convert %a : (tensor<3xi8>) -> tensor<3xi4>
      %1 = stablehlo.convert %0 : (tensor<3xi4>) -> tensor<3xi8>
      return %1 : tensor<3xi8>
    }"""
    (y,) = run(text, np.array([7, 9, -9], np.int8))
    np.testing.assert_array_equal(y.a, np.array([7, -7, 7], np.int8))


def test_dot_general_literal_path_matches_numpy():
    text = """
    func.func @main(%a: tensor<2x3x4xf32>, %b: tensor<2x5x4xf32>) -> tensor<2x3x5xf32> {
      %0 = stablehlo.dot_general %a, %b, batching_dims = [0] x [0], contracting_dims = [2] x [2] : (tensor<2x3x4xf32>, tensor<2x5x4xf32>) -> tensor<2x3x5xf32>
      return %0 : tensor<2x3x5xf32>
    }"""
    rng = np.random.default_rng(0)
    a, b = rng.standard_normal((2, 3, 4)).astype(np.float32), rng.standard_normal((2, 5, 4)).astype(np.float32)
    (y,) = run(text, a, b)
    np.testing.assert_allclose(y.a, np.einsum("bik,bjk->bij", a, b), rtol=1e-6)


def test_unknown_op_is_reported():
    text = """
    func.func @main(%a: tensor<2xf32>) -> tensor<2xf32> {
      %0 = stablehlo.cosine %a : tensor<2xf32>
      return %0 : tensor<2xf32>
    }"""
    with pytest.raises(I.UnsupportedOp):
        run(text, np.zeros(2, np.float32))


def test_a_kept_host_copy_is_dropped_when_the_tensor_is_written_in_place():
    """The interpreter keeps one host copy per device tensor; a caller that
    refills the tensor between calls (also through a view) must not meet the
    old copy, and a dead tensor's entry goes with it."""
    import gc
    import torch
    t = torch.arange(6, dtype=torch.float32)
    h = I.from_numpy(t.numpy().copy())
    I._mirror_put(t, h)
    assert I._mirror_get(t) is h
    assert I._mirror_get(t.clone()) is None                 # another tensor object, same values
    t.view(2, 3)[1, 1] = 9.0                                # written through a view: the counter is shared
    assert I._mirror_get(t) is None
    I._mirror_put(t, h)
    t.add_(1)
    assert I._mirror_get(t) is None
    I._mirror_put(t, h)
    key = id(t)
    assert key in I._MIRRORS
    del t
    gc.collect()
    assert key not in I._MIRRORS
