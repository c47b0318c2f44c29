"""The elementwise table that a planned expert dispatch runs on device tensors
(moe._dev_elementwise) against the literal interpreter's handlers, op by op,
on torch CPU tensors (the same torch operators as on the GPU): special values,
signed zeros, out-of-range conversions, integer wrap-around.  What the table
does not model must say so (_HostOnly), never answer differently."""

import itertools

import numpy as np
import pytest
import torch

from metaljax_amd import interpreter as I, ir, moe
from metaljax_amd.interpreter import REGISTRY

FLOATS = np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 3.3, -3.3, 1e-3, 88.0, -88.0, 1e20,
                   -1e20, np.inf, -np.inf, np.nan, 65504.0, 7.0, 0.1, 255.9, -129.2, 3e9, -3e9], np.float32)
INTS = np.array([0, 1, -1, 2, -2, 127, -128, 255, 256, 32767, -32768, 65535, 2**31 - 1, -2**31, 12345678, -7],
                np.int64)
ULP = {"f32": 2.0 ** -23, "bf16": 2.0 ** -7, "f16": 2.0 ** -10}
# library functions: torch's and numpy's differ in the last place
TRANSCENDENTAL = {"exponential", "log", "logistic", "tanh", "power", "rsqrt"}
# which of +0 / -0 a minimum or maximum of the two returns is the library's choice
ZERO_SIGN_FREE = {"clamp", "maximum", "minimum"}


def _t(n, el):
    return f"tensor<{n}x{el}>"


def _op(name, els, out_el, n, direction=None):
    params = ", ".join(f"%a{i}: {_t(n, el)}" for i, el in enumerate(els))
    operands = ", ".join(f"%a{i}" for i in range(len(els)))
    sig = "(" + ", ".join(_t(n, el) for el in els) + ") -> " + _t(n, out_el)
    lead = f"{direction}, " if direction else ""
    text = f"""
    func.func @main({params}) -> {_t(n, out_el)} {{
      %0 = stablehlo.{name} {lead}{operands} : {sig}
      return %0 : {_t(n, out_el)}
    }}"""
    mod = ir.parse_module(text)
    return [o for o in mod.main.body.ops if o.name == "stablehlo." + name][0]


def _host_value(el, vals):
    if el in ("bf16", "f16"):
        return I.from_numpy(np.asarray(vals, np.float32), el)
    return I.from_numpy(np.asarray(vals).astype(ir.np_dtype(el)))


def _dev_value(h):
    if h.el == "bf16":
        return moe.DevArray(torch.from_numpy(np.ascontiguousarray(h.a, np.float32)).bfloat16(), "bf16")
    return moe.DevArray(torch.from_numpy(np.ascontiguousarray(h.a)), h.el)


def _both(name, els, out_el, arrays, direction=None):
    """(literal result, device-table result or None when the table declines)."""
    op = _op(name, els, out_el, len(arrays[0]), direction)
    hs = [_host_value(el, a) for el, a in zip(els, arrays)]
    with np.errstate(all="ignore"):
        out = REGISTRY[op.name](None, op, hs, {})
    want = out[0] if isinstance(out, (list, tuple)) else out
    try:
        got = moe._dev_elementwise(op, [_dev_value(h) for h in hs], out_el)
    except moe._HostOnly:
        return want, None
    assert got.dtype == moe._tdtype(out_el), (name, els, out_el, got.dtype)
    return want, I.host(got)


def _assert_same(name, out_el, want, got):
    a, b = np.asarray(want.a), np.asarray(got.a)
    assert a.shape == b.shape and want.el == got.el == out_el
    if a.dtype.kind != "f":
        np.testing.assert_array_equal(b, a, err_msg=name)
        return
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    same = (a64 == b64) | (np.isnan(a64) & np.isnan(b64))
    if name not in ZERO_SIGN_FREE:
        same &= ~((a64 == 0) & (b64 == 0) & (np.signbit(a64) != np.signbit(b64)))
    if name in TRANSCENDENTAL:
        with np.errstate(all="ignore"):
            same |= np.abs(a64 - b64) <= 1.01 * ULP[out_el] * np.abs(a64)
    assert same.all(), (name, out_el, a[~same][:4], b[~same][:4])


@pytest.mark.parametrize("el", ["f32", "bf16", "f16"])
def test_float_ops_mean_what_the_literal_interpreter_means(el):
    pairs = np.array(list(itertools.product(FLOATS, FLOATS)), np.float32)
    for name in ("add", "subtract", "multiply", "divide", "maximum", "minimum", "power"):
        want, got = _both(name, [el, el], el, [pairs[:, 0], pairs[:, 1]])
        assert got is not None, name
        _assert_same(name, el, want, got)
    for name in ("abs", "ceil", "floor", "exponential", "log", "logistic", "negate", "rsqrt", "sqrt", "tanh",
                 "sign", "round_nearest_even"):
        want, got = _both(name, [el], el, [FLOATS])
        assert got is not None, name
        _assert_same(name, el, want, got)
    for direction in ("EQ", "NE", "LT", "LE", "GT", "GE"):
        want, got = _both("compare", [el, el], "i1", [pairs[:, 0], pairs[:, 1]], direction)
        _assert_same("compare", "i1", want, got)
    triples = np.array(list(itertools.product(FLOATS[:20], FLOATS[:20], FLOATS[:20])), np.float32)
    want, got = _both("clamp", [el, el, el], el, [triples[:, 0], triples[:, 1], triples[:, 2]])
    _assert_same("clamp", el, want, got)
    which = (np.arange(len(pairs)) % 2).astype(bool)
    want, got = _both("select", ["i1", el, el], el, [which, pairs[:, 0], pairs[:, 1]])
    _assert_same("select", el, want, got)


@pytest.mark.parametrize("src", ["f32", "bf16", "f16", "i32", "i8", "ui8", "i64", "i16"])
def test_conversions_truncate_saturate_and_map_nan_to_zero_like_the_literal_path(src):
    vals = FLOATS if src in ULP else INTS
    for out in ("i32", "i8", "ui8", "i64", "i16", "i1", "f32", "bf16", "f16"):
        want, got = _both("convert", [src], out, [vals])
        assert got is not None, (src, out)
        _assert_same("convert", out, want, got)


@pytest.mark.parametrize("el", ["i32", "i8", "ui8", "i64", "i16"])
def test_integer_ops_wrap_like_the_literal_path_and_division_is_left_to_it(el):
    pairs = np.array(list(itertools.product(INTS, INTS)), np.int64)
    for name in ("and", "or", "xor", "add", "subtract", "multiply", "maximum", "minimum"):
        want, got = _both(name, [el, el], el, [pairs[:, 0], pairs[:, 1]])
        assert got is not None, name
        _assert_same(name, el, want, got)
    want, got = _both("not", [el], el, [INTS])
    _assert_same("not", el, want, got)
    for name in ("abs", "negate", "sign"):
        want, got = _both(name, [el], el, [INTS])
        if el == "ui8":
            assert got is None                      # left to the host
        else:
            _assert_same(name, el, want, got)
    for direction in ("EQ", "LT", "GE"):
        want, got = _both("compare", [el, el], "i1", [pairs[:, 0], pairs[:, 1]], direction)
        _assert_same("compare", "i1", want, got)
    which = (np.arange(len(pairs)) % 2).astype(bool)
    want, got = _both("select", ["i1", el, el], el, [which, pairs[:, 0], pairs[:, 1]])
    _assert_same("select", el, want, got)
    nonzero = np.where(pairs[:, 1].astype(ir.np_dtype(el)) == 0, 1, pairs[:, 1])
    _, got = _both("divide", [el, el], el, [pairs[:, 0], nonzero])
    assert got is None                              # truncating division, division by zero: the literal path's


def test_every_op_the_planner_calls_elementwise_is_either_modelled_or_declined():
    known = set()
    for name in sorted(moe._ELEMENTWISE):
        short = name[len("stablehlo."):]
        if short in ("compare", "select", "convert", "clamp"):
            known.add(name)
            continue
        arity = 2 if short in ("add", "and", "divide", "maximum", "minimum", "multiply", "or", "power", "subtract",
                               "xor") else 1
        el = "i32" if short in ("and", "or", "xor", "not") else "f32"
        want, got = _both(short, [el] * arity, el, [FLOATS[:6] if el == "f32" else INTS[:6]] * arity)
        assert got is not None, name
        known.add(name)
    assert known == set(moe._ELEMENTWISE)
