"""Hand-written StableHLO modules in the shapes the reference's quantized test
functions lower to (reference tests/test_qmm.py:179-234 `_unpack_nibbles`,
`dense_sub`, `dense_perchannel`; tests/test_qmm_mxfp4.py:268-310
`mxfp4_weight`, `dense_mxfp4`, `experts_mxfp4`), plus the seeded data
generators of those tests restated with numpy alone.  jax is not available
here, so the text is authored by hand: a nibble unpack out of and / shift /
xor / concatenate, a `take` as a gather, a float subtract-and-scale, a dot.
"""

import numpy as np

E2M1 = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0)


def _t(shape, el):
    return "tensor<" + "x".join([*map(str, shape), el]) + ">"


def _unpack_nibbles(k, n):
    """packed i8 [K, N/2] -> signed codes i8 [K, N]: lines defining %w."""
    h = n // 2
    a, b = _t((h, k), "i8"), _t((h, 1, k), "i8")
    return f"""
    %t = stablehlo.transpose %packed, dims = [1, 0] : ({_t((k, h), "i8")}) -> {a}
    %c15 = stablehlo.constant dense<15> : tensor<i8>
    %b15 = stablehlo.broadcast_in_dim %c15, dims = [] : (tensor<i8>) -> {a}
    %c4 = stablehlo.constant dense<4> : tensor<i8>
    %b4 = stablehlo.broadcast_in_dim %c4, dims = [] : (tensor<i8>) -> {a}
    %c8 = stablehlo.constant dense<8> : tensor<i8>
    %b8 = stablehlo.broadcast_in_dim %c8, dims = [] : (tensor<i8>) -> {a}
    %low = stablehlo.and %t, %b15 : {a}
    %sh = stablehlo.shift_right_arithmetic %t, %b4 : {a}
    %high = stablehlo.and %sh, %b15 : {a}
    %lx = stablehlo.xor %low, %b8 : {a}
    %ls = stablehlo.subtract %lx, %b8 : {a}
    %hx = stablehlo.xor %high, %b8 : {a}
    %hs = stablehlo.subtract %hx, %b8 : {a}
    %l3 = stablehlo.reshape %ls : ({a}) -> {b}
    %h3 = stablehlo.reshape %hs : ({a}) -> {b}
    %st = stablehlo.concatenate %l3, %h3, dim = 1 : ({b}, {b}) -> {_t((h, 2, k), "i8")}
    %up = stablehlo.reshape %st : ({_t((h, 2, k), "i8")}) -> {_t((n, k), "i8")}
    %cut = stablehlo.slice %up [0:{n}, 0:{k}] : ({_t((n, k), "i8")}) -> {_t((n, k), "i8")}
    %w = stablehlo.transpose %cut, dims = [1, 0] : ({_t((n, k), "i8")}) -> {_t((k, n), "i8")}"""


def _take_rows(name, table, ng, k, n, el):
    """`jnp.take(table, g, axis=0)` with g [K] int32: negative indices wrap,
    then a gather of whole rows."""
    return f"""
    %{name}_neg = stablehlo.compare LT, %g, %gz, SIGNED : ({_t((k,), "i32")}, {_t((k,), "i32")}) -> {_t((k,), "i1")}
    %{name}_wrap = stablehlo.add %g, %gn : {_t((k,), "i32")}
    %{name}_sel = stablehlo.select %{name}_neg, %{name}_wrap, %g : {_t((k,), "i1")}, {_t((k,), "i32")}
    %{name}_idx = stablehlo.broadcast_in_dim %{name}_sel, dims = [0] : ({_t((k,), "i32")}) -> {_t((k, 1), "i32")}
    %{name} = "stablehlo.gather"(%{table}, %{name}_idx) <{{dimension_numbers = #stablehlo.gather<offset_dims = [1], collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = 1>, indices_are_sorted = false, slice_sizes = array<i64: 1, {n}>}}> : ({_t((ng, n), el)}, {_t((k, 1), "i32")}) -> {_t((k, n), el)}"""


def dense_sub(k, n, ng, m, el="bf16", twice=False):
    """x [M,K] @ ((unpack(packed) - zero[g]) * scale[g]); K rows, N columns.
    `twice` adds a second consumer of the dequantized weight."""
    out = _t((m, n), el)
    extra, ret, res = "", "%y", out
    if twice:
        extra = f"""
    %wsum = stablehlo.reduce(%wq init: %fz) applies stablehlo.add across dimensions = [0] : ({_t((k, n), el)}, tensor<{el}>) -> {_t((n,), el)}"""
        ret, res = "%y, %wsum", f"({out}, {_t((n,), el)})"
    return f"""
module @jit_dense_sub {{
  func.func public @main(%packed: {_t((k, n // 2), "i8")}, %scale: {_t((ng, n), el)}, %zero: {_t((ng, n), "i8")}, %gidx: {_t((k,), "f32")}, %x: {_t((m, k), el)}) -> {res} {{{_unpack_nibbles(k, n)}
    %g = stablehlo.convert %gidx : ({_t((k,), "f32")}) -> {_t((k,), "i32")}
    %gzs = stablehlo.constant dense<0> : tensor<i32>
    %gz = stablehlo.broadcast_in_dim %gzs, dims = [] : (tensor<i32>) -> {_t((k,), "i32")}
    %gns = stablehlo.constant dense<{ng}> : tensor<i32>
    %gn = stablehlo.broadcast_in_dim %gns, dims = [] : (tensor<i32>) -> {_t((k,), "i32")}
    %fz = stablehlo.constant dense<0.000000e+00> : tensor<{el}>{_take_rows("s", "scale", ng, k, n, el)}{_take_rows("z", "zero", ng, k, n, "i8")}
    %wf = stablehlo.convert %w : ({_t((k, n), "i8")}) -> {_t((k, n), el)}
    %zf = stablehlo.convert %z : ({_t((k, n), "i8")}) -> {_t((k, n), el)}
    %d = stablehlo.subtract %wf, %zf : {_t((k, n), el)}
    %wq = stablehlo.multiply %d, %s : {_t((k, n), el)}{extra}
    %y = stablehlo.dot_general %x, %wq, contracting_dims = [1] x [0], precision = [DEFAULT, DEFAULT] : ({_t((m, k), el)}, {_t((k, n), el)}) -> {out}
    return {ret} : {res.strip("()")}
  }}
}}
"""


def _dense_sub_with_dot(k, n, ng, el, x_shape, out_shape, dot_lines):
    """`dense_sub`'s dequantization chain (it defines %wq [K, N]) with another
    activation shape and another tail: `dot_lines` must define %y."""
    text = dense_sub(k, n, ng, 1, el)
    x_old, out_old = _t((1, k), el), _t((1, n), el)
    head, dot, tail = text.partition("    %y = stablehlo.dot_general")
    assert dot
    head = head.replace(f"%x: {x_old}) -> {out_old} {{", f"%x: {_t(x_shape, el)}) -> {_t(out_shape, el)} {{")
    return head + dot_lines + f"\n    return %y : {_t(out_shape, el)}\n  }}\n}}\n"


def einsum_sub(d, heads, head_dim, ng, b, t, el="bf16"):
    """einsum("btd,dnh->btnh", x, reshape(dequant(W), [d, n, h])): the weight
    is reshaped after the chain and N has two axes (the EinsumDense chain of
    reference tests/test_qmm.py:226-236, :329-339)."""
    n = heads * head_dim
    w2, w3 = _t((d, n), el), _t((d, heads, head_dim), el)
    x, out = (b, t, d), (b, t, heads, head_dim)
    return _dense_sub_with_dot(d, n, ng, el, x, out, f"""    %w3 = stablehlo.reshape %wq : ({w2}) -> {w3}
    %y = stablehlo.dot_general %x, %w3, contracting_dims = [2] x [0], precision = [DEFAULT, DEFAULT] : ({_t(x, el)}, {w3}) -> {_t(out, el)}""")


def einsum_out_proj(nh, h, d, ng, b, t, el="bf16"):
    """einsum("btnh,nhd->btd", x, reshape(dequant(W), [n, h, d])) as jax lowers
    it, `contracting_dims = [3, 2] x [1, 0]`: the pairing is reversed, so the
    canonical K axis runs h-major over a weight stored (and grouped) n-major
    (reference tests/test_qmm.py:208-223, :409-418)."""
    rows = nh * h
    w2, w3 = _t((rows, d), el), _t((nh, h, d), el)
    x, out = (b, t, nh, h), (b, t, d)
    return _dense_sub_with_dot(rows, d, ng, el, x, out, f"""    %w3 = stablehlo.reshape %wq : ({w2}) -> {w3}
    %y = stablehlo.dot_general %x, %w3, contracting_dims = [3, 2] x [1, 0], precision = [DEFAULT, DEFAULT] : ({_t(x, el)}, {w3}) -> {_t(out, el)}""")


def dense_i8_codes(k, n, ng, m, el="bf16"):
    """dense_sub with the codes stored as plain i8 [K, N] (no nibble unpack)."""
    text = dense_sub(k, n, ng, m, el)
    head = text[:text.index("{", text.index("@main")) + 1].replace(_t((k, n // 2), "i8"), _t((k, n), "i8")).replace("%packed", "%w")
    tail = text[text.index("    %g = stablehlo.convert %gidx"):]
    return head + "\n" + tail


def dense_int_sub(k, n, ng, m, el="bf16"):
    """The same product with the zero point subtracted in INTEGER (i8)
    arithmetic before the convert: the form that can wrap."""
    return f"""
func.func public @main(%packed: {_t((k, n // 2), "i8")}, %scale: {_t((ng, n), el)}, %zero: {_t((ng, n), "i8")}, %gidx: {_t((k,), "f32")}, %x: {_t((m, k), el)}) -> {_t((m, n), el)} {{{_unpack_nibbles(k, n)}
  %g = stablehlo.convert %gidx : ({_t((k,), "f32")}) -> {_t((k,), "i32")}
  %gzs = stablehlo.constant dense<0> : tensor<i32>
  %gz = stablehlo.broadcast_in_dim %gzs, dims = [] : (tensor<i32>) -> {_t((k,), "i32")}
  %gns = stablehlo.constant dense<{ng}> : tensor<i32>
  %gn = stablehlo.broadcast_in_dim %gns, dims = [] : (tensor<i32>) -> {_t((k,), "i32")}{_take_rows("s", "scale", ng, k, n, el)}{_take_rows("z", "zero", ng, k, n, "i8")}
  %di = stablehlo.subtract %w, %z : {_t((k, n), "i8")}
  %d = stablehlo.convert %di : ({_t((k, n), "i8")}) -> {_t((k, n), el)}
  %wq = stablehlo.multiply %d, %s : {_t((k, n), el)}
  %y = stablehlo.dot_general %x, %wq, contracting_dims = [1] x [0] : ({_t((m, k), el)}, {_t((k, n), el)}) -> {_t((m, n), el)}
  return %y : {_t((m, n), el)}
}}
"""


def dense_perchannel(k, n, m, el="bf16"):
    """(x @ convert(codes)) / scale[N]."""
    return f"""
func.func public @main(%packed: {_t((k, n // 2), "i8")}, %scale: {_t((n,), el)}, %x: {_t((m, k), el)}) -> {_t((m, n), el)} {{{_unpack_nibbles(k, n)}
  %wf = stablehlo.convert %w : ({_t((k, n), "i8")}) -> {_t((k, n), el)}
  %y0 = stablehlo.dot_general %x, %wf, contracting_dims = [1] x [0] : ({_t((m, k), el)}, {_t((k, n), el)}) -> {_t((m, n), el)}
  %sb = stablehlo.broadcast_in_dim %scale, dims = [1] : ({_t((n,), el)}) -> {_t((m, n), el)}
  %y = stablehlo.divide %y0, %sb : {_t((m, n), el)}
  return %y : {_t((m, n), el)}
}}
"""


def dense_i4_perchannel(k, n, m, el="bf16"):
    """x [M,K] @ (convert(w : i4 [K,N]) * scale[N]): weights stored as four-bit
    integers with one scale per output channel (the chain of reference
    tests/test_qmm.py:342-358)."""
    return f"""
module @jit_i4 {{
  func.func public @main(%w: {_t((k, n), "i4")}, %s: {_t((n,), el)}, %x: {_t((m, k), el)}) -> {_t((m, n), el)} {{
    %wf = stablehlo.convert %w : ({_t((k, n), "i4")}) -> {_t((k, n), el)}
    %sb = stablehlo.broadcast_in_dim %s, dims = [1] : ({_t((n,), el)}) -> {_t((k, n), el)}
    %wq = stablehlo.multiply %wf, %sb : {_t((k, n), el)}
    %y = stablehlo.dot_general %x, %wq, contracting_dims = [1] x [0], precision = [DEFAULT, DEFAULT] : ({_t((m, k), el)}, {_t((k, n), el)}) -> {_t((m, n), el)}
    return %y : {_t((m, n), el)}
  }}
}}
"""


def _e8m0_table_hex():
    with np.errstate(over="ignore"):
        t = np.ldexp(np.ones(256), np.arange(256) - 127).astype(np.float32)
    t[255] = np.nan
    return "0x" + t.tobytes().hex().upper()


def _mxfp4_weight(lead, n, k, el, vtable=None):
    """blocks ui8 [lead.., N, K/2] + E8M0 bytes [lead.., N, K/32] -> %wt [lead.., N, K]."""
    L = tuple(lead)
    vt = (list(E2M1) + [-v for v in E2M1]) if vtable is None else list(vtable)
    vals = ", ".join(("-" if np.signbit(v) else "") + f"{abs(v):.6e}" for v in np.array(vt, np.float64))
    cnt = int(np.prod(L + (n, k)))
    sc = int(np.prod(L + (n, k // 32)))
    bl, sb = _t(L + (n, k // 2), "ui8"), _t(L + (n, k // 32), "ui8")
    r = len(L)
    return f"""
    %vt = stablehlo.constant dense<[{vals}]> : tensor<16x{el}>
    %stab = stablehlo.constant dense<"{_e8m0_table_hex()}"> : tensor<256xf32>
    %m15s = stablehlo.constant dense<15> : tensor<ui8>
    %m15 = stablehlo.broadcast_in_dim %m15s, dims = [] : (tensor<ui8>) -> {bl}
    %s4s = stablehlo.constant dense<4> : tensor<ui8>
    %s4 = stablehlo.broadcast_in_dim %s4s, dims = [] : (tensor<ui8>) -> {bl}
    %lo = stablehlo.and %blocks, %m15 : {bl}
    %hi = stablehlo.shift_right_logical %blocks, %s4 : {bl}
    %lo3 = stablehlo.reshape %lo : ({bl}) -> {_t(L + (n, k // 2, 1), "ui8")}
    %hi3 = stablehlo.reshape %hi : ({bl}) -> {_t(L + (n, k // 2, 1), "ui8")}
    %nb = stablehlo.concatenate %lo3, %hi3, dim = {r + 2} : ({_t(L + (n, k // 2, 1), "ui8")}, {_t(L + (n, k // 2, 1), "ui8")}) -> {_t(L + (n, k // 2, 2), "ui8")}
    %nib = stablehlo.reshape %nb : ({_t(L + (n, k // 2, 2), "ui8")}) -> {_t((cnt, 1), "ui8")}
    %ni = stablehlo.convert %nib : ({_t((cnt, 1), "ui8")}) -> {_t((cnt, 1), "i32")}
    %vflat = "stablehlo.gather"(%vt, %ni) <{{dimension_numbers = #stablehlo.gather<collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = 1>, slice_sizes = array<i64: 1>}}> : (tensor<16x{el}>, {_t((cnt, 1), "i32")}) -> {_t((cnt,), el)}
    %sbi0 = stablehlo.reshape %scales : ({sb}) -> {_t((sc, 1), "ui8")}
    %sbi = stablehlo.convert %sbi0 : ({_t((sc, 1), "ui8")}) -> {_t((sc, 1), "i32")}
    %sflat = "stablehlo.gather"(%stab, %sbi) <{{dimension_numbers = #stablehlo.gather<collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = 1>, slice_sizes = array<i64: 1>}}> : (tensor<256xf32>, {_t((sc, 1), "i32")}) -> {_t((sc,), "f32")}
    %sc32 = stablehlo.reshape %sflat : ({_t((sc,), "f32")}) -> {_t(L + (n, k // 32), "f32")}
    %scd = stablehlo.convert %sc32 : ({_t(L + (n, k // 32), "f32")}) -> {_t(L + (n, k // 32), el)}
    %scb = stablehlo.broadcast_in_dim %scd, dims = [{", ".join(map(str, range(r + 2)))}] : ({_t(L + (n, k // 32), el)}) -> {_t(L + (n, k // 32, 32), el)}
    %v3 = stablehlo.reshape %vflat : ({_t((cnt,), el)}) -> {_t(L + (n, k // 32, 32), el)}
    %w3 = stablehlo.multiply %v3, %scb : {_t(L + (n, k // 32, 32), el)}
    %wt = stablehlo.reshape %w3 : ({_t(L + (n, k // 32, 32), el)}) -> {_t(L + (n, k), el)}"""


def dense_mxfp4(n, k, t, el="bf16", vtable=None):
    """`th,nh->tn` over an in-graph MXFP4 reconstruction."""
    return f"""
module @jit_dense_mxfp4 {{
  func.func public @main(%blocks: {_t((n, k // 2), "ui8")}, %scales: {_t((n, k // 32), "ui8")}, %x: {_t((t, k), el)}) -> {_t((t, n), el)} {{{_mxfp4_weight((), n, k, el, vtable)}
    %y = stablehlo.dot_general %x, %wt, contracting_dims = [1] x [1] : ({_t((t, k), el)}, {_t((n, k), el)}) -> {_t((t, n), el)}
    return %y : {_t((t, n), el)}
  }}
}}
"""


def experts_mxfp4(e, n, k, t, el="bf16"):
    """`etm,ehm->eth`: one weight per expert, a BATCHED dot."""
    return f"""
func.func public @main(%blocks: {_t((e, n, k // 2), "ui8")}, %scales: {_t((e, n, k // 32), "ui8")}, %x: {_t((e, t, k), el)}) -> {_t((e, t, n), el)} {{{_mxfp4_weight((e,), n, k, el)}
  %y = stablehlo.dot_general %x, %wt, batching_dims = [0] x [0], contracting_dims = [2] x [2] : ({_t((e, t, k), el)}, {_t((e, n, k), el)}) -> {_t((e, t, n), el)}
  return %y : {_t((e, t, n), el)}
}}
"""


def float_dot(k, n, m, el="bf16"):
    """An ordinary float projection with a per-row scale: nothing to recognize."""
    return f"""
func.func public @main(%w: {_t((k, n), el)}, %r: {_t((k,), el)}, %x: {_t((m, k), el)}) -> {_t((m, n), el)} {{
  %rb = stablehlo.broadcast_in_dim %r, dims = [0] : ({_t((k,), el)}) -> {_t((k, n), el)}
  %ws = stablehlo.multiply %w, %rb : {_t((k, n), el)}
  %y = stablehlo.dot_general %x, %ws, contracting_dims = [1] x [0] : ({_t((m, k), el)}, {_t((k, n), el)}) -> {_t((m, n), el)}
  return %y : {_t((m, n), el)}
}}
"""


def decode_loop(k, ng, m, steps, el="bf16"):
    """A while loop whose weights arrive as carries returned unchanged (how jax
    lowers a loop's closed-over constants); the body is one dense_sub with
    N == K so the result feeds the next step."""
    n = k
    pk, sc, zr, gi, xx = (_t((k, n // 2), "i8"), _t((ng, n), el), _t((ng, n), "i8"),
                          _t((k,), "f32"), _t((m, k), el))
    body = dense_sub(k, n, ng, m, el)
    lines = body[body.index("{", body.index("@main")) + 1:body.rindex("%y = stablehlo.dot_general")]
    lines = (lines.replace("%packed", "%cp").replace("%scale,", "%cs,").replace("(%scale", "(%cs")
             .replace("%zero,", "%cz,").replace("(%zero", "(%cz").replace("%gidx", "%cg"))
    return f"""
func.func public @main(%packed: {pk}, %scale: {sc}, %zero: {zr}, %gidx: {gi}, %x0: {xx}) -> {xx} {{
  %i0 = stablehlo.constant dense<0> : tensor<i32>
  %r:6 = stablehlo.while(%i = %i0, %cx = %x0, %cp = %packed, %cs = %scale, %cz = %zero, %cg = %gidx) : tensor<i32>, {xx}, {pk}, {sc}, {zr}, {gi}
   cond {{
    %lim = stablehlo.constant dense<{steps}> : tensor<i32>
    %p = stablehlo.compare LT, %i, %lim, SIGNED : (tensor<i32>, tensor<i32>) -> tensor<i1>
    stablehlo.return %p : tensor<i1>
  }} do {{{lines}
    %y = stablehlo.dot_general %cx, %wq, contracting_dims = [1] x [0] : ({xx}, {_t((k, n), el)}) -> {xx}
    %one = stablehlo.constant dense<1> : tensor<i32>
    %ni = stablehlo.add %i, %one : tensor<i32>
    stablehlo.return %ni, %y, %cp, %cs, %cz, %cg : tensor<i32>, {xx}, {pk}, {sc}, {zr}, {gi}
  }}
  return %r#1 : {xx}
}}
"""


# ------------------------------------------------------------ seeded data ----

def bf16_round(x):
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32) << 16
    return r.view(np.float32).reshape(np.shape(x))


def quantize(rows, cols, block, seed=0, bits=4, g_idx=None, bf16=True):
    """Codes + scale/zero maps in the keras storage layout: the generator of
    reference tests/test_qmm.py:237-252 (same draws, same order)."""
    rng = np.random.default_rng(seed)
    lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
    q = rng.integers(lo, hi + 1, size=(rows, cols)).astype(np.int8)
    bsz = rows if block < 0 else block
    ng = rows // bsz
    scale = ((rng.random((ng, cols)).astype(np.float32) + 0.5) * 0.05)
    zero = (np.zeros((ng, cols), np.int8) if block < 0 else
            rng.integers(-3, 4, size=(ng, cols)).astype(np.int8))
    if g_idx is None:
        g_idx = (np.arange(rows) // bsz).astype(np.float32)
    packed = ((q[:, 0::2] & 0x0F) | (q[:, 1::2] << 4)).astype(np.int8)
    if bf16:
        scale = bf16_round(scale)
    gi = g_idx.astype(np.int32)
    ref = scale[gi] * (q.astype(np.float32) - zero[gi].astype(np.float32))
    return q, packed, scale, zero, g_idx, ref


def random_mxfp4(shape_nk, seed=0, lo=117, hi=127):
    """blocks ui8 [.., N, K/2], E8M0 bytes [.., N, K/32] and the exact float32
    weight (reference tests/test_qmm_mxfp4.py:100-108)."""
    rng = np.random.default_rng(seed)
    *lead, n, k = shape_nk
    codes = rng.integers(0, 16, size=(*lead, n, k), dtype=np.uint8)
    blocks = (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)
    sb = rng.integers(lo, hi + 1, size=(*lead, n, k // 32), dtype=np.uint8)
    grid = np.array(list(E2M1) + [-v for v in E2M1], np.float32)
    w = grid[codes] * np.repeat(np.ldexp(np.float32(1), sb.astype(np.int32) - 127), 32, axis=-1)
    return codes, blocks, sb, w.astype(np.float32)


# ---------------------------------------------- weights stored rows-first ----

def affine_grouped(n, k, gs, t, interleave=False, el="bf16"):
    """`tk,nk->tn` over a sub-channel weight whose group axis is split out of K
    (what a packed checkpoint stores; reference tests/test_qmm.py:991-1027):
    codes i8 [N, K] viewed as [N, K/gs, gs] -- or, interleaved, [N, gs, K/gs],
    which scatters each group's columns across K at stride K/gs -- one scale /
    zero pair per group broadcast over the group, reshaped back to [N, K].
    The contraction runs over the LAST axis, so the weight can be packed by
    blocks of rows."""
    ng = k // gs
    split = (n, gs, ng) if interleave else (n, ng, gs)
    where = "[0, 2]" if interleave else "[0, 1]"
    s3, q3 = _t(split, el), _t(split, "i8")
    return f"""
module @jit_affine_grouped {{
  func.func public @main(%q: {_t((n, k), "i8")}, %scale: {_t((n, ng), "f32")}, %zero: {_t((n, ng), "i8")}, %x: {_t((t, k), el)}) -> {_t((t, n), el)} {{
    %qs = stablehlo.reshape %q : ({_t((n, k), "i8")}) -> {q3}
    %qf = stablehlo.convert %qs : ({q3}) -> {s3}
    %sc = stablehlo.convert %scale : ({_t((n, ng), "f32")}) -> {_t((n, ng), el)}
    %sb = stablehlo.broadcast_in_dim %sc, dims = {where} : ({_t((n, ng), el)}) -> {s3}
    %zc = stablehlo.convert %zero : ({_t((n, ng), "i8")}) -> {_t((n, ng), el)}
    %zb = stablehlo.broadcast_in_dim %zc, dims = {where} : ({_t((n, ng), el)}) -> {s3}
    %d = stablehlo.subtract %qf, %zb : {s3}
    %w3 = stablehlo.multiply %d, %sb : {s3}
    %w = stablehlo.reshape %w3 : ({s3}) -> {_t((n, k), el)}
    %y = stablehlo.dot_general %x, %w, contracting_dims = [1] x [1] : ({_t((t, k), el)}, {_t((n, k), el)}) -> {_t((t, n), el)}
    return %y : {_t((t, n), el)}
  }}
}}
"""


def affine_grouped_data(n, k, gs, seed, interleave=False):
    """Seeded codes / scales / zero points of `affine_grouped` and the exact
    float32 weight (reference tests/test_qmm.py:991-1010: same draws)."""
    rng = np.random.default_rng(seed)
    ng = k // gs
    q = rng.integers(-8, 8, size=(n, k)).astype(np.int8)
    scale = ((rng.random((n, ng)).astype(np.float32) + 0.5) * 0.05)
    zero = rng.integers(-3, 4, size=(n, ng)).astype(np.int8)
    g = (np.arange(k) % ng) if interleave else (np.arange(k) // gs)
    ref = np.take(scale, g, axis=1) * (q.astype(np.float32) - np.take(zero, g, axis=1))
    return q, scale, zero, ref


def dense_mxfp4_rows(n, k, t, el="bf16", e=None):
    """dense_mxfp4 as jax lowers `jnp.take`: the E2M1 decode is a private
    @_take callee (index wrap with full-extent splats, then a gather that
    batches over the indices), and every op keeps the weight's leading axis
    leading (reference tests/test_qmm_mxfp4.py:282-298, :908-916).  With `e`
    the weight is [E, N, K] and the product batches over the experts."""
    h = k // 2
    L = () if e is None else (e,)
    r = len(L)                                    # axes in front of N
    vals = ", ".join(("-" if np.signbit(v) else "") + f"{abs(v):.6e}"
                     for v in np.array(list(E2M1) + [-v for v in E2M1], np.float64))
    bl, sb = _t(L + (n, h), "ui8"), _t(L + (n, k // 32), "ui8")
    idx, idx3 = _t(L + (n, k), "i32"), _t(L + (n, k, 1), "i32")
    dims = ", ".join(str(i) for i in range(r + 2))
    if e is None:
        xs, ys = (t, k), (t, n)
        dot = f"contracting_dims = [1] x [1]"
    else:
        xs, ys = (e, t, k), (e, t, n)
        dot = f"batching_dims = [0] x [0], contracting_dims = [2] x [2]"
    return f"""
module @jit_dense_mxfp4_rows {{
  func.func public @main(%blocks: {bl}, %scales: {sb}, %x: {_t(xs, el)}) -> {_t(ys, el)} {{
    %vt = stablehlo.constant dense<[{vals}]> : tensor<16x{el}>
    %stab = stablehlo.constant dense<"{_e8m0_table_hex()}"> : tensor<256xf32>
    %m15s = stablehlo.constant dense<15> : tensor<ui8>
    %m15 = stablehlo.broadcast_in_dim %m15s, dims = [] : (tensor<ui8>) -> {bl}
    %s4s = stablehlo.constant dense<4> : tensor<ui8>
    %s4 = stablehlo.broadcast_in_dim %s4s, dims = [] : (tensor<ui8>) -> {bl}
    %lo = stablehlo.and %blocks, %m15 : {bl}
    %hi = stablehlo.shift_right_logical %blocks, %s4 : {bl}
    %lo3 = stablehlo.reshape %lo : ({bl}) -> {_t(L + (n, h, 1), "ui8")}
    %hi3 = stablehlo.reshape %hi : ({bl}) -> {_t(L + (n, h, 1), "ui8")}
    %nb = stablehlo.concatenate %lo3, %hi3, dim = {r + 2} : ({_t(L + (n, h, 1), "ui8")}, {_t(L + (n, h, 1), "ui8")}) -> {_t(L + (n, h, 2), "ui8")}
    %nib = stablehlo.reshape %nb : ({_t(L + (n, h, 2), "ui8")}) -> {_t(L + (n, k), "ui8")}
    %ni = stablehlo.convert %nib : ({_t(L + (n, k), "ui8")}) -> {idx}
    %v = func.call @_take(%vt, %ni) : (tensor<16x{el}>, {idx}) -> {_t(L + (n, k), el)}
    %sbi0 = stablehlo.convert %scales : ({sb}) -> {_t(L + (n, k // 32), "i32")}
    %sbi = stablehlo.reshape %sbi0 : ({_t(L + (n, k // 32), "i32")}) -> {_t(L + (n, k // 32, 1), "i32")}
    %s32 = "stablehlo.gather"(%stab, %sbi) <{{dimension_numbers = #stablehlo.gather<collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = {r + 2}>, slice_sizes = array<i64: 1>}}> : (tensor<256xf32>, {_t(L + (n, k // 32, 1), "i32")}) -> {_t(L + (n, k // 32), "f32")}
    %scd = stablehlo.convert %s32 : ({_t(L + (n, k // 32), "f32")}) -> {_t(L + (n, k // 32), el)}
    %scb = stablehlo.broadcast_in_dim %scd, dims = [{dims}] : ({_t(L + (n, k // 32), el)}) -> {_t(L + (n, k // 32, 32), el)}
    %v3 = stablehlo.reshape %v : ({_t(L + (n, k), el)}) -> {_t(L + (n, k // 32, 32), el)}
    %w3 = stablehlo.multiply %v3, %scb : {_t(L + (n, k // 32, 32), el)}
    %wt = stablehlo.reshape %w3 : ({_t(L + (n, k // 32, 32), el)}) -> {_t(L + (n, k), el)}
    %y = stablehlo.dot_general %x, %wt, {dot} : ({_t(xs, el)}, {_t(L + (n, k), el)}) -> {_t(ys, el)}
    return %y : {_t(ys, el)}
  }}
  func.func private @_take(%table: tensor<16x{el}>, %i: {idx}) -> {_t(L + (n, k), el)} {{
    %zs = stablehlo.constant dense<0> : tensor<i32>
    %z = stablehlo.broadcast_in_dim %zs, dims = [] : (tensor<i32>) -> {idx}
    %ns = stablehlo.constant dense<16> : tensor<i32>
    %nn = stablehlo.broadcast_in_dim %ns, dims = [] : (tensor<i32>) -> {idx}
    %neg = stablehlo.compare LT, %i, %z, SIGNED : ({idx}, {idx}) -> {_t(L + (n, k), "i1")}
    %wrap = stablehlo.add %i, %nn : {idx}
    %sel = stablehlo.select %neg, %wrap, %i : {_t(L + (n, k), "i1")}, {idx}
    %i3 = stablehlo.reshape %sel : ({idx}) -> {idx3}
    %r = "stablehlo.gather"(%table, %i3) <{{dimension_numbers = #stablehlo.gather<collapsed_slice_dims = [0], start_index_map = [0], index_vector_dim = {r + 2}>, slice_sizes = array<i64: 1>}}> : (tensor<16x{el}>, {idx3}) -> {_t(L + (n, k), el)}
    return %r : {_t(L + (n, k), el)}
  }}
}}
"""


# ------------------------------------------------- a dense MoE dispatch ----

def _tagged_mxfp4_weight(tag, blocks, scales, lead, n, k, el):
    """`_mxfp4_weight` with every SSA name suffixed by `tag` and the two
    inputs named `blocks` / `scales`: defines %wt<tag> [lead.., N, K]."""
    import re
    text = _mxfp4_weight(lead, n, k, el)
    text = text.replace("%blocks", "%BLOCKS").replace("%scales", "%SCALES")
    text = re.sub(r"%([a-z][a-z0-9]*)\b", lambda mo: f"%{mo.group(1)}{tag}", text)
    return text.replace("%BLOCKS", blocks).replace("%SCALES", scales)


def moe_block_mxfp4(E, T, H, I, K, el="f32", composite=False):
    """The gpt-oss expert block as the reference's test writes it (reference
    tests/test_moe.py:60-66, :500-511): every expert runs on every token,

        gu   = einsum("th,emh->etm", x, Wgu) + bgu        Wgu MXFP4 [E, 2I, H]
        act  = (clip(up) + 1) * (g * sigmoid(1.702 g)),   g = clip(gate); gate / up = gu[..., 0::2] / [..., 1::2]
        y    = einsum("etm,ehm->eth", act, Wd) + bd       Wd MXFP4 [E, H, I]
        out  = sum_e y[e] * S[:, e],  S = sum_k one_hot(idx) * softmax(top_k values)

    `composite`: the top-k as a stablehlo.composite (what reaches a plugin)."""
    f = el
    tk = ((f'%tk:2 = stablehlo.composite "chlo.top_k" %logits {{composite_attributes = {{k = {K} : i64}}, '
           f'decomposition = @chlo.top_k.impl, version = 1 : i32}} : ({_t((T, E), f)}) -> '
           f'({_t((T, K), f)}, {_t((T, K), "i32")})\n    %vals = stablehlo.convert %tk#0 : ({_t((T, K), f)}) -> {_t((T, K), f)}\n'
           f'    %idx = stablehlo.convert %tk#1 : ({_t((T, K), "i32")}) -> {_t((T, K), "i32")}')
          if composite else
          f'%vals, %idx = chlo.top_k(%logits, k = {K}) : {_t((T, E), f)} -> ({_t((T, K), f)}, {_t((T, K), "i32")})')
    etm, eti, eth = _t((E, T, 2 * I), f), _t((E, T, I), f), _t((E, T, H), f)
    tke = (T, K, E)
    return f"""
module @jit_moe_block {{
  func.func public @main(%x: {_t((T, H), f)}, %wr: {_t((H, E), f)}, %br: {_t((E,), f)}, %guc: {_t((E, 2 * I, H // 2), "ui8")}, %gus: {_t((E, 2 * I, H // 32), "ui8")}, %dc: {_t((E, H, I // 2), "ui8")}, %ds: {_t((E, H, I // 32), "ui8")}, %bgu: {_t((E, 2 * I), f)}, %bd: {_t((E, H), f)}) -> {_t((T, H), f)} {{{_tagged_mxfp4_weight("g", "%guc", "%gus", (E,), 2 * I, H, f)}{_tagged_mxfp4_weight("d", "%dc", "%ds", (E,), H, I, f)}
    %zero = stablehlo.constant dense<0.000000e+00> : tensor<{f}>
    %ninf = stablehlo.constant dense<0xFF800000> : tensor<f32>
    %gu0 = stablehlo.dot_general %x, %wtg, contracting_dims = [1] x [2] : ({_t((T, H), f)}, {_t((E, 2 * I, H), f)}) -> {_t((T, E, 2 * I), f)}
    %gu1 = stablehlo.transpose %gu0, dims = [1, 0, 2] : ({_t((T, E, 2 * I), f)}) -> {etm}
    %bgub = stablehlo.broadcast_in_dim %bgu, dims = [0, 2] : ({_t((E, 2 * I), f)}) -> {etm}
    %gu = stablehlo.add %gu1, %bgub : {etm}
    %gate0 = stablehlo.slice %gu [0:{E}, 0:{T}, 0:{2 * I}:2] : ({etm}) -> {eti}
    %up0 = stablehlo.slice %gu [0:{E}, 0:{T}, 1:{2 * I}:2] : ({etm}) -> {eti}
    %big = stablehlo.constant dense<-1.000000e+09> : tensor<{f}>
    %p7 = stablehlo.constant dense<7.000000e+00> : tensor<{f}>
    %m7 = stablehlo.constant dense<-7.000000e+00> : tensor<{f}>
    %gate = stablehlo.clamp %big, %gate0, %p7 : (tensor<{f}>, {eti}, tensor<{f}>) -> {eti}
    %up = stablehlo.clamp %m7, %up0, %p7 : (tensor<{f}>, {eti}, tensor<{f}>) -> {eti}
    %c17s = stablehlo.constant dense<1.702000e+00> : tensor<{f}>
    %c17 = stablehlo.broadcast_in_dim %c17s, dims = [] : (tensor<{f}>) -> {eti}
    %ones = stablehlo.constant dense<1.000000e+00> : tensor<{f}>
    %one = stablehlo.broadcast_in_dim %ones, dims = [] : (tensor<{f}>) -> {eti}
    %ga = stablehlo.multiply %gate, %c17 : {eti}
    %sg = stablehlo.logistic %ga : {eti}
    %glu = stablehlo.multiply %gate, %sg : {eti}
    %up1 = stablehlo.add %up, %one : {eti}
    %act = stablehlo.multiply %up1, %glu : {eti}
    %y0 = stablehlo.dot_general %act, %wtd, batching_dims = [0] x [0], contracting_dims = [2] x [2] : ({eti}, {_t((E, H, I), f)}) -> {eth}
    %bdb = stablehlo.broadcast_in_dim %bd, dims = [0, 2] : ({_t((E, H), f)}) -> {eth}
    %y = stablehlo.add %y0, %bdb : {eth}
    %lg = stablehlo.dot_general %x, %wr, contracting_dims = [1] x [0] : ({_t((T, H), f)}, {_t((H, E), f)}) -> {_t((T, E), f)}
    %brb = stablehlo.broadcast_in_dim %br, dims = [1] : ({_t((E,), f)}) -> {_t((T, E), f)}
    %logits = stablehlo.add %lg, %brb : {_t((T, E), f)}
    {tk}
    %v32 = stablehlo.convert %vals : ({_t((T, K), f)}) -> {_t((T, K), "f32")}
    %mx = stablehlo.reduce(%v32 init: %ninf) applies stablehlo.maximum across dimensions = [1] : ({_t((T, K), "f32")}, tensor<f32>) -> {_t((T,), "f32")}
    %mxb = stablehlo.broadcast_in_dim %mx, dims = [0] : ({_t((T,), "f32")}) -> {_t((T, K), "f32")}
    %sh = stablehlo.subtract %v32, %mxb : {_t((T, K), "f32")}
    %ex = stablehlo.exponential %sh : {_t((T, K), "f32")}
    %z32 = stablehlo.constant dense<0.000000e+00> : tensor<f32>
    %sm = stablehlo.reduce(%ex init: %z32) applies stablehlo.add across dimensions = [1] : ({_t((T, K), "f32")}, tensor<f32>) -> {_t((T,), "f32")}
    %smb = stablehlo.broadcast_in_dim %sm, dims = [0] : ({_t((T,), "f32")}) -> {_t((T, K), "f32")}
    %w32 = stablehlo.divide %ex, %smb : {_t((T, K), "f32")}
    %w = stablehlo.convert %w32 : ({_t((T, K), "f32")}) -> {_t((T, K), f)}
    %idxb = stablehlo.broadcast_in_dim %idx, dims = [0, 1] : ({_t((T, K), "i32")}) -> {_t(tke, "i32")}
    %io = stablehlo.iota dim = 2 : {_t(tke, "i32")}
    %eq = stablehlo.compare EQ, %idxb, %io, SIGNED : ({_t(tke, "i32")}, {_t(tke, "i32")}) -> {_t(tke, "i1")}
    %hot = stablehlo.convert %eq : ({_t(tke, "i1")}) -> {_t(tke, f)}
    %wb = stablehlo.broadcast_in_dim %w, dims = [0, 1] : ({_t((T, K), f)}) -> {_t(tke, f)}
    %hw = stablehlo.multiply %hot, %wb : {_t(tke, f)}
    %s = stablehlo.reduce(%hw init: %zero) applies stablehlo.add across dimensions = [1] : ({_t(tke, f)}, tensor<{f}>) -> {_t((T, E), f)}
    %st = stablehlo.transpose %s, dims = [1, 0] : ({_t((T, E), f)}) -> {_t((E, T), f)}
    %sb = stablehlo.broadcast_in_dim %st, dims = [0, 1] : ({_t((E, T), f)}) -> {eth}
    %ys = stablehlo.multiply %y, %sb : {eth}
    %out = stablehlo.reduce(%ys init: %zero) applies stablehlo.add across dimensions = [0] : ({eth}, tensor<{f}>) -> {_t((T, H), f)}
    return %out : {_t((T, H), f)}
  }}
}}
"""


def make_mxfp4_experts(rows, k, E, seed):
    """([E, rows, k/2] packed codes, [E, rows, k/32] E8M0 bytes, the exact
    float32 weight) -- the generator of reference tests/test_moe.py:487-497."""
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=(E, rows, k)).astype(np.uint8)
    exps = rng.integers(120, 128, size=(E, rows, k // 32)).astype(np.uint8)
    packed = (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)
    grid = np.array(list(E2M1) + [-v for v in E2M1], np.float32)
    scale = np.exp2(exps.astype(np.float32) - 127.0)
    ref = (grid[codes].reshape(E, rows, k // 32, 32) * scale[..., None]).reshape(E, rows, k)
    return packed, exps, ref.astype(np.float32)


def moe_block_reference(x, wr, br, gu_ref, d_ref, bgu, bd, k):
    """The block on exactly dequantized weights, in float64 numpy."""
    x, wr, br, bgu, bd = (np.asarray(a, np.float64) for a in (x, wr, br, bgu, bd))
    gu = np.einsum("th,emh->etm", x, gu_ref.astype(np.float64)) + bgu[:, None, :]
    gate = np.clip(gu[..., ::2], -1e9, 7.0)
    up = np.clip(gu[..., 1::2], -7.0, 7.0)
    act = (up + 1) * (gate / (1.0 + np.exp(-1.702 * gate)))
    y = np.einsum("etm,ehm->eth", act, d_ref.astype(np.float64)) + bd[:, None, :]
    logits = (x @ wr + br).astype(np.float32)
    order = np.argsort(-logits, axis=-1, kind="stable")[:, :k]
    vals = np.take_along_axis(logits, order, -1).astype(np.float64)
    w = np.exp(vals - vals.max(-1, keepdims=True))
    w /= w.sum(-1, keepdims=True)
    s = np.zeros_like(logits, dtype=np.float64)
    np.put_along_axis(s, order, w, -1)
    return np.einsum("eth,te->th", y, s)


def moe_block_gemma4_mxfp4(E, T, H, I, K, el="f32"):
    """keras-hub's Gemma4 router and expert block as the reference's test
    writes them (reference tests/test_moe.py:192-240), the three expert
    weights as MXFP4 checkpoints:

        probs = softmax((x * rsqrt(mean(x^2) + 1e-6) * H^-0.5 * per_dim) @ proj)
        vals, idx = top_k(probs);  w = vals / max(sum(vals), 1e-9);  S = sum_k one_hot(idx) * w
        y = einsum("eti,ehi->eth", gelu_tanh(x.Wg^T) * (x.Wu^T), Wd) * escale[:, None, None]
        out = sum_e y[e] * S[:, e]

    What sets it apart from the gpt-oss block: three products, separate gate
    and up weights, and a per-expert OUTPUT SCALE [E] reshaped to [E, 1, 1]
    and broadcast over [E, T, H] -- at T = 1 the token axis it is broadcast
    along is a unit axis on both sides."""
    f = el
    th, te, tk_, tke = _t((T, H), f), _t((T, E), f), _t((T, K), f), (T, K, E)
    eti, eth, tei = _t((E, T, I), f), _t((E, T, H), f), _t((T, E, I), f)

    ninf = {"f32": "0xFF800000", "bf16": "0xFF80", "f16": "0xFC00"}[f]

    def splat(name, value, shape):
        return (f"    %{name}s = stablehlo.constant dense<{value}> : tensor<{f}>\n"
                f"    %{name} = stablehlo.broadcast_in_dim %{name}s, dims = [] : (tensor<{f}>) -> {_t(shape, f)}\n")
    return f"""
module @jit_gemma4_block {{
  func.func public @main(%x: {th}, %proj: {_t((H, E), f)}, %perdim: {_t((H,), f)}, %gc: {_t((E, I, H // 2), "ui8")}, %gs: {_t((E, I, H // 32), "ui8")}, %uc: {_t((E, I, H // 2), "ui8")}, %us: {_t((E, I, H // 32), "ui8")}, %dc: {_t((E, H, I // 2), "ui8")}, %ds: {_t((E, H, I // 32), "ui8")}, %escale: {_t((E,), f)}) -> {th} {{{_tagged_mxfp4_weight("g", "%gc", "%gs", (E,), I, H, f)}{_tagged_mxfp4_weight("u", "%uc", "%us", (E,), I, H, f)}{_tagged_mxfp4_weight("d", "%dc", "%ds", (E,), H, I, f)}
    %zero = stablehlo.constant dense<0.000000e+00> : tensor<{f}>
    %ninf = stablehlo.constant dense<{ninf}> : tensor<{f}>
    %xx = stablehlo.multiply %x, %x : {th}
    %ss = stablehlo.reduce(%xx init: %zero) applies stablehlo.add across dimensions = [1] : ({th}, tensor<{f}>) -> {_t((T,), f)}
{splat("invh", f"{1.0 / H:.8e}", (T,))}{splat("eps", "1.000000e-06", (T,))}    %ms = stablehlo.multiply %ss, %invh : {_t((T,), f)}
    %mse = stablehlo.add %ms, %eps : {_t((T,), f)}
    %rs = stablehlo.rsqrt %mse : {_t((T,), f)}
    %rsb = stablehlo.broadcast_in_dim %rs, dims = [0] : ({_t((T,), f)}) -> {th}
    %n0 = stablehlo.multiply %x, %rsb : {th}
{splat("hs", f"{H ** -0.5:.8e}", (T, H))}    %n1 = stablehlo.multiply %n0, %hs : {th}
    %pdb = stablehlo.broadcast_in_dim %perdim, dims = [1] : ({_t((H,), f)}) -> {th}
    %n2 = stablehlo.multiply %n1, %pdb : {th}
    %lg = stablehlo.dot_general %n2, %proj, contracting_dims = [1] x [0] : ({th}, {_t((H, E), f)}) -> {te}
    %lmx = stablehlo.reduce(%lg init: %ninf) applies stablehlo.maximum across dimensions = [1] : ({te}, tensor<{f}>) -> {_t((T,), f)}
    %lmxb = stablehlo.broadcast_in_dim %lmx, dims = [0] : ({_t((T,), f)}) -> {te}
    %lsh = stablehlo.subtract %lg, %lmxb : {te}
    %lex = stablehlo.exponential %lsh : {te}
    %lsm = stablehlo.reduce(%lex init: %zero) applies stablehlo.add across dimensions = [1] : ({te}, tensor<{f}>) -> {_t((T,), f)}
    %lsmb = stablehlo.broadcast_in_dim %lsm, dims = [0] : ({_t((T,), f)}) -> {te}
    %probs = stablehlo.divide %lex, %lsmb : {te}
    %vals, %idx = chlo.top_k(%probs, k = {K}) : {te} -> ({tk_}, {_t((T, K), "i32")})
    %vs = stablehlo.reduce(%vals init: %zero) applies stablehlo.add across dimensions = [1] : ({tk_}, tensor<{f}>) -> {_t((T,), f)}
{splat("tiny", "1.000000e-09", (T,))}    %vsm = stablehlo.maximum %vs, %tiny : {_t((T,), f)}
    %vsb = stablehlo.broadcast_in_dim %vsm, dims = [0] : ({_t((T,), f)}) -> {tk_}
    %w = stablehlo.divide %vals, %vsb : {tk_}
    %idxb = stablehlo.broadcast_in_dim %idx, dims = [0, 1] : ({_t((T, K), "i32")}) -> {_t(tke, "i32")}
    %io = stablehlo.iota dim = 2 : {_t(tke, "i32")}
    %eq = stablehlo.compare EQ, %idxb, %io, SIGNED : ({_t(tke, "i32")}, {_t(tke, "i32")}) -> {_t(tke, "i1")}
    %hot = stablehlo.convert %eq : ({_t(tke, "i1")}) -> {_t(tke, f)}
    %wb = stablehlo.broadcast_in_dim %w, dims = [0, 1] : ({tk_}) -> {_t(tke, f)}
    %hw = stablehlo.multiply %hot, %wb : {_t(tke, f)}
    %s = stablehlo.reduce(%hw init: %zero) applies stablehlo.add across dimensions = [1] : ({_t(tke, f)}, tensor<{f}>) -> {te}
    %g0 = stablehlo.dot_general %x, %wtg, contracting_dims = [1] x [2] : ({th}, {_t((E, I, H), f)}) -> {tei}
    %g = stablehlo.transpose %g0, dims = [1, 0, 2] : ({tei}) -> {eti}
    %u0 = stablehlo.dot_general %x, %wtu, contracting_dims = [1] x [2] : ({th}, {_t((E, I, H), f)}) -> {tei}
    %u = stablehlo.transpose %u0, dims = [1, 0, 2] : ({tei}) -> {eti}
{splat("c3", "4.471500e-02", (E, T, I))}{splat("c2", "7.978846e-01", (E, T, I))}{splat("one", "1.000000e+00", (E, T, I))}{splat("half", "5.000000e-01", (E, T, I))}    %g2 = stablehlo.multiply %g, %g : {eti}
    %g3 = stablehlo.multiply %g2, %g : {eti}
    %g3c = stablehlo.multiply %g3, %c3 : {eti}
    %gin = stablehlo.add %g, %g3c : {eti}
    %gsc = stablehlo.multiply %gin, %c2 : {eti}
    %gth = stablehlo.tanh %gsc : {eti}
    %g1p = stablehlo.add %gth, %one : {eti}
    %gh = stablehlo.multiply %g, %half : {eti}
    %gelu = stablehlo.multiply %gh, %g1p : {eti}
    %act = stablehlo.multiply %gelu, %u : {eti}
    %y0 = stablehlo.dot_general %act, %wtd, batching_dims = [0] x [0], contracting_dims = [2] x [2] : ({eti}, {_t((E, H, I), f)}) -> {eth}
    %es3 = stablehlo.reshape %escale : ({_t((E,), f)}) -> {_t((E, 1, 1), f)}
    %esb = stablehlo.broadcast_in_dim %es3, dims = [0, 1, 2] : ({_t((E, 1, 1), f)}) -> {eth}
    %y = stablehlo.multiply %y0, %esb : {eth}
    %st = stablehlo.transpose %s, dims = [1, 0] : ({te}) -> {_t((E, T), f)}
    %sb = stablehlo.broadcast_in_dim %st, dims = [0, 1] : ({_t((E, T), f)}) -> {eth}
    %ys = stablehlo.multiply %y, %sb : {eth}
    %out = stablehlo.reduce(%ys init: %zero) applies stablehlo.add across dimensions = [0] : ({eth}, tensor<{f}>) -> {th}
    return %out : {th}
  }}
}}
"""


def gemma4_block_reference(x, proj, per_dim, g_ref, u_ref, d_ref, escale, k):
    """The Gemma4 block on exactly dequantized weights, in float64 numpy; the
    selection itself from the float32 probabilities the graph would compare."""
    x64, H = np.asarray(x, np.float64), x.shape[-1]
    normed = x64 / np.sqrt(np.mean(x64 * x64, -1, keepdims=True) + 1e-6) * H ** -0.5 * np.asarray(per_dim, np.float64)
    lg = normed @ np.asarray(proj, np.float64)
    ex = np.exp(lg - lg.max(-1, keepdims=True))
    probs = ex / ex.sum(-1, keepdims=True)
    order = np.argsort(-probs.astype(np.float32), axis=-1, kind="stable")[:, :k]
    vals = np.take_along_axis(probs, order, -1)
    w = vals / np.maximum(vals.sum(-1, keepdims=True), 1e-9)
    s = np.zeros_like(probs)
    np.put_along_axis(s, order, w, -1)
    g = np.einsum("th,eih->eti", x64, g_ref.astype(np.float64))
    u = np.einsum("th,eih->eti", x64, u_ref.astype(np.float64))
    gelu = 0.5 * g * (1.0 + np.tanh(0.7978846 * (g + 0.044715 * g ** 3)))
    y = np.einsum("eti,ehi->eth", gelu * u, d_ref.astype(np.float64)) * np.asarray(escale, np.float64)[:, None, None]
    return np.einsum("eth,te->th", y, s)


def moe_gemma4_decode_loop(E, T, H, I, K, steps, el="f32"):
    """Prefill plus a decode step inside a while body, as a sampler emits it
    (reference tests/test_moe.py:262-296): the Gemma4 block over [T, H], then
    `steps` times over the [1, H] row the previous step produced, starting
    from the prefill's last row.  The loop's closed-over weights arrive as
    carries returned unchanged, which is how jax lowers them.  Returns both
    results: ([T, H], [1, H])."""
    import re
    f = el

    def body_of(text):
        start = text.index("{", text.index("@main")) + 1
        return text[start:text.index("    return %out")]

    pre = body_of(moe_block_gemma4_mxfp4(E, T, H, I, K, el))
    step = body_of(moe_block_gemma4_mxfp4(E, 1, H, I, K, el))
    inputs = ["proj", "perdim", "gc", "gs", "uc", "us", "dc", "ds", "escale"]
    carried = {"x": "tok", **{n: "c" + n for n in inputs}}
    step = re.sub(r"%([A-Za-z_][A-Za-z0-9_]*)", lambda mo: "%" + carried.get(mo.group(1), mo.group(1) + "_b"), step)
    types = {"proj": _t((H, E), f), "perdim": _t((H,), f), "gc": _t((E, I, H // 2), "ui8"),
             "gs": _t((E, I, H // 32), "ui8"), "uc": _t((E, I, H // 2), "ui8"), "us": _t((E, I, H // 32), "ui8"),
             "dc": _t((E, H, I // 2), "ui8"), "ds": _t((E, H, I // 32), "ui8"), "escale": _t((E,), f)}
    th, one = _t((T, H), f), _t((1, H), f)
    params = ", ".join([f"%x: {th}"] + [f"%{n}: {types[n]}" for n in inputs])
    carries = ", ".join([f"%i = %i0", f"%tok = %last"] + [f"%c{n} = %{n}" for n in inputs])
    ctypes_ = ", ".join(["tensor<i32>", one] + [types[n] for n in inputs])
    back = ", ".join(["%ni", "%out_b"] + [f"%c{n}" for n in inputs])
    return f"""
module @jit_gemma4_generate {{
  func.func public @main({params}) -> ({th}, {one}) {{{pre}
    %last = stablehlo.slice %out [{T - 1}:{T}, 0:{H}] : ({th}) -> {one}
    %i0 = stablehlo.constant dense<0> : tensor<i32>
    %r:{2 + len(inputs)} = stablehlo.while({carries}) : {ctypes_}
     cond {{
      %lim = stablehlo.constant dense<{steps}> : tensor<i32>
      %p = stablehlo.compare LT, %i, %lim, SIGNED : (tensor<i32>, tensor<i32>) -> tensor<i1>
      stablehlo.return %p : tensor<i1>
    }} do {{{step}
      %onei = stablehlo.constant dense<1> : tensor<i32>
      %ni = stablehlo.add %i, %onei : tensor<i32>
      stablehlo.return {back} : {ctypes_}
    }}
    return %out, %r#1 : {th}, {one}
  }}
}}
"""
